"""Decisions that need no GPU: how the decode attention's keys are cut over workgroups, which kernel a product's
rows go to, and the view of a request's tokens."""

import types

import pytest

from somi_inference_amd.engine.request import Request, TokenView
from somi_inference_amd.kernels import attention as choice
from somi_inference_amd.kernels import linear as products
from somi_inference_amd.kernels import ops


@pytest.fixture
def device_of_256_units(monkeypatch):
    monkeypatch.setattr(ops, "compute_units", lambda: 256)
    longest = lambda page_size: (768 - 10) * page_size // 64 * 64        # what a page list of 768 entries holds
    monkeypatch.setattr(ops, "library", lambda: types.SimpleNamespace(somi_attention_decode_lds_split=longest))


def test_decode_splits_aim_at_two_workgroups_a_unit_and_more_for_small_heads(device_of_256_units):
    # 8 requests x 4 key/value heads at 8,192 possible keys: 16 splits give 512 workgroups
    assert choice.decode_splits(8, 4, 8192, 16, 128) == (512, 16)
    # 64 requests: two splits; from 128 on the requests alone are two a unit and nothing is split
    assert choice.decode_splits(64, 4, 8192, 16, 128) == (4096, 2)
    assert choice.decode_splits(128, 4, 8192, 16, 128) == (8192, 1)
    assert choice.decode_splits(256, 4, 8192, 16, 128) == (8192, 1)
    # heads of 64 the same, smaller ones more (a workgroup's tiles in flight hold fewer bytes)
    assert choice.decode_splits(64, 2, 8192, 16, 64) == (2048, 4)
    assert choice.decode_splits(64, 2, 8192, 16, 32) == (1024, 8)
    # a split is a multiple of 64 keys, at least 64, and the splits cover the context
    for tokens, groups, context in [(1, 4, 4096), (3, 7, 1000), (1, 1, 70), (500, 8, 33), (2, 4, 131072)]:
        length, count = choice.decode_splits(tokens, groups, context, 16, 128)
        assert length % 64 == 0 and length >= 64 and length * count >= context and count <= choice.MAX_SPLITS
        assert (count - 1) * length < context


def test_a_split_is_no_longer_than_the_page_list_in_lds_holds(device_of_256_units):
    # 16,384 possible keys in pages of 16: one split would need 1,024 pages, the list holds 768 - 10
    length, count = choice.decode_splits(256, 4, 16384, 16, 128)
    assert length == (768 - 10) * 16 // 64 * 64 and count == 2
    # pages of 64 tokens: the same list holds four times the keys
    assert choice.decode_splits(256, 4, 16384, 64, 128) == (16384, 1)
    # without a page size (the kernel that keeps no list) nothing is capped
    assert choice.decode_splits(256, 4, 16384, 0, 128) == (16384, 1)


def test_rows_of_a_product_into_the_stream_choose_their_kernel(device_of_256_units):
    # o of 65 to 128 requests (short K, few columns) runs in passes of the few-rows kernel; down (long K) does not
    assert products.residual_in_passes(96, 3584, 3584) and products.residual_in_passes(128, 3584, 3584)
    assert not products.residual_in_passes(96, 3584, 18944)
    assert not products.residual_in_passes(64, 3584, 3584) and not products.residual_in_passes(129, 3584, 3584)
    assert not products.residual_in_passes(96, 152064, 3584)
    # a kept product with a long K and few columns: passes of the split-K kernel up to 128 rows
    assert products.prefers_mid_passes(100, 3584, 18944) and not products.prefers_mid_passes(129, 3584, 18944)
    assert not products.prefers_mid_passes(100, 37888, 3584)
    # the few-rows choice between the kernel that splits K and the one that does not goes with the device's units
    assert products._mid_is_faster(32, 3584, 18944) and products._mid_is_faster(64, 37888, 3584)
    assert not products._mid_is_faster(16, 3584, 18944) and not products._mid_is_faster(64, 4608, 3584)


def test_token_view_reads_prompt_and_output_as_one_sequence_without_copying():
    request = Request("r", [5, 6, 7], 4)
    request.output_tokens.extend([8, 9])
    view = request.tokens
    assert isinstance(view, TokenView) and len(view) == 5 == request.num_tokens
    assert list(view) == [5, 6, 7, 8, 9] == request.all_tokens and view == [5, 6, 7, 8, 9]
    assert [view[i] for i in range(5)] == [5, 6, 7, 8, 9] and view[-1] == 9 and view[-5] == 5
    assert view[0:2] == [5, 6] and view[3:5] == [8, 9] and view[1:4] == [6, 7, 8] and view[2:2] == []
    assert view[:] == [5, 6, 7, 8, 9] and view[::2] == [5, 7, 9] and view[4:99] == [9]
    request.output_tokens.append(10)                      # a view, not a copy
    assert len(view) == 6 and view[5] == 10 and 10 in view and set(view) == {5, 6, 7, 8, 9, 10}
    with pytest.raises(IndexError):
        view[6]
    assert request != Request("r", [5, 6, 7], 4) and request == request      # a request is itself
