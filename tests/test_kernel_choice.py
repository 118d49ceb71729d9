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


def test_launch_shapes_inside_the_library_go_with_the_devices_compute_units():
    """The few-rows split-K product and the prefill attention size their launches by workgroups per compute unit.
    The library answers for a device of any size without touching a GPU: on 256 units the figures that were
    measured there, on a device of half or 304 units the same rules scaled."""
    import ctypes
    lib = ops.library()
    strips, splits = ctypes.c_int(), ctypes.c_int()

    def mid(m, n, k, swiglu, units, workspace=1 << 40):
        assert lib.somi_linear_mid_choice(m, n, k, int(swiglu), ctypes.c_int64(workspace), units,
                                          ctypes.byref(strips), ctypes.byref(splits)) == 0
        return strips.value, splits.value

    # 7B down projection, 64 rows, 256 units: 56 column tiles of 64, 296 chunks: 448 / 56 = 8 splits of 37 chunks
    assert mid(64, 3584, 18944, False, 256) == (1, 8)
    # gate_up (37,888 columns): two strips, 296 tiles < 384: 2 splits; on 128 units 296 tiles are enough: no split
    assert mid(64, 37888, 3584, True, 256) == (2, 2)
    assert mid(64, 37888, 3584, True, 128) == (2, 1)
    # the same down projection on half the device is split half as often; without a workspace not at all
    assert mid(64, 3584, 18944, False, 128) == (1, 4)
    assert mid(64, 3584, 18944, False, 256, workspace=0) == (1, 1)
    # the logits' 152,064 columns: two strips once 128-column tiles outnumber the units (1,188 tiles of 128)
    assert mid(32, 152064, 3584, False, 256)[0] == 2 and mid(32, 152064, 3584, False, 2048)[0] == 1

    NARROW, SPLIT, WIDE, TILE, TILE_WIDE = 1, 2, 3, 4, 5
    shape = lambda entries, longest, context, nq, units, tile=0, fits=1, window=0: \
        lib.somi_attention_prefill_choice(entries, longest, context, nq, window, tile, fits, units)
    # 2,048 tokens, 28 heads, 256 units: 448 groups of 128 queries < 600: 64 queries a workgroup; 896 such
    # workgroups are not below 896, so nothing is shared; on 304 units 896 < 1,064: two wavefronts share the keys
    assert shape(1, 2048, 2048, 28, 256) == NARROW
    assert shape(1, 2048, 2048, 28, 304) == SPLIT
    assert shape(1, 2048, 2048, 28, 304, fits=0) == NARROW
    # 3,072 tokens: 672 groups >= 600: 128 queries; on 304 units the bound is 712, and 1,344 workgroups of 64
    # queries are too many to share keys
    assert shape(1, 3072, 3072, 28, 256) == WIDE and shape(1, 3072, 3072, 28, 304) == NARROW
    # 512 tokens after 3,584 cached: 112 groups, below one a unit: shared keys; with 12 such portions 1,344: wide
    assert shape(1, 512, 4096, 28, 256) == SPLIT and shape(12, 512, 4096, 28, 256) == WIDE
    # a short context (no workgroup walks 1,024 keys) keeps the plain shape
    assert shape(1, 512, 512, 28, 256) == NARROW
    # the tile kernel: 256 queries a workgroup from three groups for two units on
    assert shape(1, 2048, 2048, 28, 256, tile=1) == TILE and shape(1, 8192, 8192, 28, 256, tile=1) == TILE_WIDE
    assert shape(1, 3072, 3072, 28, 256, tile=1) == TILE and shape(1, 4096, 4096, 28, 256, tile=1) == TILE_WIDE
    assert shape(1, 4096, 4096, 28, 512, tile=1) == TILE


def test_the_many_rows_product_deals_out_units_only_where_it_is_asked_to():
    """Dealing out (tile, stage) units is there for the asking and never chosen (it measured slower than whole tiles
    at every number of rows); asked for, it takes a workgroup a compute unit, within what the workspace holds."""
    streams = lambda m, n, k, tile=0, units=256: ops.linear_big_streams(m, n, k, tile, units)
    for m in (128, 256, 512, 2048):
        assert streams(m, 4608, 3584) == 0 and streams(m, 37888, 3584) == 0 and streams(m, 3584, 18944) == 0
    asked = ops.BIG_TILE_STREAM + 256
    assert streams(2048, 4608, 3584, asked) == 256 and streams(2048, 4608, 3584, asked, units=272) == 272
    assert streams(2048, 4608, 3584, asked, units=500) == 0       # more workgroups than the workspace has slots for
    assert streams(64, 256, 64, asked) == 0                        # fewer units than workgroups
    assert streams(2048, 4608, 3584, ops.BIG_TILE_NO_STREAM + 256) == 0


def test_the_last_columns_of_a_many_rows_product_share_k_where_whole_rounds_leave_a_small_tail():
    """A product whose 256 x 128 tiles are two or more whole rounds over the compute units and a tail that would
    leave most of them idle runs the tail as a product of its own with K shared; after one round (a single round of
    256 x 256 tiles is faster), where the tail is large, or up to 128 rows, the product runs whole."""
    tail = lambda m, n, k, units=256: ops.linear_big_tail(m, n, k, units)
    # gate_up at 512 rows: 2 x 296 tiles = two rounds and 80 tiles (40 column tiles) in 3 splits
    assert tail(512, 37888, 3584) == (5120, 3)
    # one whole round and a tail: 7B q/k/v at 2,048 rows (8 x 36 tiles), gate_up at 256 rows (296 tiles)
    assert tail(2048, 4608, 3584) == (0, 1) and tail(256, 37888, 3584) == (0, 1)
    # at 2,048 rows five rounds of 256 x 256 tiles cost less than nine rounds of 256 x 128 and a tail
    assert tail(2048, 37888, 3584) == (0, 1)
    # o and down (224 tiles), up to 128 rows, and a tail of more than half of the units: whole
    assert tail(2048, 3584, 18944) == (0, 1) and tail(128, 37888, 3584) == (0, 1)
    assert tail(1024, 37888, 3584) == (0, 1)                       # 4 x 296 = 1,184 tiles: a tail of 160
    # half the device: 1 x 296 tiles are two rounds of 128 and 40 tiles in 3 splits
    assert tail(256, 37888, 3584, units=128) == (5120, 3)
