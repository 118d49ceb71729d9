"""The sampling entry point that allocates nothing, called through ctypes as a caller outside Python's tensor
library would call it, against the entry point that takes a workspace: two calls in a row on one GPU, the second
with a smaller input (the fixed workspace then still holds the first call's partial results), and a size beyond
the fixed workspace, which must be refused."""

import ctypes

import pytest
import torch

from somi_inference_amd.csrc import build as kernel_build
from somi_inference_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(rows, vocab, seed):
    gen = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=gen) * 3.0).to(DEV)
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * (r % 4) for r in range(rows)], device=DEV)
    uniform = torch.rand(rows, generator=gen).to(DEV)
    return logits, temperature, uniform


def _no_alloc(lib, logits, temperature, uniform):
    rows, vocab = logits.shape
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    code = lib.somi_sample_no_alloc(ctypes.c_void_p(logits.data_ptr()), rows, vocab,
                                    ctypes.c_void_p(temperature.data_ptr()), ctypes.c_void_p(uniform.data_ptr()),
                                    ctypes.c_void_p(out.data_ptr()), stream)
    return code, out


def test_sampling_without_allocation_equals_sampling_with_a_workspace():
    lib = kernel_build.load()
    lib.somi_last_error.restype = ctypes.c_char_p
    torch.cuda.set_device(0)
    capacity = lib.somi_sample_no_alloc_capacity()
    assert capacity == ops.library().somi_sample_no_alloc_capacity() > 0
    # the second call is smaller in rows and vocabulary: it must not pick up what the first left behind
    for rows, vocab, seed in ((48, 152064, 1), (5, 4099, 2)):
        assert lib.somi_sample_workspace_floats(rows, vocab) <= capacity
        logits, temperature, uniform = _inputs(rows, vocab, seed)
        want = ops.sample(logits, temperature, uniform)
        code, got = _no_alloc(lib, logits, temperature, uniform)
        assert code == 0, lib.somi_last_error().decode()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rows, vocab)
        greedy = temperature == 0
        assert torch.equal(got[greedy].long(), logits[greedy].argmax(dim=-1))
        assert int(got.min()) >= 0 and int(got.max()) < vocab


def test_sampling_without_allocation_refuses_what_its_workspace_cannot_hold():
    lib = kernel_build.load()
    lib.somi_last_error.restype = ctypes.c_char_p
    capacity = lib.somi_sample_no_alloc_capacity()
    rows, vocab = 1024, 262144
    assert lib.somi_sample_workspace_floats(rows, vocab) > capacity
    # refused on the host before anything is launched: the pointers are never followed
    dummy = torch.zeros(4, device=DEV)
    out = torch.zeros(4, dtype=torch.int32, device=DEV)
    code = lib.somi_sample_no_alloc(ctypes.c_void_p(dummy.data_ptr()), rows, vocab, ctypes.c_void_p(dummy.data_ptr()),
                                    ctypes.c_void_p(dummy.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                                    ctypes.c_void_p(0))
    assert code != 0
    message = lib.somi_last_error().decode()
    assert "workspace" in message and str(capacity) in message
