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
        _assert_draws_follow_the_plain_rule(logits, temperature, uniform, got)


def _assert_draws_follow_the_plain_rule(logits, temperature, uniform, picked):
    """A row with a temperature takes the token whose share of softmax(logits / temperature) covers the row's
    uniform number (/root/reference/somi_inference/core/sampler.py:112-113, 172-173, with the draw by inverse CDF):
    computed here in float64 by the tensor library."""
    for row in range(logits.shape[0]):
        t = float(temperature[row])
        if t == 0.0:
            continue
        cdf = torch.cumsum(torch.softmax(logits[row].double().cpu() / t, dim=-1), dim=0)
        token, u = int(picked[row]), float(uniform[row])
        low = float(cdf[token - 1]) if token > 0 else 0.0
        assert low - 1e-4 <= u <= float(cdf[token]) + 1e-4, (row, token, low, float(cdf[token]), u)


def test_sampling_without_allocation_inside_a_captured_graph():
    """After one call outside capture (which resolves the fixed array's address on the device), the entry point is
    captured into a graph on the capturing stream and replayed on new inputs, with eager work and synchronisations
    between the replays; every replay equals the entry point that takes a workspace."""
    lib = kernel_build.load()
    lib.somi_last_error.restype = ctypes.c_char_p
    torch.cuda.set_device(0)
    rows, vocab = 6, 10007
    logits, temperature, uniform = _inputs(rows, vocab, 11)
    code, first = _no_alloc(lib, logits, temperature, uniform)            # eager: resolves the address
    assert code == 0, lib.somi_last_error().decode()
    torch.cuda.synchronize()
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        code = lib.somi_sample_no_alloc(ctypes.c_void_p(logits.data_ptr()), rows, vocab,
                                        ctypes.c_void_p(temperature.data_ptr()), ctypes.c_void_p(uniform.data_ptr()),
                                        ctypes.c_void_p(out.data_ptr()), stream)
    assert code == 0, lib.somi_last_error().decode()
    for replay in range(4):
        fresh, _, fresh_uniform = _inputs(rows, vocab, 20 + replay)
        logits.copy_(fresh)
        uniform.copy_(fresh_uniform)
        want = ops.sample(logits, temperature, uniform)                   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {replay}"
        _assert_draws_follow_the_plain_rule(logits, temperature, uniform, out)


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
