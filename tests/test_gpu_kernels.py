"""Each HIP kernel alone against a plain float32 torch reference of the same op, at sizes other than
the tiny models' (odd widths, many heads and groups, page sizes, tails)."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain import qwen2_plain as plain
from somi_inference_amd.kernels import KernelError, ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=1e-5, rtol=1e-5), "bfloat16": dict(atol=2e-2, rtol=2e-2)}


def rnd(*shape, dtype="float32", seed=0, scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=gen) * scale).to(DT[dtype]).to(DEV)


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_gathers_rows_as_float32(dtype):
    table = rnd(301, 72, dtype=dtype)
    ids = i32([0, 300, 17, 17, 5])
    out = ops.embedding(table, ids)
    assert out.dtype == torch.float32
    assert torch.equal(out, table.float()[ids.long()])
    assert torch.equal(ops.gather_rows(out, i32([4, 0])), out[[4, 0]])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [8, 200, 3584 + 24])
def test_rmsnorm_and_the_fused_residual_add(dtype, hidden):
    h = rnd(5, hidden, seed=1) + 0.5
    w = rnd(hidden, seed=2) + 1.0
    for eps in (1e-6, 0.1):
        out = ops.rmsnorm(h.clone(), w, eps, DT[dtype])
        torch.testing.assert_close(out.float(), F.rms_norm(h, (hidden,), w, eps), **TOL[dtype])
    delta = rnd(5, hidden, dtype=dtype, seed=3)
    h2 = h.clone()
    out = ops.rmsnorm(h2, w, 1e-5, DT[dtype], delta=delta)
    torch.testing.assert_close(h2, h + delta.float(), atol=1e-6, rtol=1e-6)       # the sum itself is float32
    torch.testing.assert_close(out.float(), F.rms_norm(h + delta.float(), (hidden,), w, 1e-5), **TOL[dtype])
    h3 = h.clone()
    ops.residual_add(h3, delta)
    assert torch.equal(h3, h2)
    # the reference's vector: [1,2,3,4], eps 0 -> x / sqrt(7.5) (tests/models/test_qwen2.py:18-26)
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)
    torch.testing.assert_close(ops.rmsnorm(x, torch.ones(4, device=DEV), 0.0, torch.float32), x / math.sqrt(7.5))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("m, n, k", [(1, 503, 192), (7, 64, 65), (65, 130, 17), (130, 33, 1000)])
def test_linear_plain_with_bias_and_tails(dtype, m, n, k):
    x, w, b = rnd(m, k, dtype=dtype, seed=1), rnd(n, k, dtype=dtype, seed=2, scale=0.1), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), b)
    torch.testing.assert_close(ops.linear_plain(x, w, b).float(), want, **TOL[dtype])
    torch.testing.assert_close(ops.linear_plain(x, w, None, torch.float32), F.linear(x.float(), w.float()),
                               atol=1e-4, rtol=1e-4)
    # a row's result does not depend on how many rows are in the launch
    assert torch.equal(ops.linear_plain(x[:1].contiguous(), w, b), ops.linear_plain(x, w, b)[:1])
    with pytest.raises(KernelError, match="features"):
        ops.linear_plain(x, rnd(n, k + 1, dtype=dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq, nkv, d, page", [(4, 2, 16, 16), (12, 2, 48, 8), (8, 1, 80, 4), (3, 3, 128, 32)])
def test_rope_and_cache_write(dtype, nq, nkv, d, page):
    n, pages, theta = 9, 6, 1e4
    qkv = rnd(n, (nq + 2 * nkv) * d, dtype=dtype, seed=4)
    positions = i32([0, 1, 2, 3, 40, 41, 7, 1000, 5])
    slot_list = [page * 5 + 1, page * 5 + 2, 3, 0, page * 2, page * 2 + 1, page * 4 - 1, page * 3, 2]
    if page < 4:
        pytest.skip("needs distinct slots")
    slots = i32(slot_list)
    kc = torch.zeros(pages, nkv, page, d, dtype=DT[dtype], device=DEV)
    vc = torch.zeros(pages, nkv, d, page, dtype=DT[dtype], device=DEV)      # V is transposed inside a page
    inv_freq = plain.rope_inv_freq(d, theta).to(DEV)
    before = qkv.clone()
    ops.rope_kv_store(qkv, positions, slots, inv_freq, d, nq, nkv, d, kc, vc)
    heads = before.float().view(n, nq + 2 * nkv, d).cpu()
    cos, sin = plain.rope_cos_sin(positions.cpu(), d, theta)
    want_q = plain.apply_rope(heads[:, :nq].transpose(0, 1), cos, sin).transpose(0, 1)
    want_k = plain.apply_rope(heads[:, nq:nq + nkv].transpose(0, 1), cos, sin).transpose(0, 1)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == "float32" else dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(qkv.float().view(n, -1, d)[:, :nq].cpu(), want_q, **tol)
    for t, slot in enumerate(slot_list):
        pg, off = divmod(slot, page)
        torch.testing.assert_close(kc[pg, :, off].float().cpu(), want_k[t], **tol)
        assert torch.equal(vc[pg, :, :, off].cpu(), before.view(n, -1, d)[t, nq + nkv:].cpu())
    written = torch.zeros(pages * page, dtype=torch.bool)
    written[slot_list] = True
    untouched = kc.float().permute(0, 2, 1, 3).reshape(pages * page, -1).cpu()[~written]
    assert float(untouched.abs().sum()) == 0.0, "a slot that was not addressed was written"
    # no rotation table: q unchanged, k and v stored as they are
    qkv2 = before.clone()
    ops.rope_kv_store(qkv2, positions, slots, None, 0, nq, nkv, d, kc, vc)
    assert torch.equal(qkv2, before)
    assert torch.equal(kc[slot_list[0] // page, :, slot_list[0] % page], before.view(n, -1, d)[0, nq:nq + nkv])


def dense_attention_reference(q, keys, values, positions, lens_before, window, scale):
    """q: [N, nq, D] of one request laid out after its cached tokens; keys/values: [L, nkv, D]."""
    nq, nkv = q.shape[1], keys.shape[1]
    out = torch.zeros_like(q)
    for t in range(q.shape[0]):
        p = positions[t]
        lo = max(0, p - window + 1) if window else 0
        k = keys[lo:p + 1].repeat_interleave(nq // nkv, dim=1)
        v = values[lo:p + 1].repeat_interleave(nq // nkv, dim=1)
        scores = torch.einsum("hd,lhd->hl", q[t], k) * scale
        out[t] = torch.einsum("hl,lhd->hd", torch.softmax(scores, dim=-1), v)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq, nkv, d, page, window", [
    (8, 4, 32, 4, 0),          # the reference's microbenchmark shape (benchmarks/bench_paged_attention.py:88-104)
    (12, 2, 64, 16, 0), (8, 1, 48, 8, 0), (6, 3, 128, 16, 37), (5, 5, 16, 3, 5), (14, 2, 256, 16, 0)])
def test_paged_attention_over_permuted_pages_for_portions_and_single_tokens(dtype, nq, nkv, d, page, window):
    # two requests: one brings a portion of 9 tokens after 30 cached ones, one a single token after 200
    cached, new = [30, 200], [9, 1]
    total = [c + n for c, n in zip(cached, new)]
    n_pages = sum((t + page - 1) // page for t in total) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(3)).tolist()
    tables, at = [], 0
    for t in total:
        count = (t + page - 1) // page
        tables.append(perm[at:at + count])
        at += count
    width = max(len(t) for t in tables)
    block_table = i32([t + [0] * (width - len(t)) for t in tables])
    keys = [rnd(t, nkv, d, dtype=dtype, seed=10 + i) for i, t in enumerate(total)]
    values = [rnd(t, nkv, d, dtype=dtype, seed=20 + i) for i, t in enumerate(total)]
    kc = rnd(n_pages, nkv, page, d, dtype=dtype, seed=99)      # garbage everywhere else must be inert
    vc = rnd(n_pages, nkv, d, page, dtype=dtype, seed=98)      # (reference tests/core/test_paged_attention.py:243-256)
    for r, t in enumerate(total):
        for pos in range(t):
            kc[tables[r][pos // page], :, pos % page] = keys[r][pos]
            vc[tables[r][pos // page], :, :, pos % page] = values[r][pos]
    n = sum(new)
    q = rnd(n, nq * d, dtype=dtype, seed=5, scale=2.0)
    positions = [cached[0] + i for i in range(new[0])] + [cached[1]]
    entry = [0] * new[0] + [1]
    scale = d ** -0.5
    out = ops.paged_attention_plain(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale)
    qh = q.float().view(n, nq, d).cpu()
    want = torch.cat([
        dense_attention_reference(qh[:new[0]], keys[0].float().cpu(), values[0].float().cpu(), positions[:new[0]], cached[0], window, scale),
        dense_attention_reference(qh[new[0]:], keys[1].float().cpu(), values[1].float().cpu(), positions[new[0]:], cached[1], window, scale)])
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == "float32" else dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(out.float().view(n, nq, d).cpu(), want, **tol)


def test_paged_attention_refuses_what_it_cannot_do():
    q = rnd(1, 5 * 16)
    kc = rnd(2, 2, 4, 16)
    with pytest.raises(KernelError, match="divisible"):      # reference: AssertionError on bad GQA (tests/core/test_paged_attention.py:340-350)
        ops.paged_attention_plain(q, 80, kc, rnd(2, 2, 16, 4), i32([[0]]), i32([0]), i32([0]), 5, 0, 0.25)
    big = rnd(1, 2 * 272)
    kc2 = rnd(2, 2, 4, 272)
    with pytest.raises(KernelError, match="head_dim"):
        ops.paged_attention_plain(big, 544, kc2, rnd(2, 2, 272, 4), i32([[0]]), i32([0]), i32([0]), 2, 0, 0.1)
    with pytest.raises(KernelError, match="GPU"):
        ops.silu_mul(torch.zeros(2, 4))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul(dtype):
    gu = rnd(7, 2 * 203, dtype=dtype, seed=6, scale=3.0)
    want = F.silu(gu.float()[:, :203]) * gu.float()[:, 203:]
    torch.testing.assert_close(ops.silu_mul(gu).float(), want, **TOL[dtype])
    # the reference's vector: gate = up = 10 -> silu(10) * 10 (tests/models/test_qwen2_mlp.py:22-39)
    ten = torch.full((1, 2), 10.0, device=DEV)
    assert ops.silu_mul(ten).item() == pytest.approx(10.0 / (1 + math.exp(-10.0)) * 10.0, rel=1e-6)


def test_sample_greedy_takes_the_first_maximum():
    logits = torch.tensor([[1.0, 3.0, 2.0], [5.0, 5.0, 4.0], [-1.0, -3.0, -1.0]], device=DEV)   # reference test_sampler.py:58-66
    zero = torch.zeros(3, device=DEV)
    assert ops.sample(logits, zero, zero).tolist() == [1, 0, 0]
    wide = rnd(4, 152064 // 8 + 5, seed=8)
    assert ops.sample(wide, torch.zeros(4, device=DEV), torch.zeros(4, device=DEV)).tolist() == wide.argmax(-1).tolist()


def test_sample_draws_by_inverse_cdf_of_the_softmax():
    logits = torch.tensor([[0.0, math.log(2.0), math.log(3.0), -float("inf"), math.log(2.0)]], device=DEV)
    temp = torch.ones(1, device=DEV)
    edges = torch.tensor([1, 3, 6, 6, 8]) / 8.0             # cumulative probabilities 1/8, 3/8, 6/8, 6/8, 1
    for u, want in [(0.0, 0), (0.124, 0), (0.126, 1), (0.374, 1), (0.376, 2), (0.749, 2), (0.751, 4), (0.999999, 4)]:
        got = ops.sample(logits, temp, torch.tensor([u], device=DEV)).item()
        assert got == want, f"u={u}: token {got}, expected {want} (edges {edges.tolist()})"
    # temperature sharpens: at T = 0.5 probabilities are proportional to 1, 4, 9, 0, 4 (of 18)
    half = torch.full((1,), 0.5, device=DEV)
    assert ops.sample(logits, half, torch.tensor([1.5 / 18], device=DEV)).item() == 1
    assert ops.sample(logits, half, torch.tensor([5.5 / 18], device=DEV)).item() == 2
    # a wide row: the empirical distribution of many uniform draws matches the softmax
    wide = rnd(1, 1237, seed=9, scale=2.0)
    probs = torch.softmax(wide[0].float() / 0.8, dim=-1).cpu()
    us = torch.rand(4000, generator=torch.Generator().manual_seed(1))
    rows = wide.expand(4000, -1).contiguous()
    picks = ops.sample(rows, torch.full((4000,), 0.8, device=DEV), us.to(DEV)).cpu().long()
    want = torch.searchsorted(torch.cumsum(probs.double(), 0), us.double()).clamp(max=1236)
    assert (picks == want).float().mean() > 0.995          # equal up to float32 rounding at bucket edges


def test_repetition_penalty_rule():
    row = torch.tensor([2.0, 1.5, -1.0, 0.5], device=DEV)   # reference test_sampler.py:85-93, 251-263
    ops.repetition_penalty(row, i32([0, 2]), 2.0)
    assert row.tolist() == [1.0, 1.5, -2.0, 0.5]
    with pytest.raises(KernelError, match="penalty"):
        ops.repetition_penalty(row, i32([0]), 0.0)


def test_repetition_penalty_of_several_rows_in_one_launch():
    logits = rnd(4, 777, seed=21, scale=3.0)
    histories = [[5, 5, 9, 700], [], list(range(0, 777, 3)), [776, 0]]
    penalties = [2.0, 1.7, 0.5, 1.0]                       # row 1 has no ids, row 3 a penalty of 1: both stay
    offsets, ids = [0], []
    for history in histories:
        ids += sorted(set(history))
        offsets.append(len(ids))
    work = logits.clone()
    ops.repetition_penalty_rows(work, i32(offsets), i32(ids), torch.tensor(penalties, device=DEV),
                                max(len(set(h)) for h in histories))
    for row in range(4):
        want = plain.penalize_repetition(logits[row].cpu(), histories[row], penalties[row])
        assert torch.equal(work[row].cpu(), want), f"row {row}"


def _midpoint_p(z: torch.Tensor, rank: int) -> float:
    """A top-p value halfway between the cumulative probabilities of the entries of rank ``rank`` and ``rank + 1`` of
    softmax(z), so that rounding in a cumulative sum cannot move the cut."""
    cumulative = torch.cumsum(torch.softmax(torch.sort(z.double(), descending=True).values, dim=-1), dim=-1)
    return float((cumulative[rank] + cumulative[rank + 1]) / 2)


@pytest.mark.parametrize("vocab", [5, 1237, 152064 // 8 + 5, 152064])
def test_top_k_and_top_p_masks_against_the_sorted_rule(vocab):
    """Rows of one launch with different rules: greedy (untouched), top-k, top-p, both, neither."""
    logits = rnd(6, vocab, seed=30 + vocab % 7, scale=2.0)
    temps = [0.0, 0.8, 1.3, 0.7, 1.0, 0.9]
    ks = [2, min(50, vocab - 1), -1, min(300, vocab - 1), vocab + 5, 1]
    host = logits.cpu()
    ps = [0.3, 1.0, _midpoint_p(host[2] / temps[2], min(40, vocab - 2)), 0.0, 1.0, 0.5]
    # row 3: the p sits between two entries of what top-k left
    ps[3] = _midpoint_p(plain.keep_top_k(host[3] / temps[3], ks[3]), min(17, vocab - 2))
    work = logits.clone()
    ops.sample_filter(work, torch.tensor(temps, device=DEV), i32(ks), torch.tensor(ps, device=DEV))
    got = work.cpu()
    for row in range(6):
        if temps[row] == 0.0:
            want = host[row]
        else:
            scaled = plain.keep_top_p(plain.keep_top_k(host[row] / temps[row], ks[row]), ps[row])
            want = torch.where(torch.isinf(scaled), scaled, host[row])
        assert torch.equal(got[row], want), (
            f"row {row}: kept {int((~torch.isinf(got[row])).sum())}, expected {int((~torch.isinf(want)).sum())}")
    # the masked rows go on into the draw: it lands on a kept entry
    picks = ops.sample(work, torch.tensor(temps, device=DEV), torch.full((6,), 0.999, device=DEV)).tolist()
    assert all(not math.isinf(got[row, picks[row]]) for row in range(6))


def test_top_k_and_top_p_masks_with_equal_entries():
    # reference test_sampler.py:96-106: exactly k survive also where the k-th value is shared
    row = torch.tensor([[5.0, 4.0, 4.0, 1.0]], device=DEV)
    one = torch.ones(1, device=DEV)
    work = row.clone()
    ops.sample_filter(work, one, i32([2]), one)
    assert work[0].tolist() == [5.0, 4.0, -math.inf, -math.inf]          # of equal entries the earlier ones stay
    # :108-128: softmax of 4, 3, 2, 1 is 0.64, 0.24, ...: p = 0.5 keeps the first entry only, p = 0.7 the first two
    for p, kept in [(0.5, 1), (0.7, 2), (0.9, 3), (0.99, 4)]:
        work = torch.tensor([[4.0, 3.0, 2.0, 1.0]], device=DEV)
        ops.sample_filter(work, one, i32([-1]), torch.tensor([p], device=DEV))
        assert int((~torch.isinf(work)).sum()) == kept, p
    # many shared values (logits in steps of 0.5, negative ones and both zeros among them): the number kept and the
    # values kept are those of the sorted rule, whichever of the equal entries a sort would have put first
    gen = torch.Generator().manual_seed(5)
    coarse = (torch.randn(3, 6000, generator=gen) * 2.0 / 0.5).round() * 0.5
    coarse[0, 17] = -0.0
    temps = torch.tensor([1.0, 0.5, 2.0], device=DEV)
    for ks, ps in [([40, 700, 5999], [1.0, 1.0, 1.0]), ([-1, -1, -1], [0.35, 0.8, 0.97]), ([100, 2000, 30], [0.6, 0.9, 0.2])]:
        work = coarse.to(DEV)
        ops.sample_filter(work, temps, i32(ks), torch.tensor(ps, device=DEV))
        for r in range(3):
            scaled = coarse[r] / temps[r].item()
            want = plain.keep_top_p(plain.keep_top_k(scaled, ks[r]), ps[r])
            kept_got = torch.sort(scaled[~torch.isinf(work[r].cpu())]).values
            kept_want = torch.sort(want[~torch.isinf(want)]).values
            assert kept_got.shape == kept_want.shape and torch.equal(kept_got, kept_want), (r, ks, ps)


@pytest.mark.parametrize("m, n, k", [(1, 503, 192), (7, 64, 72), (16, 130, 200), (17, 33, 1000), (48, 3584 + 16, 3584),
                                     (64, 70, 18944), (8, 152064 // 16 + 3, 512), (2, 32768 + 16, 128), (20, 65536 + 48, 64)])
def test_linear_skinny_mfma_against_float32(m, n, k):
    x, w, b = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.05), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), b)
    scale = float(want.abs().max())
    got32 = ops.linear_skinny(x, w, b, torch.float32)
    torch.testing.assert_close(got32, want, atol=2e-5 * scale * math.sqrt(k), rtol=1e-4)     # float32 sums of exact products
    got = ops.linear_skinny(x, w, b)
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, atol=scale * 2 ** -8, rtol=2 ** -7)         # one rounding to bfloat16
    torch.testing.assert_close(ops.linear_skinny(x, w, None, torch.float32), F.linear(x.float(), w.float()),
                               atol=2e-5 * scale * math.sqrt(k), rtol=1e-4)
    # the same rows give the same bits whatever else is in the batch, as long as the number of 16-row
    # tiles (which sets how K is split over wavefronts) is the same
    first = (m - 1) // 16 * 16
    assert torch.equal(ops.linear_skinny(x[first:first + 1].contiguous().repeat(first + 1, 1), w, b, torch.float32)[-1:],
                       got32[first:first + 1])


def test_linear_skinny_refuses_what_it_cannot_do():
    with pytest.raises(KernelError, match="64 rows"):
        ops.linear_skinny(rnd(65, 64, dtype="bfloat16"), rnd(8, 64, dtype="bfloat16"))
    with pytest.raises(KernelError, match="multiple of 8"):
        ops.linear_skinny(rnd(2, 12, dtype="bfloat16"), rnd(8, 12, dtype="bfloat16"))
    with pytest.raises(KernelError, match="bfloat16"):
        ops.linear_skinny(rnd(2, 16), rnd(8, 16))


@pytest.mark.parametrize("nq, nkv, d, page, window, splits", [
    (8, 4, 32, 4, 0, 1), (12, 2, 64, 16, 0, 3), (8, 1, 48, 8, 0, 2), (6, 3, 128, 16, 37, 4), (28, 4, 128, 16, 0, 5),
    (40, 2, 16, 8, 0, 1), (14, 2, 256, 16, 0, 2), (5, 5, 80, 4, 5, 3), (7, 1, 112, 32, 100, 2)])
def test_attention_decode_mfma_against_dense_softmax(nq, nkv, d, page, window, splits):
    """The reference's own check of its decode kernel: dense softmax over the tokens gathered through a
    permuted table (tests/core/test_paged_attention.py:292-338), here for portions and single tokens,
    several splits of the keys, 1 to 20 query heads per key/value head and head sizes in steps of 16."""
    cached, new = [30, 200, 0], [9, 1, 3]
    total = [c + n for c, n in zip(cached, new)]
    n_pages = sum((t + page - 1) // page for t in total) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(3)).tolist()
    tables, at = [], 0
    for t in total:
        count = (t + page - 1) // page
        tables.append(perm[at:at + count])
        at += count
    width = max(len(t) for t in tables)
    block_table = i32([t + [0] * (width - len(t)) for t in tables])
    keys = [rnd(t, nkv, d, dtype="bfloat16", seed=10 + i) for i, t in enumerate(total)]
    values = [rnd(t, nkv, d, dtype="bfloat16", seed=20 + i) for i, t in enumerate(total)]
    kc = rnd(n_pages, nkv, page, d, dtype="bfloat16", seed=99)
    vc = rnd(n_pages, nkv, d, page, dtype="bfloat16", seed=98)
    for r, t in enumerate(total):
        for pos in range(t):
            kc[tables[r][pos // page], :, pos % page] = keys[r][pos]
            vc[tables[r][pos // page], :, :, pos % page] = values[r][pos]
    n = sum(new)
    q = rnd(n, nq * d, dtype="bfloat16", seed=5, scale=2.0)
    positions, entry = [], []
    for e, (c, k) in enumerate(zip(cached, new)):
        positions += [c + i for i in range(k)]
        entry += [e] * k
    scale = d ** -0.5
    split_len = ((max(total) + splits - 1) // splits + 15) // 16 * 16
    num_splits = (max(total) + split_len - 1) // split_len
    out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale,
                         split_len, num_splits, out)
    qh = q.float().view(n, nq, d).cpu()
    want, at = [], 0
    for e, k in enumerate(new):
        want.append(dense_attention_reference(qh[at:at + k], keys[e].float().cpu(), values[e].float().cpu(),
                                              positions[at:at + k], cached[e], window, scale))
        at += k
    torch.testing.assert_close(out.float().view(n, nq, d).cpu(), torch.cat(want), atol=2e-2, rtol=2e-2)
    plain_out = ops.paged_attention_plain(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale)
    torch.testing.assert_close(out.float(), plain_out.float(), atol=2e-2, rtol=2e-2)
    # a list of tokens: only those rows are written
    out2 = torch.zeros_like(out)
    ops.attention_decode(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale,
                         split_len, num_splits, out2, token_list=i32([9, 2]))
    assert torch.equal(out2[[9, 2]], out[[9, 2]]) and float(out2[[0, 1, 3, 12]].abs().sum()) == 0.0


def test_attention_decode_refuses_what_it_cannot_do():
    q, kc, vc = rnd(1, 2 * 24, dtype="bfloat16"), rnd(2, 2, 4, 24, dtype="bfloat16"), rnd(2, 2, 24, 4, dtype="bfloat16")
    out = torch.zeros(1, 48, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError, match="multiple of 16"):
        ops.attention_decode(q, 48, kc, vc, i32([[0]]), i32([0]), i32([0]), 2, 0, 0.2, 16, 1, out)
    q, kc, vc = rnd(1, 2 * 16, dtype="bfloat16"), rnd(2, 2, 6, 16, dtype="bfloat16"), rnd(2, 2, 16, 6, dtype="bfloat16")
    out = torch.zeros(1, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError, match="multiple of 4"):
        ops.attention_decode(q, 32, kc, vc, i32([[0]]), i32([0]), i32([0]), 2, 0, 0.2, 16, 1, out)


def tile_kernel_takes(d, page):
    """The sizes the 32 x 32 tile kernel of the prefill attention takes (launch shapes 4 and 5)."""
    return d in (64, 128) and page >= 8 and page & (page - 1) == 0


@pytest.mark.parametrize("nq, nkv, d, page, window", [
    (8, 4, 32, 4, 0), (12, 2, 64, 16, 0), (8, 1, 48, 8, 0), (6, 3, 128, 16, 37), (28, 4, 128, 16, 0),
    (4, 2, 16, 8, 0), (14, 2, 256, 16, 0), (5, 5, 80, 4, 5), (7, 1, 112, 32, 100), (3, 1, 208, 16, 0),
    (14, 2, 64, 8, 20), (8, 2, 128, 32, 0), (5, 1, 128, 8, 150), (6, 6, 64, 64, 0)])
@pytest.mark.parametrize("shape", [0, 1, 2, 3, 4, 5], ids=["auto", "narrow", "split", "wide", "tile", "tile-wide"])
def test_attention_prefill_mfma_against_dense_softmax(nq, nkv, d, page, window, shape):
    """Portions of several requests in one launch: a long one that starts at position 0, one that continues
    after 150 cached tokens, a portion of two tokens, single tokens after 77 and after 0 cached ones.  Each
    launch shape of the two kernels that stage tiles through LDS is asked for in turn; the tile kernel refuses the
    sizes it does not take."""
    if shape >= 4 and not tile_kernel_takes(d, page):
        q, kc, vc = rnd(4, nq * d, dtype="bfloat16"), rnd(2, nkv, page, d, dtype="bfloat16"), rnd(2, nkv, d, page, dtype="bfloat16")
        with pytest.raises(KernelError, match="tile kernel does not take"):
            ops.attention_prefill(q, nq * d, kc, vc, i32([[1]]), i32([0, 4]), i32([0]), 4, nq, window, d ** -0.5,
                                  torch.zeros_like(q), shape=shape)
        return
    cached, new = [0, 150, 30, 77, 0], [203, 130, 2, 1, 1]
    total = [c + n for c, n in zip(cached, new)]
    n_pages = sum((t + page - 1) // page for t in total) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(4)).tolist()
    tables, at = [], 0
    for t in total:
        count = (t + page - 1) // page
        tables.append(perm[at:at + count])
        at += count
    width = max(len(t) for t in tables)
    block_table = i32([t + [0] * (width - len(t)) for t in tables])
    keys = [rnd(t, nkv, d, dtype="bfloat16", seed=10 + i) for i, t in enumerate(total)]
    values = [rnd(t, nkv, d, dtype="bfloat16", seed=20 + i) for i, t in enumerate(total)]
    kc = rnd(n_pages, nkv, page, d, dtype="bfloat16", seed=99)
    vc = rnd(n_pages, nkv, d, page, dtype="bfloat16", seed=98)
    for r, t in enumerate(total):
        for pos in range(t):
            kc[tables[r][pos // page], :, pos % page] = keys[r][pos]
            vc[tables[r][pos // page], :, :, pos % page] = values[r][pos]
    n = sum(new)
    q = rnd(n, nq * d, dtype="bfloat16", seed=5, scale=2.0)
    positions, entry, starts = [], [], [0]
    for e, (c, k) in enumerate(zip(cached, new)):
        positions += [c + i for i in range(k)]
        entry += [e] * k
        starts.append(starts[-1] + k)
    scale = d ** -0.5
    out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q, nq * d, kc, vc, block_table, i32(starts), i32(cached), max(new), nq, window, scale, out,
                          shape=shape)
    qh = q.float().view(n, nq, d).cpu()
    want, at = [], 0
    for e, k in enumerate(new):
        want.append(dense_attention_reference(qh[at:at + k], keys[e].float().cpu(), values[e].float().cpu(),
                                              positions[at:at + k], cached[e], window, scale))
        at += k
    torch.testing.assert_close(out.float().view(n, nq, d).cpu(), torch.cat(want), atol=2e-2, rtol=2e-2)
    plain_out = ops.paged_attention_plain(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale)
    torch.testing.assert_close(out.float(), plain_out.float(), atol=2e-2, rtol=2e-2)
    # a mixed step: the long portions by this kernel, the short ones (two tokens, single tokens) token by token by
    # the decode kernel with the keys of a request split over workgroups; one output tensor
    mixed = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q, nq * d, kc, vc, block_table, i32(starts), i32(cached), max(new), nq, window, scale, mixed,
                          shape=shape, entry_len=i32([k if k > 8 else 0 for k in new]))
    short = [t for e, k in enumerate(new) if k <= 8 for t in range(starts[e], starts[e] + k)]
    assert bool(torch.isnan(mixed[short].float()).all()) and not bool(torch.isnan(mixed[:starts[2]].float()).any())
    ops.attention_decode(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale, 64, 3, mixed,
                         token_list=i32(short))
    torch.testing.assert_close(mixed.float(), plain_out.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("m, inter, k", [(1, 48, 72), (8, 18944 // 8, 512), (17, 160, 200), (40, 4096 + 32, 64), (64, 32, 3584)])
def test_linear_skinny_with_the_gate_fused_in(m, inter, k):
    x = rnd(m, k, dtype="bfloat16", seed=1)
    gate, up = rnd(inter, k, dtype="bfloat16", seed=2, scale=0.1), rnd(inter, k, dtype="bfloat16", seed=3, scale=0.1)
    merged = torch.stack([gate.view(-1, 16, k), up.view(-1, 16, k)], dim=1).reshape(-1, k).contiguous()
    want = F.silu(x.float() @ gate.float().t()) * (x.float() @ up.float().t())
    got = ops.linear_skinny_swiglu(x, merged)
    scale = float(want.abs().max())
    torch.testing.assert_close(got.float(), want, atol=scale * 2 ** -7, rtol=2 ** -6)
    # the unfused way over the same interleaved matrix
    unfused = ops.silu_mul(ops.linear_skinny(x, merged), block=16)
    torch.testing.assert_close(unfused.float(), want, atol=scale * 2 ** -6, rtol=2 ** -5)
    with pytest.raises(KernelError, match="does not fit"):
        ops.linear_skinny_swiglu(x, merged[:-16].contiguous())


@pytest.mark.parametrize("m, n, k", [(1, 70, 72), (17, 130, 200), (40, 200, 2048), (64, 70, 18944), (33, 3584 + 16, 1000),
                                     (48, 16384 + 80, 256), (64, 640, 8192)])
def test_linear_mid_shared_rows_and_split_k_against_float32(m, n, k):
    """The product for some tens of rows: x shared inside a workgroup, K split over workgroups with the partial
    sums added by a second kernel.  Shapes with one and several splits, a K that ends inside a chunk, columns
    that do not fill a tile."""
    x, w, b = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.05), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), b)
    scale = float(want.abs().max())
    got32 = ops.linear_mid(x, w, b, torch.float32)
    torch.testing.assert_close(got32, want, atol=2e-5 * scale * math.sqrt(k), rtol=1e-4)     # float32 sums of exact products
    got = ops.linear_mid(x, w, b)
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, atol=scale * 2 ** -8, rtol=2 ** -7)         # one rounding to bfloat16
    torch.testing.assert_close(ops.linear_mid(x, w, None, torch.float32), F.linear(x.float(), w.float()),
                               atol=2e-5 * scale * math.sqrt(k), rtol=1e-4)
    assert torch.equal(ops.linear_mid(x, w, b, torch.float32), got32)                         # a fixed order of additions
    with pytest.raises(KernelError, match="64 rows"):
        ops.linear_mid(rnd(65, k, dtype="bfloat16"), w)


@pytest.mark.parametrize("m, inter, k", [(8, 48, 72), (33, 160, 1536), (64, 4096 + 32, 64), (50, 96, 8192)])
def test_linear_mid_with_the_gate_fused_in(m, inter, k):
    x = rnd(m, k, dtype="bfloat16", seed=1)
    gate, up = rnd(inter, k, dtype="bfloat16", seed=2, scale=0.1), rnd(inter, k, dtype="bfloat16", seed=3, scale=0.1)
    merged = torch.stack([gate.view(-1, 16, k), up.view(-1, 16, k)], dim=1).reshape(-1, k).contiguous()
    want = F.silu(x.float() @ gate.float().t()) * (x.float() @ up.float().t())
    got = ops.linear_mid(x, merged, swiglu=True)
    scale = float(want.abs().max())
    torch.testing.assert_close(got.float(), want, atol=scale * 2 ** -7, rtol=2 ** -6)
    torch.testing.assert_close(got.float(), ops.linear_skinny_swiglu(x, merged).float(), atol=scale * 2 ** -7, rtol=2 ** -6)


@pytest.mark.parametrize("mid", [False, True], ids=["skinny", "mid"])
@pytest.mark.parametrize("m, hidden, n_out, inter", [(1, 64, 72, 48), (8, 3584, 4608, 256), (16, 200, 33, 160), (5, 1000, 503, 96),
                                                     (17, 1000, 503, 96), (40, 200, 33, 160), (33, 520, 1056, 4112),
                                                     (64, 3584, 4608, 1024), (48, 1536, 256, 18944)])
def test_products_fused_with_the_residual_add_and_the_norm(m, hidden, n_out, inter, mid):
    """h += x.W1^T (+ b) with the rows' sums of squares and the next norm's weighted rows as by-products, then
    rmsnorm(h).W2^T as the product of those rows scaled per row: against float32 formulas and against the
    unfused kernels (norm, then product)."""
    eps = 1e-5
    x = rnd(m, inter, dtype="bfloat16", seed=1)
    w1, b1 = rnd(hidden, inter, dtype="bfloat16", seed=2, scale=0.1), rnd(hidden, seed=3)
    h = rnd(m, hidden, seed=4, scale=2.0)
    norm_w = 1.0 + rnd(hidden, seed=5, scale=0.1)
    want_h = h + F.linear(x.float(), w1.float(), b1)
    got_h = h.clone()
    stats, weighted = ops.linear_residual(x, w1, b1, got_h, norm_w, mid=mid)
    torch.testing.assert_close(got_h, want_h, atol=2e-5 * float(want_h.abs().max()) * math.sqrt(inter), rtol=1e-5)
    width = 16 * ((m + 15) // 16)
    assert stats.shape[1] == width and float(stats[:, m:].abs().max() if m < width else 0.0) == 0.0
    torch.testing.assert_close(stats.sum(dim=0)[:m], got_h.pow(2).sum(dim=1), rtol=1e-5, atol=1e-6)
    assert torch.equal(weighted, (norm_w * got_h).to(torch.bfloat16))
    no_bias = h.clone()
    assert ops.linear_residual(x, w1, None, no_bias, mid=mid)[1] is None
    torch.testing.assert_close(no_bias, h + F.linear(x.float(), w1.float()), atol=2e-5 * float(want_h.abs().max()) * math.sqrt(inter), rtol=1e-5)

    w2, b2 = rnd(n_out, hidden, dtype="bfloat16", seed=6, scale=0.05), rnd(n_out, seed=7)
    normed = ops.rmsnorm(got_h, norm_w, eps, torch.bfloat16)                      # the unfused way
    unfused = ops.linear_skinny(normed, w2, b2)
    fused = ops.linear_scaled(weighted, eps, stats, w2, b2, mid=mid)
    want = F.linear(plain_rms(got_h, norm_w, eps), w2.float(), b2)               # float32 throughout
    scale = float(want.abs().max())
    torch.testing.assert_close(fused.float(), want, atol=scale * 2 ** -6, rtol=2 ** -6)
    torch.testing.assert_close(fused.float(), unfused.float(), atol=scale * 2 ** -6, rtol=2 ** -6)
    gate, up = rnd(inter, hidden, dtype="bfloat16", seed=8, scale=0.1), rnd(inter, hidden, dtype="bfloat16", seed=9, scale=0.1)
    merged = torch.stack([gate.view(-1, 16, hidden), up.view(-1, 16, hidden)], dim=1).reshape(-1, hidden).contiguous()
    gated = ops.linear_scaled(weighted, eps, stats, merged, swiglu=True, mid=mid)
    exact = plain_rms(got_h, norm_w, eps)
    want_gated = F.silu(exact @ gate.float().t()) * (exact @ up.float().t())
    torch.testing.assert_close(gated.float(), want_gated, atol=float(want_gated.abs().max()) * 2 ** -5, rtol=2 ** -5)
    with pytest.raises(KernelError, match="64 rows"):
        ops.linear_residual(rnd(65, inter, dtype="bfloat16"), w1, None, rnd(65, hidden), mid=mid)


@pytest.mark.parametrize("m", [65, 70, 96, 128])
@pytest.mark.parametrize("n, k", [(192, 8200), (136, 264)])
def test_product_into_the_stream_of_65_to_128_rows(m, n, k):
    """The chooser's passes of 64 rows (with a long K: of the kernel that splits K, the short last pass too), their
    statistics side by side, and the product that reads them."""
    from somi_inference_amd.kernels import linear as chooser
    x = rnd(m, k, dtype="bfloat16", seed=1)
    w1, b1 = rnd(n, k, dtype="bfloat16", seed=2, scale=0.1), rnd(n, seed=3)
    h = rnd(m, n, seed=4, scale=2.0)
    norm_w = 1.0 + rnd(n, seed=5, scale=0.1)
    want_h = h + F.linear(x.float(), w1.float(), b1)
    got_h = h.clone()
    stats, weighted = chooser.linear_residual(x, w1, b1, got_h, norm_w)
    torch.testing.assert_close(got_h, want_h, atol=2e-5 * float(want_h.abs().max()) * math.sqrt(k), rtol=1e-5)
    assert stats.shape[1] == 16 * ((m + 15) // 16)
    torch.testing.assert_close(stats.sum(dim=0)[:m], got_h.pow(2).sum(dim=1), rtol=1e-5, atol=1e-6)
    assert torch.equal(weighted, (norm_w * got_h).to(torch.bfloat16))
    w2 = rnd(80, n, dtype="bfloat16", seed=6, scale=0.05)
    got = chooser.linear_scaled(weighted, 1e-5, stats, w2)
    want = F.linear(plain_rms(got_h, norm_w, 1e-5), w2.float())
    torch.testing.assert_close(got.float(), want, atol=float(want.abs().max()) * 2 ** -6, rtol=2 ** -6)


@pytest.mark.parametrize("scaled", [True, False], ids=["normed", "as-is"])
@pytest.mark.parametrize("m, nq, nkv, d, hidden, page", [(1, 4, 2, 32, 64, 16), (9, 12, 2, 64, 200, 8), (16, 3, 3, 128, 520, 4),
                                                         (24, 6, 2, 96, 264, 8), (37, 5, 1, 96, 1000, 16), (64, 28, 4, 128, 3584, 16)])
def test_qkv_product_with_the_rotation_and_the_cache_store(m, nq, nkv, d, hidden, page, scaled):
    """q/k/v projection, rotary encoding and cache write in one kernel: against the float32 formulas (norm as a
    row scale, product, rotation) and against the three separate kernels."""
    eps, theta, pages = 1e-5, 1e4, 12
    n_out = (nq + 2 * nkv) * d
    w, b = rnd(n_out, hidden, dtype="bfloat16", seed=2, scale=0.05), rnd(n_out, seed=3)
    positions = i32([(7 * t * t + 3) % 5000 for t in range(m)])
    slot_list = [(11 * t + 5) % (pages * page) for t in range(m)]            # distinct: 11 is coprime to the pool
    assert len(set(slot_list)) == m
    slot_list[m // 2] = -1 if m > 2 else slot_list[m // 2]                     # a token without a slot is not stored
    slots = i32(slot_list)
    inv_freq = plain.rope_inv_freq(d, theta).to(DEV)
    if scaled:                                   # rows still to be normed, as a product into the stream leaves them
        h = rnd(m, hidden, seed=4, scale=2.0)
        norm_w = 1.0 + rnd(hidden, seed=5, scale=0.1)
        x = (norm_w * h).to(torch.bfloat16)
        stats = torch.zeros(3, 16 * ((m + 15) // 16), device=DEV)
        stats[1, :m] = h.pow(2).sum(dim=1)
        exact_x = x.float() * torch.rsqrt(h.pow(2).mean(dim=1, keepdim=True) + eps)
    else:
        x, stats = rnd(m, hidden, dtype="bfloat16", seed=4), None
        exact_x = x.float()
    kc = torch.zeros(pages, nkv, page, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(pages, nkv, d, page, dtype=torch.bfloat16, device=DEV)
    q = ops.linear_rope_store(x, eps, stats, w, b, positions, slots, inv_freq, nq, nkv, d, kc, vc)
    heads = F.linear(exact_x, w.float(), b).view(m, nq + 2 * nkv, d).cpu()
    cos, sin = plain.rope_cos_sin(positions.cpu(), d, theta)
    want_q = plain.apply_rope(heads[:, :nq].transpose(0, 1), cos, sin).transpose(0, 1)
    want_k = plain.apply_rope(heads[:, nq:nq + nkv].transpose(0, 1), cos, sin).transpose(0, 1)
    scale = float(heads.abs().max())
    tol = dict(atol=scale * 2 ** -7, rtol=2 ** -7)
    torch.testing.assert_close(q.float().view(m, nq, d).cpu(), want_q, **tol)
    for t, slot in enumerate(slot_list):
        if slot < 0:
            continue
        pg, off = divmod(slot, page)
        torch.testing.assert_close(kc[pg, :, off].float().cpu(), want_k[t], **tol)
        torch.testing.assert_close(vc[pg, :, :, off].float().cpu(), heads[t, nq + nkv:], **tol)
    written = torch.zeros(pages * page, dtype=torch.bool)
    written[[slot for slot in slot_list if slot >= 0]] = True
    for cache in (kc.permute(0, 2, 1, 3), vc.permute(0, 3, 1, 2)):
        untouched = cache.float().reshape(pages * page, -1).cpu()[~written]
        assert float(untouched.abs().sum()) == 0.0, "a slot that was not addressed was written"
    # the separate kernels: product (with the norm as a row scale), then rotation and store
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    qkv = ops.linear_scaled(x, eps, stats, w, b) if scaled else ops.linear_skinny(x, w, b)
    ops.rope_kv_store(qkv, positions, slots, inv_freq, d, nq, nkv, d, kc2, vc2)
    # the same sums in the same order, rounded at the same places: the same bits
    assert torch.equal(q, qkv[:, :nq * d]) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    if scaled:
        # the rows' sums as some columns of the table of more rows, q into a given tensor: the same bits again
        table = torch.full((3, 64 + stats.shape[1] + 16), 1e9, device=DEV)
        table[:, 64:64 + stats.shape[1]] = stats
        kc3, vc3, q3 = torch.zeros_like(kc), torch.zeros_like(vc), torch.full_like(q, 3.0)
        assert ops.linear_rope_store(x, eps, table[:, 64:64 + stats.shape[1]], w, b, positions, slots, inv_freq, nq, nkv, d,
                                     kc3, vc3, out=q3) is q3
        assert torch.equal(q, q3) and torch.equal(kc, kc3) and torch.equal(vc, vc3)
        with pytest.raises(KernelError, match="consecutive floats"):
            ops.linear_rope_store(x, eps, table[:, 1:2 * stats.shape[1]:2][:, :stats.shape[1]], w, b, positions, slots,
                                  inv_freq, nq, nkv, d, kc3, vc3)
    with pytest.raises(KernelError, match="multiple of 32"):
        ops.linear_rope_store(x, eps, stats, rnd(4 * 48, hidden, dtype="bfloat16"), None, positions, slots,
                              plain.rope_inv_freq(48, theta).to(DEV), 2, 1, 48,
                              torch.zeros(2, 1, page, 48, dtype=torch.bfloat16, device=DEV),
                              torch.zeros(2, 1, 48, page, dtype=torch.bfloat16, device=DEV))


def plain_rms(h, w, eps):
    return w * h * torch.rsqrt(h.pow(2).mean(dim=-1, keepdim=True) + eps)


# ------------------------------------------------------------------------------ the many-rows product
BIG_SHAPES = [(65, 130, 64), (128, 256, 192), (300, 520, 200), (512, 96, 72), (2048, 264, 1032), (257, 384, 8)]


def _interleave16(gate, up):
    b, h = 16, gate.shape[1]
    return torch.stack([gate.view(-1, b, h), up.view(-1, b, h)], dim=1).reshape(-1, h).contiguous()


@pytest.mark.parametrize("tile", [0, 1, 128, 256])
@pytest.mark.parametrize("m,n,k", BIG_SHAPES)
def test_many_rows_product_plain_with_bias_and_row_scale(m, n, k, tile):
    """x . w^T (+ bias) against F.linear in float32, with tails in M, N and K (K = 200 and 72 end inside a stage,
    K = 8 is one piece), for every tile (1: the 128-row tile that up to 128 rows take by themselves); then the same with the rows scaled as an RMS norm would."""
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.3), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), bias)
    got = ops.linear_big(x, w, bias, tile=tile)
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, atol=0.02 * float(want.abs().max()), rtol=2e-2)
    plain = ops.linear_big(x, w, tile=tile)
    torch.testing.assert_close(plain.float(), F.linear(x.float(), w.float()), atol=0.02 * float(want.abs().max()), rtol=2e-2)
    # row statistics in 3 partial sums, wider than M as the producers make them
    eps = 1e-5
    width = 16 * ((m + 15) // 16)
    stats = torch.zeros(3, width, device=DEV)
    stats[:, :m] = torch.rand(3, m, device=DEV) * k
    scale = torch.rsqrt(stats[:, :m].sum(0) / k + eps)
    scaled = ops.linear_big(x, w, bias, eps=eps, stats=stats, tile=tile)
    want_scaled = scale[:, None] * F.linear(x.float(), w.float()) + bias
    torch.testing.assert_close(scaled.float(), want_scaled, atol=0.02 * float(want_scaled.abs().max()), rtol=2e-2)


def test_many_rows_product_reads_strided_rows_and_refuses_what_it_cannot_take():
    wide = rnd(300, 256 + 64, dtype="bfloat16", seed=4)
    x = wide[:, :256]                                # a view: rows 320 elements apart
    w = rnd(200, 256, dtype="bfloat16", seed=5, scale=0.2)
    torch.testing.assert_close(ops.linear_big(x, w).float(), F.linear(x.float(), w.float()), atol=0.1, rtol=2e-2)
    with pytest.raises(KernelError, match="multiples of 8"):
        ops.linear_big(rnd(70, 36, dtype="bfloat16"), rnd(8, 36, dtype="bfloat16"))
    with pytest.raises(KernelError, match="features"):
        ops.linear_big(rnd(70, 64, dtype="bfloat16"), rnd(8, 32, dtype="bfloat16"))
    with pytest.raises(KernelError, match="bfloat16"):
        ops.linear_big(rnd(70, 64), rnd(8, 64))
    with pytest.raises(KernelError, match="tile code"):
        ops.linear_big(rnd(70, 64, dtype="bfloat16"), rnd(8, 64, dtype="bfloat16"), tile=64)


@pytest.mark.parametrize("tile", [0, 1, 128, 256])
@pytest.mark.parametrize("m,inter,k", [(65, 16, 64), (100, 528, 136), (130, 272, 200), (512, 1040, 192), (2048, 48, 72)])
def test_many_rows_product_with_the_gate_in_its_end(m, inter, k, tile):
    x = rnd(m, k, dtype="bfloat16", seed=6)
    gate, up = rnd(inter, k, dtype="bfloat16", seed=7, scale=0.2), rnd(inter, k, dtype="bfloat16", seed=8, scale=0.2)
    want = F.silu(x.float() @ gate.float().t()) * (x.float() @ up.float().t())
    got = ops.linear_big(x, _interleave16(gate, up), swiglu=True, tile=tile)
    assert got.shape == (m, inter)
    torch.testing.assert_close(got.float(), want, atol=0.02 * float(want.abs().max()), rtol=2e-2)
    eps, width = 1e-6, 16 * ((m + 15) // 16)
    stats = torch.zeros(2, width, device=DEV)
    stats[:, :m] = torch.rand(2, m, device=DEV) * k * 4
    s = torch.rsqrt(stats[:, :m].sum(0) / k + eps)[:, None]
    want = F.silu(s * (x.float() @ gate.float().t())) * (s * (x.float() @ up.float().t()))
    got = ops.linear_big(x, _interleave16(gate, up), swiglu=True, eps=eps, stats=stats, tile=tile)
    torch.testing.assert_close(got.float(), want, atol=0.02 * float(want.abs().max()) + 1e-3, rtol=2e-2)


@pytest.mark.parametrize("m,n,k", [(300, 2 * 17920 + 96, 1032), (129, 2 * 33000, 1032), (1000, 18016, 1032)])
def test_many_rows_product_whose_last_columns_share_k(m, n, k):
    """More 256 x 128 tiles than compute units, with a tail that is small: the whole rounds run as they are and the
    last columns as a product of their own with K shared (a row stride of the output that is not its width, the
    weight and bias from an offset).  Plain with bias and row scale and gated, against float32 and against the same
    product on whole tiles."""
    columns, splits = ops.linear_big_tail(m, n, k)
    if ops.compute_units() == 256:
        assert columns > 0 and splits > 1
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.3), rnd(n, seed=3)
    eps, width = 1e-5, 16 * ((m + 15) // 16)
    stats = torch.zeros(3, width, device=DEV)
    stats[:, :m] = torch.rand(3, m, device=DEV) * k
    scale = torch.rsqrt(stats[:, :m].sum(0) / k + eps)
    want = scale[:, None] * F.linear(x.float(), w.float()) + bias
    got = ops.linear_big(x, w, bias, eps=eps, stats=stats)
    whole = ops.linear_big(x, w, bias, eps=eps, stats=stats, tile=128)
    tol = dict(atol=0.02 * float(want.abs().max()), rtol=2e-2)
    torch.testing.assert_close(got.float(), want, **tol)
    assert torch.equal(got[:, :n - columns], whole[:, :n - columns])          # the whole rounds are the same launch
    torch.testing.assert_close(got.float(), whole.float(), atol=float(want.abs().max()) * 2 ** -7, rtol=2 ** -7)
    inter = n // 32 * 16
    gate, up = w[:inter], rnd(inter, k, dtype="bfloat16", seed=8, scale=0.3)
    mixed = _interleave16(gate, up)
    assert ops.linear_big_tail(m, 2 * inter, k) == (columns - (n - 2 * inter), splits) or columns == 0
    s = scale[:, None]
    want = F.silu(s * (x.float() @ gate.float().t())) * (s * (x.float() @ up.float().t()))
    got = ops.linear_big(x, mixed, swiglu=True, eps=eps, stats=stats)
    whole = ops.linear_big(x, mixed, swiglu=True, eps=eps, stats=stats, tile=128)
    torch.testing.assert_close(got.float(), want, atol=0.02 * float(want.abs().max()) + 1e-3, rtol=2e-2)
    torch.testing.assert_close(got.float(), whole.float(), atol=float(want.abs().max()) * 2 ** -6, rtol=2 ** -6)


@pytest.mark.parametrize("tile", [0, 1, 128, 256])
@pytest.mark.parametrize("m,n,k", [(65, 132, 64), (128, 600, 264), (300, 520, 200), (1024, 72, 1032), (257, 256, 136)])
def test_many_rows_product_into_the_residual_stream(m, n, k, tile):
    """h += x . w^T + bias in float32, with the next norm's weighted rows and the rows' sums of squares; feeding
    those into the scaled product gives the product of the normed rows."""
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=9), rnd(n, k, dtype="bfloat16", seed=10, scale=0.2), rnd(n, seed=11)
    h0 = rnd(m, n, seed=12)
    norm_w = rnd(n, seed=13).abs() + 0.5
    want_h = h0 + F.linear(x.float(), w.float(), bias)
    h = h0.clone()
    stats, weighted = ops.linear_big_residual(x, w, bias, h, norm_w, tile=tile)
    torch.testing.assert_close(h, want_h, atol=2e-4 * float(want_h.abs().max()) + 1e-4, rtol=1e-4)
    torch.testing.assert_close(weighted.float(), norm_w * want_h, atol=0.01 * float((norm_w * want_h).abs().max()), rtol=1e-2)
    torch.testing.assert_close(stats[:, :m].sum(0), want_h.pow(2).sum(1), rtol=1e-4, atol=1e-3)
    plain_h = h0.clone()
    none_stats, none_weighted = ops.linear_big_residual(x, w, None, plain_h, tile=tile)
    assert none_weighted is None
    torch.testing.assert_close(plain_h, h0 + F.linear(x.float(), w.float()), atol=2e-4 * float(want_h.abs().max()) + 1e-4, rtol=1e-4)
    # the next product, of the normed rows: norm(h) . w2^T
    eps = 1e-5
    w2 = rnd(96, n, dtype="bfloat16", seed=14, scale=0.2)
    if n % 8 == 0:
        got = ops.linear_big(weighted, w2, eps=eps, stats=stats)
        normed = norm_w * want_h * torch.rsqrt(want_h.pow(2).mean(1, keepdim=True) + eps)
        want = normed @ w2.float().t()
        torch.testing.assert_close(got.float(), want, atol=0.02 * float(want.abs().max()), rtol=2e-2)


@pytest.mark.parametrize("tile", [1, 0, 128], ids=["128-row", "chosen", "256x128"])
@pytest.mark.parametrize("m,n,k", [(100, 520, 2056), (65, 130, 1024), (300, 96, 1032), (260, 300, 2056), (513, 200, 1536)])
def test_many_rows_product_plain_with_k_split_over_workgroups(m, n, k, tile):
    """The plain form where its tiles are few and K is long (q/k/v of some hundred rows): the workgroups of a tile
    share its K, and a second kernel scales the rows, adds the bias and rounds.  Against float32 formulas and the
    unsplit kernel, with and without the rows' scales."""
    assert ops.linear_big_splits(m, n, k, tile=tile) > 1
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.3), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), bias)
    tol = dict(atol=0.02 * float(want.abs().max()), rtol=2e-2)
    got = ops.linear_big(x, w, bias, tile=tile)
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, **tol)
    whole = ops.linear_big(x, w, bias, tile=tile, split_k=False)
    torch.testing.assert_close(got.float(), whole.float(), atol=float(want.abs().max()) * 2 ** -7, rtol=2 ** -7)
    torch.testing.assert_close(ops.linear_big(x, w, tile=tile).float(), F.linear(x.float(), w.float()), **tol)
    eps, width = 1e-5, 16 * ((m + 15) // 16)
    stats = torch.zeros(2, width, device=DEV)
    stats[:, :m] = torch.rand(2, m, device=DEV) * k * 4
    s = torch.rsqrt(stats[:, :m].sum(0) / k + eps)[:, None]
    scaled = ops.linear_big(x, w, bias, eps=eps, stats=stats, tile=tile)
    want_scaled = s * (x.float() @ w.float().t()) + bias
    torch.testing.assert_close(scaled.float(), want_scaled, atol=0.02 * float(want_scaled.abs().max()), rtol=2e-2)


@pytest.mark.parametrize("tile", [0, 1, 128, 256])
@pytest.mark.parametrize("m,n,k", [(65, 130, 64), (128, 1000, 264), (300, 521, 200), (257, 72, 1032)])
def test_many_rows_product_in_float32(m, n, k, tile):
    """x . w^T (+ bias) written as float32 (logits of many rows): against F.linear, closer than a bfloat16 result could
    be; and through the chooser, which takes it for more than 64 rows."""
    from somi_inference_amd.kernels import linear as chooser
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.3), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), bias)
    tol = dict(atol=2e-5 * float(want.abs().max()) * math.sqrt(k), rtol=1e-5)
    out = torch.full((m, n), 7.0, device=DEV)                    # what was there is not added to
    got = ops.linear_big_f32(x, w, bias, tile=tile, out=out)
    assert got is out and got.dtype == torch.float32
    torch.testing.assert_close(got, want, **tol)
    torch.testing.assert_close(ops.linear_big_f32(x, w, tile=tile), F.linear(x.float(), w.float()), **tol)
    if tile == 0:
        chosen = chooser.linear(x, w, bias, out_dtype=torch.float32)
        assert chosen.dtype == torch.float32 and torch.equal(chosen, got)


@pytest.mark.parametrize("tile", [1, 0, 128], ids=["128-row", "chosen", "256x128"])
@pytest.mark.parametrize("m,n,k", [(100, 520, 2056), (128, 264, 4096), (65, 130, 1024), (7, 72, 3000), (300, 96, 1032),
                                   (260, 300, 2056), (513, 200, 1536)])
def test_many_rows_product_into_the_stream_with_k_split_over_workgroups(m, n, k, tile):
    """Few tiles and a long K: the 128-row tile and the 256 x 128 tile split K over workgroups, and a second kernel
    adds the splits' sums into the stream and leaves the weighted rows and the sums of squares as the unsplit kernel
    does (K that ends inside a stage, N that is no multiple of 4 or of the tile, rows that do not fill a tile,
    several row tiles)."""
    assert ops.linear_big_splits(m, n, k, tile=tile) > 1
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=9), rnd(n, k, dtype="bfloat16", seed=10, scale=0.2), rnd(n, seed=11)
    h0 = rnd(m, n, seed=12)
    norm_w = rnd(n, seed=13).abs() + 0.5
    want_h = h0 + F.linear(x.float(), w.float(), bias)
    tol = dict(atol=2e-4 * float(want_h.abs().max()) + 1e-4, rtol=1e-4)
    h = h0.clone()
    stats, weighted = ops.linear_big_residual(x, w, bias, h, norm_w, tile=tile)
    torch.testing.assert_close(h, want_h, **tol)
    assert torch.equal(weighted, (norm_w * h).to(torch.bfloat16))
    torch.testing.assert_close(stats[:, :m].sum(0), h.pow(2).sum(1), rtol=1e-4, atol=1e-3)
    whole = h0.clone()
    whole_stats, whole_weighted = ops.linear_big_residual(x, w, bias, whole, norm_w, tile=tile, split_k=False)
    assert whole_stats.shape == stats.shape
    torch.testing.assert_close(h, whole, **tol)
    torch.testing.assert_close(stats[:, :m], whole_stats[:, :m], rtol=1e-3, atol=1e-3)
    again = h0.clone()                                   # the workspace is used again: the same bits
    ops.linear_big_residual(x, w, bias, again, norm_w, tile=tile)
    assert torch.equal(again, h)
    no_bias = h0.clone()
    assert ops.linear_big_residual(x, w, None, no_bias, tile=tile)[1] is None
    torch.testing.assert_close(no_bias, h0 + F.linear(x.float(), w.float()), **tol)


@pytest.mark.parametrize("scaled", [True, False], ids=["normed", "as-is"])
@pytest.mark.parametrize("m, nq, nkv, d, hidden, page", [(65, 4, 2, 32, 1032, 16), (100, 12, 2, 64, 2056, 8),
                                                         (128, 28, 4, 128, 3584, 16), (300, 6, 2, 96, 2056, 8),
                                                         (513, 5, 1, 64, 1536, 32)])
def test_qkv_product_of_many_rows_rotates_and_stores_where_it_adds_its_splits(m, nq, nkv, d, hidden, page, scaled):
    """The q/k/v product of some hundred rows shares K among workgroups; the kernel that adds their sums scales the
    rows, adds the bias, rotates q and k and stores k and v in their pages.  Against the float32 formulas and
    against the same product followed by the rotation kernel (the same sums rounded at the same places)."""
    eps, theta = 1e-5, 1e4
    pages = (m + page - 1) // page + 3
    n_out = (nq + 2 * nkv) * d
    assert ops.linear_big_splits(m, n_out, hidden) > 1
    w, b = rnd(n_out, hidden, dtype="bfloat16", seed=2, scale=0.05), rnd(n_out, seed=3)
    positions = i32([(7 * t * t + 3) % 5000 for t in range(m)])
    order = torch.randperm(pages * page, generator=torch.Generator().manual_seed(5)).tolist()[:m]
    order[m // 2] = -1                                                        # a token without a slot is not stored
    slots = i32(order)
    inv_freq = plain.rope_inv_freq(d, theta).to(DEV)
    if scaled:
        h = rnd(m, hidden, seed=4, scale=2.0)
        norm_w = 1.0 + rnd(hidden, seed=5, scale=0.1)
        x = (norm_w * h).to(torch.bfloat16)
        stats = torch.zeros(3, 16 * ((m + 15) // 16), device=DEV)
        stats[1, :m] = h.pow(2).sum(dim=1)
        exact_x = x.float() * torch.rsqrt(h.pow(2).mean(dim=1, keepdim=True) + eps)
    else:
        x, stats = rnd(m, hidden, dtype="bfloat16", seed=4), None
        exact_x = x.float()
    kc = torch.zeros(pages, nkv, page, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(pages, nkv, d, page, dtype=torch.bfloat16, device=DEV)
    q = ops.linear_big_rope_store(x, eps, stats, w, b, positions, slots, inv_freq, nq, nkv, d, kc, vc)
    heads = F.linear(exact_x, w.float(), b).view(m, nq + 2 * nkv, d).cpu()
    cos, sin = plain.rope_cos_sin(positions.cpu(), d, theta)
    want_q = plain.apply_rope(heads[:, :nq].transpose(0, 1), cos, sin).transpose(0, 1)
    want_k = plain.apply_rope(heads[:, nq:nq + nkv].transpose(0, 1), cos, sin).transpose(0, 1)
    tol = dict(atol=float(heads.abs().max()) * 2 ** -7, rtol=2 ** -7)
    torch.testing.assert_close(q.float().view(m, nq, d).cpu(), want_q, **tol)
    stored = [t for t, slot in enumerate(order) if slot >= 0]
    at = torch.tensor([order[t] for t in stored])
    torch.testing.assert_close(kc[at // page, :, at % page].float().cpu(), want_k[stored], **tol)
    torch.testing.assert_close(vc[at // page, :, :, at % page].float().cpu(), heads[stored, nq + nkv:], **tol)
    written = torch.zeros(pages * page, dtype=torch.bool)
    written[at] = True
    for cache in (kc.permute(0, 2, 1, 3), vc.permute(0, 3, 1, 2)):
        assert float(cache.float().reshape(pages * page, -1).cpu()[~written].abs().sum()) == 0.0, \
            "a slot that was not addressed was written"
    # the separate kernels: the same product with its sums added by the plain kernel, then the rotation and the store
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    qkv = ops.linear_big(x, w, b, eps=eps, stats=stats) if scaled else ops.linear_big(x, w, b)
    ops.rope_kv_store(qkv, positions, slots, inv_freq, d, nq, nkv, d, kc2, vc2)
    assert torch.equal(q, qkv[:, :nq * d]) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    with pytest.raises(KernelError, match="does not share K"):
        big = rnd(2048, hidden, dtype="bfloat16", seed=6)
        ops.linear_big_rope_store(big, eps, None, rnd(32 * 128 * 3, hidden, dtype="bfloat16"), None, i32([0] * 2048),
                                  i32([-1] * 2048), plain.rope_inv_freq(128, theta).to(DEV), 32, 32, 128,
                                  torch.zeros(1, 32, 16, 128, dtype=torch.bfloat16, device=DEV),
                                  torch.zeros(1, 32, 128, 16, dtype=torch.bfloat16, device=DEV))


STREAM = ops.BIG_TILE_STREAM
STREAMED_TILES = [STREAM + 1, STREAM + 128, STREAM + 256]
STREAMED_IDS = ["128-row", "256x128", "256x256"]
# (tile, stage) units dealt out to 256 workgroups: between one and a few stages each, so that a tile's K is walked by
# up to a dozen workgroups (300 x 1100), by two or three (700 x 520), with tails in M, N and K (K = 200 ends in a stage)
STREAMED_SHAPES = [(300, 1100, 2056), (100, 2072, 2056), (700, 520, 4104), (2048, 264, 1032), (1500, 3000, 200)]


@pytest.mark.parametrize("tile", STREAMED_TILES, ids=STREAMED_IDS)
@pytest.mark.parametrize("m,n,k", STREAMED_SHAPES)
def test_many_rows_product_with_its_units_dealt_out_plain_and_float32(m, n, k, tile):
    """The streamed form of the many-rows product: workgroups walk equal ranges of (tile, stage) units, the segments
    that do not cover a tile's K leave their sums in slots, and a second kernel ends the tiles that were shared.
    Plain (bias, row scales, bfloat16) and float32 results against F.linear and against the same tile unstreamed."""
    if ops.linear_big_streams(m, n, k, tile=tile) == 0:
        pytest.skip("too few units for this tile")
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=1), rnd(n, k, dtype="bfloat16", seed=2, scale=0.3), rnd(n, seed=3)
    want = F.linear(x.float(), w.float(), bias)
    tol = dict(atol=0.02 * float(want.abs().max()), rtol=2e-2)
    got = ops.linear_big(x, w, bias, tile=tile)
    torch.testing.assert_close(got.float(), want, **tol)
    whole = ops.linear_big(x, w, bias, tile=tile - STREAM + ops.BIG_TILE_NO_STREAM, split_k=False)
    torch.testing.assert_close(got.float(), whole.float(), atol=float(want.abs().max()) * 2 ** -7, rtol=2 ** -7)
    assert torch.equal(ops.linear_big(x, w, bias, tile=tile), got)              # the slots are used again: the same bits
    eps, width = 1e-5, 16 * ((m + 15) // 16)
    stats = torch.zeros(2, width, device=DEV)
    stats[:, :m] = torch.rand(2, m, device=DEV) * k * 4
    s = torch.rsqrt(stats[:, :m].sum(0) / k + eps)[:, None]
    scaled = ops.linear_big(x, w, None, eps=eps, stats=stats, tile=tile)
    want_scaled = s * (x.float() @ w.float().t())
    torch.testing.assert_close(scaled.float(), want_scaled, atol=0.02 * float(want_scaled.abs().max()), rtol=2e-2)
    out = torch.full((m, n), 7.0, device=DEV)
    f32 = ops.linear_big_f32(x, w, bias, tile=tile, out=out)
    torch.testing.assert_close(f32, want, atol=2e-5 * float(want.abs().max()) * math.sqrt(k), rtol=1e-5)


@pytest.mark.parametrize("tile", STREAMED_TILES, ids=STREAMED_IDS)
@pytest.mark.parametrize("m,inter,k", [(700, 272, 4104), (1500, 1488, 200), (100, 1040, 2056), (2048, 144, 1032)])
def test_many_rows_product_with_its_units_dealt_out_and_the_gate_in_its_end(m, inter, k, tile):
    if ops.linear_big_streams(m, 2 * inter, k, tile=tile) == 0:
        pytest.skip("too few units for this tile")
    x = rnd(m, k, dtype="bfloat16", seed=6)
    gate, up = rnd(inter, k, dtype="bfloat16", seed=7, scale=0.2), rnd(inter, k, dtype="bfloat16", seed=8, scale=0.2)
    eps, width = 1e-6, 16 * ((m + 15) // 16)
    stats = torch.zeros(2, width, device=DEV)
    stats[:, :m] = torch.rand(2, m, device=DEV) * k * 4
    s = torch.rsqrt(stats[:, :m].sum(0) / k + eps)[:, None]
    want = F.silu(s * (x.float() @ gate.float().t())) * (s * (x.float() @ up.float().t()))
    got = ops.linear_big(x, _interleave16(gate, up), swiglu=True, eps=eps, stats=stats, tile=tile)
    assert got.shape == (m, inter)
    torch.testing.assert_close(got.float(), want, atol=0.02 * float(want.abs().max()) + 1e-3, rtol=2e-2)
    whole = ops.linear_big(x, _interleave16(gate, up), swiglu=True, eps=eps, stats=stats,
                           tile=tile - STREAM + ops.BIG_TILE_NO_STREAM)
    torch.testing.assert_close(got.float(), whole.float(), atol=float(want.abs().max()) * 2 ** -7 + 1e-3, rtol=2 ** -7)


@pytest.mark.parametrize("tile", STREAMED_TILES, ids=STREAMED_IDS)
@pytest.mark.parametrize("m,n,k", STREAMED_SHAPES)
def test_many_rows_product_with_its_units_dealt_out_into_the_residual_stream(m, n, k, tile):
    if ops.linear_big_streams(m, n, k, tile=tile) == 0:
        pytest.skip("too few units for this tile")
    x, w, bias = rnd(m, k, dtype="bfloat16", seed=9), rnd(n, k, dtype="bfloat16", seed=10, scale=0.2), rnd(n, seed=11)
    h0 = rnd(m, n, seed=12)
    norm_w = rnd(n, seed=13).abs() + 0.5
    want_h = h0 + F.linear(x.float(), w.float(), bias)
    tol = dict(atol=2e-4 * float(want_h.abs().max()) + 1e-4, rtol=1e-4)
    h = h0.clone()
    stats, weighted = ops.linear_big_residual(x, w, bias, h, norm_w, tile=tile)
    torch.testing.assert_close(h, want_h, **tol)
    assert torch.equal(weighted, (norm_w * h).to(torch.bfloat16))
    torch.testing.assert_close(stats[:, :m].sum(0), h.pow(2).sum(1), rtol=1e-4, atol=1e-3)
    whole = h0.clone()
    whole_stats, _ = ops.linear_big_residual(x, w, bias, whole, norm_w, tile=tile - STREAM + ops.BIG_TILE_NO_STREAM,
                                             split_k=False)
    assert whole_stats.shape == stats.shape
    torch.testing.assert_close(h, whole, **tol)
    torch.testing.assert_close(stats[:, :m], whole_stats[:, :m], rtol=1e-3, atol=1e-3)
    again = h0.clone()
    ops.linear_big_residual(x, w, bias, again, norm_w, tile=tile)
    assert torch.equal(again, h)


@pytest.mark.parametrize("nq, nkv, d, page, window", [(8, 2, 128, 16, 0), (14, 2, 64, 8, 700), (4, 4, 128, 64, 1500)])
@pytest.mark.parametrize("shape", [0, 4, 5], ids=["auto", "tile", "tile-wide"])
def test_attention_prefill_tile_kernel_over_long_contexts(nq, nkv, d, page, window, shape):
    """Many steps of the tile kernel: a prompt of 1,100 tokens from position 0, 300 tokens after 2,000 cached ones
    (a block table of 144 to 288 pages), a portion that ends inside its first tile, and one whose length is no
    multiple of anything; with and without a window that the long requests outgrow.  Against the plain kernel."""
    cached, new = [0, 2000, 5, 31], [1100, 300, 20, 333]
    total = [c + n for c, n in zip(cached, new)]
    n_pages = sum((t + page - 1) // page for t in total) + 2
    perm = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(8)).add(1).tolist()
    tables, at = [], 0
    for t in total:
        count = (t + page - 1) // page
        tables.append(perm[at:at + count])
        at += count
    width = max(len(t) for t in tables) + 1
    block_table = i32([t + [0] * (width - len(t)) for t in tables])
    kc = torch.full((n_pages, nkv, page, d), float("nan"), dtype=torch.bfloat16, device=DEV)      # what is no key of a request is NaN
    vc = torch.full((n_pages, nkv, d, page), float("nan"), dtype=torch.bfloat16, device=DEV)
    for r, t in enumerate(total):
        keys, values = rnd(t, nkv, d, dtype="bfloat16", seed=50 + r), rnd(t, nkv, d, dtype="bfloat16", seed=60 + r)
        pos = torch.arange(t, device=DEV)
        pages = torch.tensor(tables[r], device=DEV)[pos // page]
        kc[pages, :, pos % page] = keys
        vc[pages, :, :, pos % page] = values
    n = sum(new)
    q = rnd(n, nq * d, dtype="bfloat16", seed=9, scale=1.5)
    positions, entry, starts = [], [], [0]
    for e, (c, k) in enumerate(zip(cached, new)):
        positions += [c + i for i in range(k)]
        entry += [e] * k
        starts.append(starts[-1] + k)
    scale = d ** -0.5
    want = ops.paged_attention_plain(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale)
    assert bool(torch.isfinite(want.float()).all())
    out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q, nq * d, kc, vc, block_table, i32(starts), i32(cached), max(new), nq, window, scale, out,
                          max_context=max(total), shape=shape)
    assert bool(torch.isfinite(out.float()).all())
    torch.testing.assert_close(out.float(), want.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("shape", [1, 3, 4, 5, "decode"], ids=["narrow", "wide", "tile", "tile-wide", "decode"])
def test_attention_scores_that_are_large_products_of_a_few_channels(d, shape):
    """Queries and keys whose products sit in three channels of size nine: scores spread over +-100, so the softmax
    sees every bit of them.  The scale belongs on the float32 scores (/root/reference/somi_inference/models/qwen2.py:
    179, core/flash_attention_triton.py:113, 159): a kernel that rounds scale * q to bfloat16 before the product is
    off by 6e-2 here, one that scales the float32 product by 1e-2 (the output's own rounding), against the dense
    float32 softmax of the same bfloat16 inputs."""
    n, nq, nkv, page = 300, 4, 1, 16
    gen = torch.Generator().manual_seed(1)
    q = torch.randn(n, nq, d, generator=gen) * 0.3
    k = torch.randn(n, nkv, d, generator=gen) * 0.3
    big = [3, d // 2 + 6, d - 27]
    q[:, :, big] = torch.randn(n, nq, 3, generator=gen) * 9.0
    k[:, :, big] = torch.randn(n, nkv, 3, generator=gen) * 9.0
    v = torch.randn(n, nkv, d, generator=gen)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    scale = d ** -0.5
    want = dense_attention_reference(q.float(), k.float(), v.float(), list(range(n)), 0, 0, scale)
    assert float((torch.einsum("ihd,jhd->hij", q.float(), k.float().expand(n, nq, d)) * scale).abs().max()) > 60.0
    pages = (n + page - 1) // page
    table = torch.randperm(pages, generator=gen).tolist()
    kc = torch.zeros(pages, nkv, page, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(pages, nkv, d, page, dtype=torch.bfloat16, device=DEV)
    pos = torch.arange(n, device=DEV)
    where = torch.tensor(table, device=DEV)[pos // page]
    kc[where, :, pos % page] = k.to(DEV)
    vc[where, :, :, pos % page] = v.to(DEV)
    flat = q.reshape(n, nq * d).contiguous().to(DEV)
    out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    if shape == "decode":
        ops.attention_decode(flat, nq * d, kc, vc, i32([table]), i32([0] * n), i32(list(range(n))), nq, 0, scale, 64, 5, out)
    else:
        ops.attention_prefill(flat, nq * d, kc, vc, i32([table]), i32([0, n]), i32([0]), n, nq, 0, scale, out, shape=shape)
    error = (out.float().view(n, nq, d).cpu() - want).abs()
    assert float(error.max()) < 2e-2, f"max error {float(error.max()):.3e}"


@pytest.mark.parametrize("width, first", [(10_000, 150_000), (13_000, 200_000), (25_000, 390_000)])
def test_attention_prefill_under_very_wide_block_tables(width, first):
    """Contexts of hundreds of thousands of tokens: block tables of 10,000 pages (the tile kernel with a long list
    of pages in LDS), of 13,000 (beyond what it holds beside its tiles: the 16 x 16 kernel with the list in dynamic
    LDS) and of 25,000 (beyond that too: the kernel that reads the table from memory).  A portion of 130 tokens at
    position `first` beside one of 70 from position 0; the logical pages share a pool of 500 physical ones, which
    the plain kernel reads through the same table.  Queries are enlarged so that a few of the keys carry the sum."""
    nq, nkv, d, page = 4, 2, 128, 16
    cached, new = [first, 0], [130, 70]
    pool = 500
    columns = torch.arange(width)
    block_table = torch.stack([1 + (columns * 7 + r) % pool for r in range(2)]).to(torch.int32).to(DEV)
    kc = rnd(pool + 1, nkv, page, d, dtype="bfloat16", seed=71)
    vc = rnd(pool + 1, nkv, d, page, dtype="bfloat16", seed=72)
    n = sum(new)
    q = rnd(n, nq * d, dtype="bfloat16", seed=73, scale=3.0)
    positions, entry, starts = [], [], [0]
    for e, (c, k) in enumerate(zip(cached, new)):
        positions += [c + i for i in range(k)]
        entry += [e] * k
        starts.append(starts[-1] + k)
    assert (max(positions) // page) < width
    scale = d ** -0.5
    want = ops.paged_attention_plain(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, 0, scale)
    assert float(want.float().abs().max()) > 0.5, "the sums are flat: a wrong key would not show"
    out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q, nq * d, kc, vc, block_table, i32(starts), i32(cached), max(new), nq, 0, scale, out,
                          max_context=first + 130)
    torch.testing.assert_close(out.float(), want.float(), atol=3e-2, rtol=3e-2)
    # single tokens at the far end, with the keys split over workgroups
    last = [starts[1] - 1, n - 1]
    dec = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, 0, scale, 2048, (first + 130 + 2047) // 2048,
                         dec, token_list=i32(last))
    torch.testing.assert_close(dec[last].float(), want[last].float(), atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("nq, nkv, d, page, window", [(8, 2, 64, 16, 0), (6, 3, 128, 16, 21), (4, 1, 32, 8, 0), (14, 2, 256, 16, 0),
                                                     (5, 5, 80, 4, 9), (7, 1, 128, 8, 40), (4, 2, 64, 32, 0)])
def test_attention_ignores_whatever_lies_beyond_a_requests_keys(nq, nkv, d, page, window):
    """Pages are handed out again without being cleared, and pages a window has passed read as page 0.  Everything
    in the cache that is not a visible key of the request is NaN here (the tail of its last page, every other
    page, the pages below the window): a masked key has the weight 0, but 0 x NaN is NaN, so the kernels must not
    let such a value reach a product.  Decode (with the keys split) and prefill (every launch shape), MFMA and
    plain kernels."""
    cached, new = [37, 150, 0, 77], [1, 1, 70, 12]
    total = [c + n for c, n in zip(cached, new)]
    n_pages = sum((t + page - 1) // page for t in total) + 2
    perm = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(6)).add(1).tolist()     # page 0 stays poisoned
    tables, at = [], 0
    for t in total:
        count = (t + page - 1) // page
        tables.append(perm[at:at + count])
        at += count
    kc = torch.full((n_pages, nkv, page, d), float("nan"), dtype=torch.bfloat16, device=DEV)
    vc = torch.full((n_pages, nkv, d, page), float("nan"), dtype=torch.bfloat16, device=DEV)
    keys = [rnd(t, nkv, d, dtype="bfloat16", seed=30 + i) for i, t in enumerate(total)]
    values = [rnd(t, nkv, d, dtype="bfloat16", seed=40 + i) for i, t in enumerate(total)]
    for r, t in enumerate(total):
        first_kept = 0
        if window:
            # a page wholly below the window of the request's first new token has been given back: page 0
            first_kept = max(0, cached[r] - window + 1) // page
            tables[r] = [0] * first_kept + tables[r][first_kept:]
        for pos in range(first_kept * page, t):
            kc[tables[r][pos // page], :, pos % page] = keys[r][pos]
            vc[tables[r][pos // page], :, :, pos % page] = values[r][pos]
    width = max(len(t) for t in tables)
    block_table = i32([t + [0] * (width - len(t)) for t in tables])
    n = sum(new)
    q = rnd(n, nq * d, dtype="bfloat16", seed=7, scale=2.0)
    positions, entry, starts = [], [], [0]
    for e, (c, k) in enumerate(zip(cached, new)):
        positions += [c + i for i in range(k)]
        entry += [e] * k
        starts.append(starts[-1] + k)
    scale = d ** -0.5
    qh = q.float().view(n, nq, d).cpu()
    want, at = [], 0
    for e, k in enumerate(new):
        want.append(dense_attention_reference(qh[at:at + k], keys[e].float().cpu(), values[e].float().cpu(),
                                              positions[at:at + k], cached[e], window, scale))
        at += k
    want = torch.cat(want).view(n, nq * d)
    plain_out = ops.paged_attention_plain(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale)
    assert bool(torch.isfinite(plain_out.float()).all()), "the plain kernel let a value from outside the visible keys through"
    torch.testing.assert_close(plain_out.float().cpu(), want, atol=2e-2, rtol=2e-2)
    for shape in (0, 1, 2, 3) + ((4, 5) if tile_kernel_takes(d, page) else ()):
        out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_prefill(q, nq * d, kc, vc, block_table, i32(starts), i32(cached), max(new), nq, window, scale, out,
                              shape=shape)
        assert bool(torch.isfinite(out.float()).all()), f"prefill shape {shape}: not finite"
        torch.testing.assert_close(out.float().cpu(), want, atol=2e-2, rtol=2e-2)
    for split_len, splits in ((64, 4), (256, 1), (16, 15)):
        out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_decode(q, nq * d, kc, vc, block_table, i32(entry), i32(positions), nq, window, scale, split_len,
                             splits, out)
        assert bool(torch.isfinite(out.float()).all()), f"decode splits of {split_len}: not finite"
        torch.testing.assert_close(out.float().cpu(), want, atol=2e-2, rtol=2e-2)
