"""Pins the plain implementation by what fixes it beside the reference's text: vectors held by the
reference's own tests, special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake (wrong sign or pairing, norm in the wrong place) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain import qwen2_plain as P


# ------------------------------------------------------------------------------ RMSNorm
def test_rmsnorm_vector_of_reference_tests():
    # /root/reference/tests/models/test_qwen2.py:18-36: [1,2,3,4], eps 0, weight 1 -> x / sqrt(7.5); weight 2 doubles
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    out = P.rms_norm(x, torch.ones(4), 0.0)
    torch.testing.assert_close(out, x / math.sqrt(7.5))
    torch.testing.assert_close(P.rms_norm(x, torch.full((4,), 2.0), 0.0), 2 * x / math.sqrt(7.5))


def test_rmsnorm_is_library_rms_norm_and_not_layernorm():
    x = torch.randn(5, 24) + 3.0          # a mean far from zero separates it from LayerNorm
    w = torch.randn(24)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5))
    assert not torch.allclose(P.rms_norm(x, w, 1e-5), F.layer_norm(x, (24,), w, None, 1e-5), atol=1e-2)


def test_rmsnorm_scale_invariance_at_eps_zero():
    x = torch.randn(3, 16)
    torch.testing.assert_close(P.rms_norm(7.0 * x, torch.ones(16), 0.0), P.rms_norm(x, torch.ones(16), 0.0))


# ------------------------------------------------------------------------------ RoPE
def test_rotate_half_vector_of_reference_tests():
    # /root/reference/tests/models/test_qwen2.py:100-106
    torch.testing.assert_close(P.rotate_half(torch.tensor([1.0, 2.0, 3.0, 4.0])), torch.tensor([-3.0, -4.0, 1.0, 2.0]))


def test_rope_table_values_of_reference_tests():
    # /root/reference/tests/models/test_qwen2.py:67-88: position 0 -> cos 1, sin 0; D=8, theta=1e6:
    # cos[1][0] = cos(1), cos[1][1] = cos(1e6^-0.25)
    cos, sin = P.rope_cos_sin(torch.arange(4), 8, 1_000_000.0)
    torch.testing.assert_close(cos[0], torch.ones(8))
    torch.testing.assert_close(sin[0], torch.zeros(8))
    assert cos[1][0].item() == pytest.approx(math.cos(1.0), abs=1e-6)
    assert cos[1][1].item() == pytest.approx(math.cos(1_000_000.0 ** -0.25), abs=1e-6)
    torch.testing.assert_close(cos[:, :4], cos[:, 4:])          # emb = cat(freq, freq)


def test_rope_identity_at_position_zero_and_norm_preserving():
    # /root/reference/tests/models/test_qwen2.py:110-145
    x = torch.randn(3, 5, 16)
    cos, sin = P.rope_cos_sin(torch.zeros(5, dtype=torch.long), 16, 1e4)
    torch.testing.assert_close(P.apply_rope(x, cos, sin), x)
    cos, sin = P.rope_cos_sin(torch.arange(5), 16, 1e4)
    torch.testing.assert_close(P.apply_rope(x, cos, sin).norm(dim=-1), x.norm(dim=-1))


def test_rope_scores_depend_on_distance_only():
    """<rope(q, m), rope(k, n)> depends on m - n: a shift of all positions changes nothing.  A wrong
    sign in rotate_half, or pairing neighbours (2i, 2i+1) while the table is cat(freq, freq), breaks it."""
    q, k = torch.randn(1, 6, 32, dtype=torch.float64), torch.randn(1, 6, 32, dtype=torch.float64)
    def scores(shift):
        cos, sin = P.rope_cos_sin(torch.arange(6) + shift, 32, 1e4, torch.float64)
        return P.apply_rope(q, cos, sin)[0] @ P.apply_rope(k, cos, sin)[0].t()
    torch.testing.assert_close(scores(0), scores(37), atol=1e-9, rtol=1e-9)
    assert not torch.allclose(scores(0), q[0] @ k[0].t(), atol=1e-3)      # and it does encode position


def test_rope_pairs_element_i_with_i_plus_half():
    # one position, one frequency: element 0 and element D/2 form the rotated pair
    x = torch.zeros(1, 1, 8)
    x[0, 0, 0] = 1.0
    cos, sin = P.rope_cos_sin(torch.tensor([1]), 8, 1e4)
    out = P.apply_rope(x, cos, sin)[0, 0]
    assert out[0].item() == pytest.approx(math.cos(1.0), abs=1e-6)
    assert out[4].item() == pytest.approx(math.sin(1.0), abs=1e-6)
    assert out[1].item() == 0.0


# ------------------------------------------------------------------------------ attention
def test_attention_is_library_sdpa_with_repeated_kv():
    q, k, v = torch.randn(6, 9, 16), torch.randn(2, 9, 16), torch.randn(2, 9, 16)
    want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None],
                                          is_causal=True)[0]
    torch.testing.assert_close(P.causal_attention(q, k, v), want, atol=1e-5, rtol=1e-5)


def test_attention_head_mapping_is_h_div_group_not_h_mod():
    # value heads are constant vectors: query head h must return kv head h // (nq/nkv)
    q, k = torch.randn(4, 3, 8), torch.randn(2, 3, 8)
    v = torch.stack([torch.full((3, 8), 1.0), torch.full((3, 8), 2.0)])
    out = P.causal_attention(q, k, v)
    assert [round(out[h, -1, 0].item()) for h in range(4)] == [1, 1, 2, 2]


def test_attention_first_row_single_token_and_hand_case():
    # /root/reference/tests/models/test_qwen2.py:149-190, 220-227: row 0 = v[0]; T = 1 -> out = v;
    # 2x2 identity: row 1 = softmax([0, 1/sqrt(2)]) mix of the values
    q = k = v = torch.eye(2).unsqueeze(0)
    out = P.causal_attention(q, k, v)
    torch.testing.assert_close(out[0, 0], v[0, 0])
    w = torch.softmax(torch.tensor([0.0, 1.0 / math.sqrt(2.0)]), dim=0)
    torch.testing.assert_close(out[0, 1], w[0] * v[0, 0] + w[1] * v[0, 1])
    one = torch.randn(3, 1, 8)
    torch.testing.assert_close(P.causal_attention(one, one, one), one)


def test_attention_future_tokens_do_not_reach_back():
    # /root/reference/tests/models/test_qwen2_attention.py:24-45
    q, k, v = torch.randn(2, 6, 8), torch.randn(2, 6, 8), torch.randn(2, 6, 8)
    base = P.causal_attention(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[:, 4:] += 5.0
    v2[:, 4:] -= 3.0
    torch.testing.assert_close(P.causal_attention(q, k2, v2)[:, :4], base[:, :4])


def test_attention_rejects_indivisible_heads():
    # /root/reference/tests/models/test_qwen2.py:212-218
    with pytest.raises(ValueError, match="divisible"):
        P.causal_attention(torch.randn(5, 2, 4), torch.randn(2, 2, 4), torch.randn(2, 2, 4))


def test_attention_window_counts_the_token_itself():
    # window 1 -> every token sees only itself -> out = v; window >= T -> full causal
    q, k, v = torch.randn(2, 7, 8), torch.randn(2, 7, 8), torch.randn(2, 7, 8)
    torch.testing.assert_close(P.causal_attention(q, k, v, window=1), v)
    torch.testing.assert_close(P.causal_attention(q, k, v, window=7), P.causal_attention(q, k, v))
    # window 3: row 5 must ignore key 2 and see key 3
    k2, v2 = k.clone(), v.clone()
    k2[:, 2] += 9.0
    torch.testing.assert_close(P.causal_attention(q, k2, v, window=3)[:, 5], P.causal_attention(q, k, v, window=3)[:, 5])
    v2[:, 3] += 9.0
    assert not torch.allclose(P.causal_attention(q, k, v2, window=3)[:, 5], P.causal_attention(q, k, v, window=3)[:, 5])


# ------------------------------------------------------------------------------ feed-forward, blocks
def test_swiglu_all_ones_vector_of_reference_tests():
    # /root/reference/tests/models/test_qwen2_mlp.py:22-39: all-ones weights, x=[1,2,3,4], H4 I8 -> 8 * silu(10) * 10
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    out = P.swiglu(x, torch.ones(8, 4), torch.ones(8, 4), torch.ones(4, 8))
    want = 8 * (10.0 / (1.0 + math.exp(-10.0))) * 10.0
    torch.testing.assert_close(out, torch.full((1, 4), want))


def test_swiglu_is_library_silu_on_the_gate_half():
    x, wg, wu, wd = torch.randn(3, 6), torch.randn(10, 6), torch.randn(10, 6), torch.randn(6, 10)
    torch.testing.assert_close(P.swiglu(x, wg, wu, wd), (F.silu(x @ wg.t()) * (x @ wu.t())) @ wd.t())
    assert not torch.allclose(P.swiglu(x, wg, wu, wd), P.swiglu(x, wu, wg, wd), atol=1e-3)   # gate and up are not symmetric


def _tiny_weights(layers=1, h=8, i=12, nq=2, nkv=1, d=4, v=17, zero_proj=False):
    cfg = dict(num_hidden_layers=layers, hidden_size=h, intermediate_size=i, num_attention_heads=nq,
               num_key_value_heads=nkv, head_dim=d, vocab_size=v, rope_theta=1e4, rms_norm_eps=1e-6,
               tie_word_embeddings=True)
    w = {"model.embed_tokens.weight": torch.randn(v, h), "model.norm.weight": torch.ones(h)}
    for l in range(layers):
        p = f"model.layers.{l}"
        make = (lambda *s: torch.zeros(*s)) if zero_proj else (lambda *s: torch.randn(*s) * 0.3)
        w[f"{p}.input_layernorm.weight"] = torch.ones(h)
        w[f"{p}.post_attention_layernorm.weight"] = torch.ones(h)
        for name, rows in (("q_proj", nq * d), ("k_proj", nkv * d), ("v_proj", nkv * d)):
            w[f"{p}.self_attn.{name}.weight"] = make(rows, h)
            w[f"{p}.self_attn.{name}.bias"] = make(rows)
        w[f"{p}.self_attn.o_proj.weight"] = make(h, nq * d)
        w[f"{p}.mlp.gate_proj.weight"] = make(i, h)
        w[f"{p}.mlp.up_proj.weight"] = make(i, h)
        w[f"{p}.mlp.down_proj.weight"] = make(h, i)
    return cfg, w


def test_decoder_layer_with_zero_projections_is_identity():
    # /root/reference/tests/models/test_qwen2_decoder_layer.py:31-62
    cfg, w = _tiny_weights(zero_proj=True)
    h = torch.randn(5, 8)
    torch.testing.assert_close(P.decoder_layer(h, w, 0, cfg, torch.arange(5)), h)


def _layer_with_constant_attention(h=8, i=12, nq=2, nkv=1, d=4):
    """One layer whose attention term does not depend on its input: q/k/v matrices and the q/k biases are
    zero, the value bias and o_proj are random, so every softmax is uniform over equal values and the term is
    c = o_proj(bv repeated for the query heads).  The feed-forward weights are random."""
    cfg, w = _tiny_weights(h=h, i=i, nq=nq, nkv=nkv, d=d)
    p = "model.layers.0.self_attn"
    for name in ("q_proj", "k_proj", "v_proj"):
        w[f"{p}.{name}.weight"] = torch.zeros_like(w[f"{p}.{name}.weight"])
    w[f"{p}.q_proj.bias"] = torch.zeros(nq * d)
    w[f"{p}.k_proj.bias"] = torch.zeros(nkv * d)
    bv = w[f"{p}.v_proj.bias"]
    c = w[f"{p}.o_proj.weight"] @ bv.view(nkv, d).repeat_interleave(nq // nkv, dim=0).reshape(nq * d)
    return cfg, w, c


def test_each_norm_weight_sits_before_its_own_half_of_the_layer():
    """/root/reference/somi_inference/models/qwen2.py:333-339: input_layernorm feeds the attention,
    post_attention_layernorm feeds the feed-forward.  A zero input_layernorm weight makes the attention's input
    zero, so the attention term is the constant o_proj(repeat(bv)) (biases only) whatever h is, and the
    feed-forward still sees h + that constant; a zero post_attention_layernorm weight makes the feed-forward
    term vanish (swiglu(0) = 0) and leaves h + attention.  With the two weights swapped both fail."""
    cfg, w = _tiny_weights()
    p = "model.layers.0"
    h, positions = torch.randn(5, 8), torch.arange(5)
    norm2 = torch.linspace(0.5, 1.5, 8)
    bv = w[f"{p}.self_attn.v_proj.bias"]
    constant = w[f"{p}.self_attn.o_proj.weight"] @ bv.view(1, 4).repeat_interleave(2, dim=0).reshape(8)
    assert constant.abs().max() > 1e-3

    first_off = dict(w)
    first_off[f"{p}.input_layernorm.weight"] = torch.zeros(8)
    first_off[f"{p}.post_attention_layernorm.weight"] = norm2
    mid = h + constant
    x = norm2 * mid * torch.rsqrt(mid.pow(2).mean(-1, keepdim=True) + 1e-6)
    mlp = (F.silu(x @ w[f"{p}.mlp.gate_proj.weight"].t()) * (x @ w[f"{p}.mlp.up_proj.weight"].t())) \
        @ w[f"{p}.mlp.down_proj.weight"].t()
    torch.testing.assert_close(P.decoder_layer(h, first_off, 0, cfg, positions), mid + mlp, atol=1e-5, rtol=1e-5)

    second_off = dict(w)
    second_off[f"{p}.input_layernorm.weight"] = torch.linspace(1.5, 0.5, 8)
    second_off[f"{p}.post_attention_layernorm.weight"] = torch.zeros(8)
    got = P.decoder_layer(h, second_off, 0, cfg, positions)
    normed = second_off[f"{p}.input_layernorm.weight"] * h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6)
    attention = P.attention_block(normed, w, f"{p}.self_attn", cfg, positions, None)
    torch.testing.assert_close(got, h + attention, atol=1e-5, rtol=1e-5)
    assert not torch.allclose(got, h + constant, atol=1e-3)        # the attention does see its normed input


def test_feed_forward_reads_the_stream_after_the_attention_was_added():
    """/root/reference/somi_inference/models/qwen2.py:335-339: residual = h + attn; the second norm and the
    feed-forward read that sum, not the layer's input.  With an attention term that is a known constant c the
    layer is h + c + swiglu(rms_norm(h + c)), computed here inline with library routines.  A parallel block
    (feed-forward from norm2(h)) or a feed-forward added to h alone fails it."""
    cfg, w, c = _layer_with_constant_attention()
    assert c.abs().max() > 1e-2
    p = "model.layers.0"
    norm2 = torch.linspace(0.6, 1.7, 8)
    w[f"{p}.input_layernorm.weight"] = torch.linspace(1.4, 0.3, 8)
    w[f"{p}.post_attention_layernorm.weight"] = norm2
    h = torch.randn(6, 8)
    mid = h + c
    x = F.rms_norm(mid, (8,), norm2, 1e-6)
    mlp = F.linear(F.silu(F.linear(x, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(x, w[f"{p}.mlp.up_proj.weight"]),
                   w[f"{p}.mlp.down_proj.weight"])
    got = P.decoder_layer(h, w, 0, cfg, torch.arange(6))
    torch.testing.assert_close(got, mid + mlp, atol=1e-5, rtol=1e-5)
    # what the two plausible mistakes would give is far from it
    x_parallel = F.rms_norm(h, (8,), norm2, 1e-6)
    mlp_parallel = F.linear(F.silu(F.linear(x_parallel, w[f"{p}.mlp.gate_proj.weight"]))
                            * F.linear(x_parallel, w[f"{p}.mlp.up_proj.weight"]), w[f"{p}.mlp.down_proj.weight"])
    assert not torch.allclose(got, mid + mlp_parallel, atol=1e-3)


def test_model_is_causal_and_tied_head_uses_embedding():
    cfg, w = _tiny_weights(layers=2)
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    full = P.model_logits(cfg, w, ids)
    torch.testing.assert_close(P.model_logits(cfg, w, ids[:5]), full[:5])
    assert full.shape == (8, 17)
    # untied: the head matrix is used instead of the embedding
    w2 = dict(w)
    w2["lm_head.weight"] = torch.randn(17, 8)
    cfg2 = dict(cfg, tie_word_embeddings=False)
    assert not torch.allclose(P.model_logits(cfg2, w2, ids), full)


def test_logits_at_chosen_rows_are_the_rows_of_all_logits():
    cfg, w = _tiny_weights(layers=2)
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    torch.testing.assert_close(P.model_logits(cfg, w, ids, rows=[7, 2]), P.model_logits(cfg, w, ids)[[7, 2]])


def test_model_logits_do_not_depend_on_a_shift_of_positions():
    # only distances count: the same tokens at positions p.. and p+s.. give the same logits
    cfg, w = _tiny_weights(layers=2)
    w = {k: v.double() for k, v in w.items()}
    ids = [3, 1, 4, 1, 5, 9]
    torch.testing.assert_close(P.model_logits(cfg, w, ids, first_position=0),
                               P.model_logits(cfg, w, ids, first_position=29), atol=1e-9, rtol=1e-9)


# ------------------------------------------------------------------------------ projections, head split, final norm
def test_linear_is_library_linear_with_its_bias():
    # /root/reference/somi_inference/models/qwen2.py:268-271: nn.Linear, weight [out, in]; a transposed weight or a
    # dropped bias fails
    x, w, b = torch.randn(5, 7), torch.randn(3, 7), torch.randn(3)
    torch.testing.assert_close(P.linear(x, w, b), F.linear(x, w, b))
    torch.testing.assert_close(P.linear(x, w), F.linear(x, w))
    assert not torch.allclose(P.linear(x, w, b), F.linear(x, w), atol=1e-3)


def _attention_weights(prefix, h, nq, nkv, d, fill):
    w = {}
    for name, rows in (("q_proj", nq * d), ("k_proj", nkv * d), ("v_proj", nkv * d)):
        w[f"{prefix}.{name}.weight"] = fill(rows, h)
        w[f"{prefix}.{name}.bias"] = fill(rows)
    w[f"{prefix}.o_proj.weight"] = fill(h, nq * d)
    return w


def test_a_value_bias_alone_comes_out_as_the_output_projection_of_the_bias():
    """/root/reference/somi_inference/models/qwen2.py:270, 290, 297: v = x . Wv^T + bv.  With every attention
    tensor zero but the value bias and the output projection, every softmax is uniform over equal values, so
    each token's output is o_proj(bv repeated for the query heads of its kv head), whatever x is.  A value bias
    that is dropped (a key bias cancels in the softmax and would not be missed) gives zero instead."""
    h, nq, nkv, d = 10, 4, 2, 6
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rope_theta=1e4)
    w = _attention_weights("a", h, nq, nkv, d, lambda *s: torch.zeros(*s))
    bv = torch.randn(nkv * d)
    wo = torch.randn(h, nq * d)
    w["a.v_proj.bias"], w["a.o_proj.weight"] = bv, wo
    out = P.attention_block(torch.randn(7, h), w, "a", cfg, torch.arange(7), None)
    merged = bv.view(nkv, d).repeat_interleave(nq // nkv, dim=0).reshape(nq * d)      # query head h reads kv head h // 2
    torch.testing.assert_close(out, (wo @ merged).expand(7, h))
    assert out.abs().max() > 1e-2


def test_heads_are_contiguous_blocks_of_head_dim_of_a_projection():
    """/root/reference/somi_inference/models/qwen2.py:292-297, 285: view(.., n_heads, head_dim): head h of a
    projection is its elements [h D, (h + 1) D), and the heads are merged in the same order before o_proj.
    Checked against a loop that slices those ranges explicitly and calls the library's attention once per query
    head; heads interleaved (element i belongs to head i mod n) fail it."""
    h, nq, nkv, d, t = 12, 4, 2, 8, 6
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rope_theta=1e4)
    w = _attention_weights("a", h, nq, nkv, d, lambda *s: torch.randn(*s) * 0.5)
    x, positions = torch.randn(t, h), torch.arange(t)
    got = P.attention_block(x, w, "a", cfg, positions, None)
    q = F.linear(x, w["a.q_proj.weight"], w["a.q_proj.bias"])
    k = F.linear(x, w["a.k_proj.weight"], w["a.k_proj.bias"])
    v = F.linear(x, w["a.v_proj.weight"], w["a.v_proj.bias"])
    cos, sin = P.rope_cos_sin(positions, d, 1e4)
    rotate = lambda block: block * cos + P.rotate_half(block) * sin
    merged = torch.zeros(t, nq * d)
    for head in range(nq):
        kv = head // (nq // nkv)
        qh = rotate(q[:, head * d:(head + 1) * d])
        kh = rotate(k[:, kv * d:(kv + 1) * d])
        vh = v[:, kv * d:(kv + 1) * d]
        merged[:, head * d:(head + 1) * d] = F.scaled_dot_product_attention(qh[None], kh[None], vh[None], is_causal=True)[0]
    torch.testing.assert_close(got, F.linear(merged, w["a.o_proj.weight"]), atol=1e-5, rtol=1e-5)


def test_final_norm_stands_between_the_last_layer_and_the_head():
    """/root/reference/somi_inference/models/qwen2.py:378, 386 and qwen2_adapter.py:60-62: logits =
    head(norm(h)).  The norm's weight scales the logits linearly (a norm applied after the head, or none, does
    not), and a model without layers has the closed form E . rmsnorm(E[id])."""
    cfg, w = _tiny_weights(layers=2)
    ids = [3, 1, 4, 1, 5]
    base = P.model_logits(cfg, w, ids)
    doubled = dict(w)
    doubled["model.norm.weight"] = 2.0 * w["model.norm.weight"]
    torch.testing.assert_close(P.model_logits(cfg, doubled, ids), 2.0 * base)
    skewed = dict(w)
    skewed["model.norm.weight"] = torch.linspace(0.5, 2.0, 8)
    assert not torch.allclose(P.model_logits(cfg, skewed, ids), base, atol=1e-3)
    empty = dict(cfg, num_hidden_layers=0)
    table = w["model.embed_tokens.weight"]
    rows = table[torch.tensor(ids)]
    want = (skewed["model.norm.weight"] * rows * torch.rsqrt(rows.pow(2).mean(-1, keepdim=True) + 1e-6)) @ table.t()
    torch.testing.assert_close(P.model_logits(empty, skewed, ids), want)


# ------------------------------------------------------------------------------ sampling rules
def test_sampling_vectors_of_reference_tests():
    # /root/reference/tests/core/test_sampler.py:58-128
    assert int(P.sampling_distribution(torch.tensor([1.0, 3.0, 2.0]), [], 0.0).argmax()) == 1
    assert int(P.sampling_distribution(torch.tensor([2.0, 1.5]), [0], 0.0, penalty=2.0).argmax()) == 1
    kept = P.keep_top_k(torch.tensor([5.0, 4.0, 4.0, 1.0]), 2)
    assert int(torch.isfinite(kept).sum()) == 2
    kept = P.keep_top_p(torch.tensor([4.0, 3.0, 2.0, 1.0]), 0.5)
    assert torch.isfinite(kept).tolist() == [True, False, False, False]
    out = P.penalize_repetition(torch.tensor([-1.0, 0.5, 0.5]), [0], 2.0)
    assert out.tolist() == [-2.0, 0.5, 0.5]


def test_sampling_order_penalty_temperature_topk_topp():
    logits = torch.tensor([3.0, 2.9, 1.0, -2.0])
    dist = P.sampling_distribution(logits, [0], 0.5, top_k=2, top_p=1.0, penalty=3.0)
    # penalty first: 3.0 -> 1.0, so the two largest are now ids 1 and 0/2 tie broken by topk; id 3 is out
    assert dist[3] == 0 and dist[1] > 0.9
    assert dist.sum().item() == pytest.approx(1.0)
