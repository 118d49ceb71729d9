"""Plain Qwen2.5 decoder: every function cites the reference lines it is written from.

All paths are under /root/reference/somi_inference/.
"""

from __future__ import annotations

import json
import math
import os

import torch
from safetensors.torch import load_file


# ----------------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """models/qwen2.py:55-62: variance = mean(x^2) over the last dim; x * rsqrt(variance + eps); times weight.
    No mean subtraction, no bias."""
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


def rope_inv_freq(head_dim: int, theta: float, dtype=torch.float32) -> torch.Tensor:
    """models/qwen2.py:76: inv_freq[j] = 1 / theta^(2j / head_dim), j = 0 .. head_dim/2 - 1."""
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2).to(dtype) / head_dim))


def rope_cos_sin(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32):
    """models/qwen2.py:77-81, 88-89: freq = outer(position, inv_freq); emb = cat(freq, freq); cos, sin of emb."""
    freq = torch.outer(positions.to(dtype), rope_inv_freq(head_dim, theta, dtype))
    emb = torch.cat((freq, freq), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """models/qwen2.py:95-99: [x1, x2] -> [-x2, x1] with x1, x2 the two halves of the last dim."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """models/qwen2.py:102-113: x * cos + rotate_half(x) * sin, cos/sin broadcast over heads.
    x: [heads, T, D]; cos, sin: [T, D]."""
    return x * cos.unsqueeze(0) + rotate_half(x) * sin.unsqueeze(0)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int | None = None,
                     scale: float | None = None) -> torch.Tensor:
    """models/qwen2.py:158-186: each kv head is repeated nq/nkv times (repeat_interleave, so query head h
    uses kv head h // (nq/nkv)); scores = q.k^T * D^-0.5; entries above the diagonal are -inf; softmax in
    float32; weights . v.  q: [nq, T, D]; k, v: [nkv, T, D] -> [nq, T, D].

    ``window`` (not in the reference, which stores the argument and ignores it, models/qwen2.py:262,272):
    a token sees the last ``window`` keys, itself included.
    """
    nq, t, d = q.shape
    nkv = k.shape[0]
    if nq % nkv != 0:
        raise ValueError(f"num_q_heads ({nq}) must be divisible by num_kv_heads ({nkv})")   # models/qwen2.py:116-123
    rep = nq // nkv
    k = k.repeat_interleave(rep, dim=0)
    v = v.repeat_interleave(rep, dim=0)
    scale = d ** -0.5 if scale is None else scale
    scores = torch.einsum("hid,hjd->hij", q, k) * scale
    i = torch.arange(t).unsqueeze(1)
    j = torch.arange(t).unsqueeze(0)
    hidden = j > i
    if window is not None:
        hidden = hidden | (j <= i - window)
    scores = scores.masked_fill(hidden.unsqueeze(0), float("-inf"))
    weights = torch.softmax(scores, dim=-1)
    return torch.einsum("hij,hjd->hid", weights, v)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """nn.Linear as used in models/qwen2.py:268-271, 221-222: y = x . W^T + b, W stored [out, in]."""
    y = x @ weight.t()
    return y if bias is None else y + bias


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """models/qwen2.py:226-229 with the merged weight of models/qwen2_adapter.py:183-190 (gate rows first):
    gate, up = halves of x . W_gate_up^T; y = down(silu(gate) * up), silu(z) = z * sigmoid(z)."""
    gate = x @ w_gate.t()
    up = x @ w_up.t()
    return ((gate * torch.sigmoid(gate)) * up) @ w_down.t()


def attention_block(x: torch.Tensor, w: dict, prefix: str, cfg: dict, positions: torch.Tensor,
                    window: int | None) -> torch.Tensor:
    """models/qwen2.py:288-300, 274-286: project q/k/v (with bias), split into heads of head_dim contiguous
    elements, rotate q and k, attend, merge heads, project with o (no bias)."""
    t = x.shape[0]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    bias = lambda name: w.get(f"{prefix}.{name}.bias")
    q = linear(x, w[f"{prefix}.q_proj.weight"], bias("q_proj")).view(t, nq, d).transpose(0, 1)
    k = linear(x, w[f"{prefix}.k_proj.weight"], bias("k_proj")).view(t, nkv, d).transpose(0, 1)
    v = linear(x, w[f"{prefix}.v_proj.weight"], bias("v_proj")).view(t, nkv, d).transpose(0, 1)
    cos, sin = rope_cos_sin(positions, d, cfg["rope_theta"], x.dtype)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    out = causal_attention(q, k, v, window)
    return linear(out.transpose(0, 1).reshape(t, nq * d), w[f"{prefix}.o_proj.weight"])


def decoder_layer(h: torch.Tensor, w: dict, index: int, cfg: dict, positions: torch.Tensor) -> torch.Tensor:
    """models/qwen2.py:325-339: h = h + attn(norm1(h)); h = h + mlp(norm2(h))."""
    p = f"model.layers.{index}"
    eps = cfg["rms_norm_eps"]
    h = h + attention_block(rms_norm(h, w[f"{p}.input_layernorm.weight"], eps), w, f"{p}.self_attn", cfg,
                            positions, layer_window(cfg, index))
    x = rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], eps)
    return h + swiglu(x, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                      w[f"{p}.mlp.down_proj.weight"])


def layer_window(cfg: dict, index: int) -> int | None:
    """Meaning of the config.json keys (the reference ignores them): with use_sliding_window, layers from
    max_window_layers on see the last sliding_window keys."""
    if not cfg.get("use_sliding_window", False):
        return None
    return cfg["sliding_window"] if index >= cfg["max_window_layers"] else None


# ----------------------------------------------------------------------------- whole model
def read_model(model_dir: str, dtype=torch.float32) -> tuple[dict, dict]:
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as handle:
        cfg = json.load(handle)
    if "head_dim" not in cfg:
        cfg["head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]   # models/qwen2_adapter.py:213
    if "rope_theta" not in cfg:
        cfg["rope_theta"] = (cfg.get("rope_parameters") or {}).get("rope_theta", 1_000_000.0)   # qwen2_adapter.py:208-211
    cfg.setdefault("rms_norm_eps", 1e-6)
    weights = {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, weights


def model_logits(cfg: dict, w: dict, token_ids: list[int], first_position: int = 0,
                 rows: list[int] | None = None) -> torch.Tensor:
    """models/qwen2.py:380-386 then models/qwen2_adapter.py:60-62: embed, layers, final norm, logits = h . E^T
    (or lm_head when the checkpoint is untied).  Returns logits at every position, [T, V], or at ``rows`` only
    (the reference projects the last position alone, models/qwen2_adapter.py:95: the head works row by row)."""
    ids = torch.tensor(token_ids, dtype=torch.long)
    h = w["model.embed_tokens.weight"][ids]
    positions = torch.arange(first_position, first_position + len(token_ids))
    for index in range(cfg["num_hidden_layers"]):
        h = decoder_layer(h, w, index, cfg, positions)
    h = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    if rows is not None:
        h = h[torch.tensor(rows, dtype=torch.long)]
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return h @ head.t()


def greedy_generate(cfg: dict, w: dict, prompt: list[int], max_new_tokens: int, eos: int | None = None) -> list[int]:
    """core/continuous_batching.py:140-177 for one request with temperature 0: the next token is the argmax of
    the last position's logits; stop after max_new_tokens or at eos (which is kept)."""
    tokens, out = list(prompt), []
    for _ in range(max_new_tokens):
        nxt = int(torch.argmax(model_logits(cfg, w, tokens)[-1]))
        out.append(nxt)
        tokens.append(nxt)
        if eos is not None and nxt == eos:
            break
    return out


# ----------------------------------------------------------------------------- sampling
def penalize_repetition(logits: torch.Tensor, history: list[int], penalty: float) -> torch.Tensor:
    """core/sampler.py:80-102: for each distinct id in the history, logit > 0 ? logit / p : logit * p."""
    out = logits.clone()
    if penalty == 1.0 or not history:
        return out
    for token in set(history):
        out[token] = out[token] / penalty if out[token] > 0 else out[token] * penalty
    return out


def keep_top_k(logits: torch.Tensor, k: int) -> torch.Tensor:
    """core/sampler.py:116-133: keep exactly min(k, V) entries (those torch.topk returns), others -> -inf."""
    if k == -1:
        return logits.clone()
    keep = torch.topk(logits, min(k, logits.numel())).indices
    out = torch.full_like(logits, float("-inf"))
    out[keep] = logits[keep]
    return out


def keep_top_p(logits: torch.Tensor, p: float) -> torch.Tensor:
    """core/sampler.py:135-157: sort descending, softmax, cumulative sum; remove entries whose cumulative
    probability exceeds p, shifted right by one so the entry that crosses p stays and the first always stays."""
    if p == 1.0:
        return logits.clone()
    ordered, order = torch.sort(logits, descending=True)
    cumulative = torch.cumsum(torch.softmax(ordered.float(), dim=-1), dim=-1)
    remove = cumulative > p
    remove[1:] = remove[:-1].clone()
    remove[0] = False
    out = logits.clone()
    out[order[remove]] = float("-inf")
    return out


def sampling_distribution(logits: torch.Tensor, history: list[int], temperature: float, top_k: int = -1,
                          top_p: float = 1.0, penalty: float = 1.0) -> torch.Tensor:
    """core/sampler.py:48-55 order: penalty, temperature, top-k, top-p, then softmax (:172).  With temperature 0
    the result is one-hot at the argmax and top-k / top-p are skipped (:123, 142, 169-170)."""
    z = penalize_repetition(logits.float(), history, penalty)
    if temperature == 0.0:
        out = torch.zeros_like(z)
        out[int(torch.argmax(z))] = 1.0
        return out
    z = z / temperature
    z = keep_top_p(keep_top_k(z, top_k), top_p)
    return torch.softmax(z, dim=-1)
