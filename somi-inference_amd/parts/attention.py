"""Grouped-query attention over the paged cache.

Reference: somi_inference/models/qwen2.py:252-300 (q/k/v projections with bias,
o projection without, heads as contiguous head_dim blocks of the projection,
rotary encoding on q and k before k is cached), :158-186 (causal softmax
attention, scale head_dim^-0.5, query head h reads key/value head
h // (nq / nkv)) and somi_inference/core/paged_attention.py:352-413 (the same
over cache pages).  The reference has one function for whole prompts that never
reads the cache and one for single decoded tokens; here one kernel contract
serves any mix: keys and values of the step's tokens are written to their pages
first, then every token attends over its request's pages up to its own position.
"""

from __future__ import annotations

import torch

from ..kernels import attention as attention_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, WeightSpec
from .base import Fetch, LayerCache, Mixer, PagedKVSpec, PartSpec, Runtime
from .linear import NormedRows, Projection
from .registry import build_part


class GroupedQueryAttention(Mixer):
    graph_safe = True
    takes_normed_rows = True      # x only goes through the q/k/v projection, which norms rows while loading them
    entry_split = attention_kernels.DECODE_PORTION    # longer portions take the tile kernel, the rest the decode kernel

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: PartSpec, qkv_bias: bool = True, out_bias: bool = False,
                 window: int | None = None, scale: float | None = None, shares_cache: bool = False,
                 names: dict[str, str] | None = None) -> None:
        """``names``: what the checkpoint calls this part's tensors, role -> name under the prefix.  Roles: ``q``,
        ``k``, ``v``, ``o`` (defaults ``q_proj`` ... ``o_proj``), ``position`` (``rotary_emb``), and ``qkv`` for a
        checkpoint that stores the three projections as one matrix, q rows first, then k, then v."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES) - {"qkv"}
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)} and 'qkv'")
        self.names = {**self.ROLES, **(names or {})}
        if num_heads % num_kv_heads != 0:
            # the reference's message (qwen2.py:116-123)
            raise ValueError(f"num_q_heads ({num_heads}) must be divisible by num_kv_heads ({num_kv_heads})")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qkv_bias, self.out_bias = bool(qkv_bias), bool(out_bias)
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.shares_cache = bool(shares_cache)     # reads the cache another layer writes: no k/v of its own
        self.position = build_part("position", position, prefix=self.name(self.names["position"]))

    ROLES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj", "position": "rotary_emb"}

    # ------------------------------------------------------------------ weights
    def _projections(self) -> list[tuple[str, int]]:
        """The checkpoint's input projections in the order their rows are stacked, with their widths."""
        q_width, kv_width = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        if self.shares_cache:
            return [(self.names["q"], q_width)]
        if "qkv" in self.names:
            return [(self.names["qkv"], q_width + 2 * kv_width)]
        return [(self.names["q"], q_width), (self.names["k"], kv_width), (self.names["v"], kv_width)]

    def weight_specs(self) -> list[WeightSpec]:
        specs = []
        for proj, width in self._projections():
            specs.append(WeightSpec(self.name(f"{proj}.weight"), (width, self.hidden_size), MATRIX))
            if self.qkv_bias:
                specs.append(WeightSpec(self.name(f"{proj}.bias"), (width,), VECTOR))
        out = self.names["o"]
        specs.append(WeightSpec(self.name(f"{out}.weight"), (self.hidden_size, self.num_heads * self.head_dim), MATRIX))
        if self.out_bias:
            specs.append(WeightSpec(self.name(f"{out}.bias"), (self.hidden_size,), VECTOR))
        return specs + self.position.weight_specs()

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        names = [p for p, _ in self._projections()]
        self.qkv = Projection.stacked(
            [fetch(self.name(f"{p}.weight")) for p in names],
            [fetch(self.name(f"{p}.bias")) for p in names] if self.qkv_bias else None, label="q/k/v")
        out = self.names["o"]
        self.out = Projection(fetch(self.name(f"{out}.weight")),
                              fetch(self.name(f"{out}.bias")) if self.out_bias else None, label="o")
        self.position.load(fetch, runtime)

    def flops(self, tokens: int, attended: int) -> float:
        """The projections, and q.k and p.v (two operations a product, head_dim channels, every query head) over the
        (token, key) pairs the step's tokens see."""
        return (self.qkv.flops(tokens) + self.out.flops(tokens)
                + 4.0 * self.num_heads * self.head_dim * attended)

    # -------------------------------------------------------------------- cache
    def cache_spec(self) -> PagedKVSpec | None:
        if self.shares_cache:
            return None
        return PagedKVSpec(self.num_kv_heads, self.head_dim, self.window)

    # ------------------------------------------------------------------ forward
    def forward(self, x: torch.Tensor, step, cache: LayerCache | None) -> torch.Tensor:
        if cache is None or cache.k is None:
            raise ValueError(f"{self.prefix}: attention needs a paged cache")
        view = step.paged[cache.group]
        nkv_new = 0 if self.shares_cache else self.num_kv_heads
        rotation = self.position.rotation_table()
        with stage(self.qkv.label):
            qkv = self._project_rotate_store(x, step, view, cache, rotation)     # a few rows: one kernel
        if qkv is None:
            qkv = self.qkv(x)                               # [N, (nq + 2 nkv) * D]
            with stage("position encoding, k/v into pages"):
                if rotation is None:
                    self.position.encode_qk(qkv, step, self.num_heads, nkv_new, self.head_dim)
                    inv_freq, rotary_dim = None, 0
                else:
                    inv_freq, rotary_dim = rotation
                ops.rope_kv_store(qkv, step.positions, view.slot_mapping if nkv_new else None, inv_freq, rotary_dim,
                                  self.num_heads, nkv_new, self.head_dim,
                                  cache.k if nkv_new else None, cache.v if nkv_new else None)
        with stage("attention"):
            attended = attention_kernels.paged_attention(
                qkv, self.num_heads, cache.k, cache.v, view.block_table, step,
                window=self.window or 0, scale=self.scale)
        return self.out.deferred(attended)        # the residual stream may add it in the kernel that computes it

    def _project_rotate_store(self, x, step, view, cache: LayerCache, rotation) -> torch.Tensor | None:
        """q of the step's tokens, rotated, with k and v in their pages, by the q/k/v product itself (up to 64 rows) or
        by the kernel that adds the sums of its K splits (some hundred rows); None where neither applies (many rows,
        float32, a head that is not rotated as a whole, no k/v of its own)."""
        if rotation is None or self.shares_cache:
            return None
        inv_freq, rotary_dim = rotation
        rows = x.shape[0]
        if (rotary_dim != self.head_dim or self.head_dim % 32 or cache.k.dtype != torch.bfloat16
                or not self.qkv.fusable(rows)):
            return None
        if isinstance(x, NormedRows):
            weighted, eps, stats = x.weighted, x.norm.eps, x.stats
        elif x.dtype == torch.bfloat16 and x.data_ptr() % 16 == 0:
            weighted, eps, stats = x, 0.0, None
        else:
            return None
        if rows > ops.FUSED_MAX_ROWS:
            # some hundred rows: the many-rows product shares a tile's K among workgroups, and the kernel that adds
            # their sums rotates and stores (more rows have tiles enough: the product, then the rotation)
            if ops.linear_big_splits(rows, self.qkv.out_features, self.qkv.in_features) <= 1:
                return None
            return ops.linear_big_rope_store(weighted, eps, stats, self.qkv.weight, self.qkv.bias, step.positions,
                                             view.slot_mapping, inv_freq, self.num_heads, self.num_kv_heads,
                                             self.head_dim, cache.k, cache.v)
        return ops.linear_rope_store(weighted, eps, stats, self.qkv.weight, self.qkv.bias, step.positions,
                                     view.slot_mapping, inv_freq, self.num_heads, self.num_kv_heads, self.head_dim,
                                     cache.k, cache.v)
