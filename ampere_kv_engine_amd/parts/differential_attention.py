"""Differential attention: every head holds two attention maps over the same values and puts out their difference.

    q = W_q h: per head [map 1 | map 2], each `head_dim` wide;  k = W_k h likewise per key head;  v = W_v h (`value_dim`)
    with `position` (a `rope_scaled` specification) every map's q and k are rotated over their first dims dimensions
    a_m = softmax((q_m . k_m) * scale over the keys j <= i, and i - j < window where there is one) v,   m = 1, 2
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + `constant`        (four vectors of `head_dim`; one number for the layer)
    o = a_1 - lambda a_2;   o <- o / rms(o) * (1 - `constant`)   (over the head's value_dim values, no weight)
    out = W_o (concat_h(o_h) * sigmoid(W_g h))                   (a gate per output value, from the layer's input)

Query head h reads key head h // (q_heads / kv_heads).  A key head's record in the pages is its two maps side by side
(2 * head_dim wide), its values lie there once: the cache holds what an attention of kv_heads heads of twice the key
width would.  The four projections are one product.  Scores, softmax weights, lambda, the difference and its norm are
float32; lambda is formed once, at load.
"""

from __future__ import annotations

import torch

from ..weights.spec import BIAS, TensorSpec
from .base import PagedKV, Part, build_part, register_part
from .linear import Linear

MAPS = 2


class DifferentialAttention(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.q_heads, self.kv_heads = int(spec["q_heads"]), int(spec["kv_heads"])
        self.dim, self.vdim = int(spec["head_dim"]), int(spec["value_dim"])
        self.scale, self.constant, self.eps = float(spec["scale"]), float(spec["constant"]), float(spec["eps"])
        self.window = int(spec["window"]) if spec.get("window") is not None else None
        self.name = spec.get("name", "attn")
        if self.q_heads % self.kv_heads:
            raise ValueError(f"q_heads {self.q_heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.window is not None and self.window <= 0:
            raise ValueError(f"window must be positive or None, got {self.window}")
        self.position = build_part("position", spec["position"], runtime) if spec.get("position") is not None else None
        if self.position is not None and self.position.dims > self.dim:
            raise ValueError(f"a rotation over {self.position.dims} dimensions does not fit maps of {self.dim}")
        self.q_size, self.k_size = self.q_heads * MAPS * self.dim, self.kv_heads * MAPS * self.dim
        self.v_size, self.o_size = self.kv_heads * self.vdim, self.q_heads * self.vdim
        self.qkvg = Linear(runtime, self.hidden, [self.q_size, self.k_size, self.v_size, self.o_size], ["q", "k", "v", "g"])
        self.out = Linear(runtime, self.o_size, [self.hidden], ["o"])
        self.lam = None
        runtime.kernels.check_gated_attention_sizes(self.q_heads * MAPS, self.kv_heads, self.dim, self.vdim, runtime.page_size)

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _own_specs(self, p):
        return [TensorSpec(p + name, (self.dim,), BIAS) for name in ("lq1", "lk1", "lq2", "lk2")]

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.qkvg.tensors(p) + self.out.tensors(p) + self._own_specs(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.qkvg.load(fetch, p)
        self.out.load(fetch, p)
        lq1, lk1, lq2, lk2 = (fetch(spec).to(torch.float32) for spec in self._own_specs(p))
        self.lam = (torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + self.constant).reshape(1).contiguous()

    def weight_bytes(self):
        return self.qkvg.weight_bytes() + self.out.weight_bytes()

    def cache_request(self):
        return PagedKV(self.kv_heads, MAPS * self.dim, self.window, value_dim=self.vdim)

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        projected = ctx.arena.take((tokens, self.q_size + self.k_size + self.v_size + self.o_size), dtype)
        self.qkvg.forward(x, projected)
        meta = ctx.paged[cache.group]
        q = ctx.arena.take((tokens, self.q_size), dtype)
        rotation = {}
        if self.position is not None:
            rotation = dict(table=self.position.table, rot_dims=self.position.dims, positions=ctx.positions)
        k.unit_norm_write(projected, self.q_heads, self.kv_heads, self.dim, self.vdim, None,
                          meta.slot_map if writes_cache else None, cache.k, cache.v, q, maps=MAPS, **rotation)
        maps = ctx.arena.take((tokens, MAPS * self.o_size), dtype)
        k.gated_attention(q, cache.k, cache.v, None, 0, ctx, meta, self.q_heads, self.kv_heads, self.dim, self.vdim,
                          self.scale, None, None, self.window, False, maps, maps=MAPS)
        gated = ctx.arena.take((tokens, self.o_size), dtype)
        k.difference_norm_gate(maps, self.lam, self.eps, 1.0 - self.constant, projected,
                               self.q_size + self.k_size + self.v_size, self.q_heads, self.vdim, gated)
        return self.out.forward(gated, ctx.arena.take((tokens, self.hidden), dtype))


register_part("mixer", "differential_attention", DifferentialAttention)
