"""Grouped-query attention without positions in its scores, for designs whose scores and weights are float32:

    q = W_q h (+ b), k = W_k h (+ b), v = W_v h (+ b);  q and k divided by their root mean square per head (no weight) -
    or, with `projection_norm_eps`, over their whole projection, all heads at once, and multiplied by weights of that size
    (tensors `<q>.norm`, `<k>.norm`, kept float32)
    score = (q . k) * scale;  with `softcap` c: score <- c * tanh(score / c)
    a query at position i sees the keys j <= i - of its own chunk only, floor(i / chunk) = floor(j / chunk), where the
    mixer has chunks (counted from position 0 of the request); of the last `window` positions where it has a window - and,
    with `keep_first`, of the request's first so many positions as well, whose pages the cache then never gives back
    weights: softmax - with `sink`, one more term exp(0) in the denominator that has no value:
             p_j = exp(s_j) / (1 + sum exp(s_j)); with `sink="learned"` the term is exp(sink_h), a number per head (tensor
             `sink`, kept float32)
    with `position` (a `rope_scaled` specification): q and k are rotated over their first dims dimensions by the token's
    position (after the norm, where there is one; pairs in halves or interleaved, as the specification says), inside the
    kernel that writes the keys to their pages
    head h's output times sigmoid(w_g[h] . h), one number per head and token (`head_gate`), before W_o.

Keys are `head_dim` wide, values `value_dim`; query head h reads kv head h // (q_heads / kv_heads).  Keys are cached
after their norm.  All five projections are one product over the layer's input.
"""

from __future__ import annotations

import torch

from ..weights.spec import BIAS, NORM, TensorSpec
from .base import PagedKV, Part, SharesProducts, build_part, register_part
from .linear import Linear


class GatedAttention(Part, SharesProducts):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.q_heads, self.kv_heads = int(spec["q_heads"]), int(spec["kv_heads"])
        self.dim, self.vdim = int(spec["head_dim"]), int(spec["value_dim"])
        self.scale = float(spec["scale"])
        self.softcap = float(spec["softcap"]) if spec.get("softcap") is not None else None
        self.chunk = int(spec["chunk"]) if spec.get("chunk") is not None else None
        self.window = int(spec["window"]) if spec.get("window") is not None else None
        self.sink = bool(spec.get("sink", False))
        self.learned_sink = spec.get("sink") == "learned"
        self.sink_logits = None
        self.position = build_part("position", spec["position"], runtime) if spec.get("position") is not None else None
        if self.position is not None and self.position.dims > int(spec["head_dim"]):
            raise ValueError(f"a rotation over {self.position.dims} dimensions does not fit heads of {spec['head_dim']}")
        self.unit_eps = float(spec["unit_norm_eps"]) if spec.get("unit_norm_eps") is not None else None
        self.projection_eps = float(spec["projection_norm_eps"]) if spec.get("projection_norm_eps") is not None else None
        if self.unit_eps is not None and self.projection_eps is not None:
            raise ValueError("queries and keys are normed head by head or over the whole projection, not both")
        self.keep_first = int(spec.get("keep_first") or 0)
        if self.keep_first < 0 or (self.keep_first and spec.get("window") is None):
            raise ValueError("kept first tokens come with a window, and their number is not negative")
        self.q_norm_weight = self.k_norm_weight = None
        self.head_gate = bool(spec.get("head_gate", False))
        self.name = spec.get("name", "attn")
        if self.q_heads % self.kv_heads:
            raise ValueError(f"q_heads {self.q_heads} is not a multiple of kv_heads {self.kv_heads}")
        for what, value in (("chunk", self.chunk), ("window", self.window)):
            if value is not None and value <= 0:
                raise ValueError(f"{what} must be positive or None, got {value}")
        if self.softcap is not None and self.softcap <= 0:
            raise ValueError(f"softcap must be positive or None, got {self.softcap}")
        self.q_size, self.k_size, self.v_size = self.q_heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim
        names = dict(q="q", k="k", v="v", g="g", o="o", sink="sink")
        names.update(spec.get("names") or {})
        self.names = names
        bias = spec.get("bias_suffix")           # q, k and v have bias vectors named after them, with this suffix
        sizes, stacked = [self.q_size, self.k_size, self.v_size], [names["q"], names["k"], names["v"]]
        biases = [n + bias for n in stacked] if bias else None
        if self.head_gate:
            sizes.append(self.q_heads)
            stacked.append(names["g"])
            if biases:
                biases.append(None)
        self.width = sum(sizes)
        self.qkvg = self.inputs = Linear(runtime, self.hidden, sizes, stacked, bias_names=biases)
        if self.learned_sink:
            self.inputs = None      # (a tensor of its own beside the products: side by side with others it runs by itself)
        self.out = self.outputs = Linear(runtime, self.q_heads * self.vdim, [self.hidden], [names["o"]])
        runtime.kernels.check_gated_attention_sizes(self.q_heads, self.kv_heads, self.dim, self.vdim, runtime.page_size)

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _sink_spec(self, p):
        return [TensorSpec(p + self.names["sink"], (self.q_heads,), BIAS)] if self.learned_sink else []

    def _norm_specs(self, p):
        if self.projection_eps is None:
            return []
        return [TensorSpec(p + self.names["q"] + ".norm", (self.q_size,), NORM),
                TensorSpec(p + self.names["k"] + ".norm", (self.k_size,), NORM)]

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.qkvg.tensors(p) + self.out.tensors(p) + self._sink_spec(p) + self._norm_specs(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.qkvg.load(fetch, p)
        self.out.load(fetch, p)
        if self.learned_sink:
            self.sink_logits = fetch(self._sink_spec(p)[0]).to(torch.float32).contiguous()
        if self.projection_eps is not None:
            self.q_norm_weight, self.k_norm_weight = (fetch(spec).to(torch.float32).contiguous()
                                                      for spec in self._norm_specs(p))

    def weight_bytes(self):
        return self.qkvg.weight_bytes() + self.out.weight_bytes()

    def cache_request(self):
        return PagedKV(self.kv_heads, self.dim, self.window, value_dim=self.vdim, chunk=self.chunk,
                       keep_first=self.keep_first)

    def attend_columns(self, projected, at, ctx, cache, writes_cache, out, out_at, out_scale):
        """The heads' gated outputs, before the output product, from this mixer's columns of a projection."""
        k = self.rt.kernels
        meta = ctx.paged[cache.group]
        q = ctx.arena.take((projected.shape[0], self.q_size), self.rt.dtype)
        rotation = {}
        if self.position is not None:
            rotation = dict(table=self.position.table, rot_dims=self.position.dims, positions=ctx.positions)
            if self.position.interleaved:
                rotation["interleaved"] = True
        eps = self.unit_eps
        if self.projection_eps is not None:
            eps = self.projection_eps
            rotation.update(q_weight=self.q_norm_weight, k_weight=self.k_norm_weight, whole=True)
        k.unit_norm_write(projected, self.q_heads, self.kv_heads, self.dim, self.vdim, eps,
                          meta.slot_map if writes_cache else None, cache.k, cache.v, q, at=at, **rotation)
        more = {"sink_logits": self.sink_logits} if self.learned_sink else {}
        if self.keep_first:
            more["keep_first"] = self.keep_first
        k.gated_attention(q, cache.k, cache.v, projected if self.head_gate else None,
                          at + self.q_size + self.k_size + self.v_size, ctx, meta, self.q_heads, self.kv_heads, self.dim,
                          self.vdim, self.scale, self.softcap, self.chunk, self.window, self.sink, out, out_at=out_at,
                          out_scale=out_scale, **more)

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        tokens, dtype = x.shape[0], self.rt.dtype
        projected = ctx.arena.take((tokens, self.width), dtype)
        self.qkvg.forward(x, projected)
        merged = ctx.arena.take((tokens, self.q_heads * self.vdim), dtype)
        self.attend_columns(projected, 0, ctx, cache, writes_cache, merged, 0, 1.0)
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.out.forward(merged, out)


register_part("mixer", "gated_attention", GatedAttention)
