"""Retention: linear attention with a fixed decay per head and neither softmax nor denominator.

    q = W_q h, k = W_k h (heads x head_dim), v = W_v h (heads x value_dim), no biases
    q and k are rotated by position over their first `rotary_dims` dimensions (dimension i with i + rotary_dims / 2,
    angle position * base^(-2i / rotary_dims)); k is then multiplied by `key_scale` (head_dim^(-1/2) unless given)
    per head:  S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t         (S [head_dim, value_dim], from zero)
    out = W_o (concat_h(o_h / rms(o_h)) * silu(W_g h))

Options, for other designs of the same recurrence: `input_activation="silu"` - q, k and v pass silu before anything
else; `norm="all_heads"` - the heads' outputs are normed together, o / rms(o over all heads) times a weight per value
(tensor `norm`), instead of head by head without a weight; `gate="sigmoid"` - the gate is sigmoid(W_g h) instead of
silu(W_g h).

What a request carries between steps is S of every head, float32, in its slot.  Angles, the rotation, the state, its
sums and the unit norm are float32; the four projections are one product.
"""

from __future__ import annotations

import numpy as np
import torch

from ..weights.spec import NORM, TensorSpec
from .base import Part, SharesProducts, SlotState, register_part
from .linear import Linear


class Retention(Part, SharesProducts):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.heads, self.dim, self.vdim = int(spec["heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        self.rot_dims, self.base = int(spec.get("rotary_dims") or 0), float(spec.get("rotary_base") or 0.0)
        self.eps = float(spec["eps"])
        self.key_scale = float(spec["key_scale"]) if spec.get("key_scale") is not None else self.dim ** -0.5
        decay = [float(d) for d in spec["decay"]]
        self.name = spec.get("name", "retention")
        self.input_activation = spec.get("input_activation")
        self.norm_over, self.gate = spec.get("norm", "per_head"), spec.get("gate", "silu")
        if self.input_activation not in (None, "silu"):
            raise ValueError(f"the inputs pass 'silu' or nothing, not {self.input_activation!r}")
        if self.norm_over not in ("per_head", "all_heads") or self.gate not in ("silu", "sigmoid"):
            raise ValueError(f"norm is 'per_head' or 'all_heads' and gate 'silu' or 'sigmoid', not {self.norm_over!r}, {self.gate!r}")
        # the recurrence's own kernel norms head by head and gates with silu; anything else is a kernel after it
        self.finishes_itself = self.norm_over == "per_head" and self.gate == "silu"
        self.norm_weight = None
        if len(decay) != self.heads:
            raise ValueError(f"{self.heads} heads need {self.heads} decays, got {len(decay)}")
        if self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ValueError(f"rotary_dims must be even and at most head_dim {self.dim}, got {self.rot_dims}")
        names = dict(q="q", k="k", v="v", g="g", o="o", norm="norm")
        names.update(spec.get("names") or {})
        qk, vs = self.heads * self.dim, self.heads * self.vdim
        self.qkvg = self.inputs = Linear(runtime, self.hidden, [qk, qk, vs, vs], [names["q"], names["k"], names["v"], names["g"]])
        self.out = self.outputs = Linear(runtime, vs, [self.hidden], [names["o"]])
        self.norm_name = names["norm"]
        self.decay = torch.tensor(decay, dtype=torch.float32, device=runtime.device)
        self.table = None
        if self.rot_dims:
            # the frequencies rounded once from double precision; cos and sin of every position the engine can reach,
            # float32 [max_seq_len, rotary_dims / 2, 2], one table for all layers with the same constants
            half = self.rot_dims // 2
            reach = (runtime.max_seq_len + runtime.page_size - 1) // runtime.page_size * runtime.page_size     # whole pages
            freq = torch.from_numpy((self.base ** (-2.0 * np.arange(half, dtype=np.float64) / self.rot_dims)).astype(np.float32))
            self.table = runtime.shared_buffer(
                ("rotary_first_dims", self.rot_dims, self.base, reach), (reach, half, 2), torch.float32,
                lambda table: runtime.kernels.rope_table(freq.to(runtime.device), table))
        runtime.kernels.check_retention_sizes(self.heads, self.dim, self.vdim)

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _norm_spec(self, p):
        return [TensorSpec(p + self.norm_name, (self.heads * self.vdim,), NORM)] if self.norm_over == "all_heads" else []

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.qkvg.tensors(p) + self.out.tensors(p) + self._norm_spec(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.qkvg.load(fetch, p)
        self.out.load(fetch, p)
        if self.norm_over == "all_heads":
            self.norm_weight = fetch(self._norm_spec(p)[0]).to(torch.float32).contiguous()

    def weight_bytes(self):
        return self.qkvg.weight_bytes() + self.out.weight_bytes()

    def cache_request(self):
        return SlotState((self.heads * self.dim * self.vdim,), torch.float32)

    def attend_columns(self, projected, at, ctx, cache, writes_cache, out, out_at, out_scale):
        """The heads' normed outputs times silu(W_g h), before W_o, from this mixer's columns of a projection."""
        k = self.rt.kernels
        more = {"input_activation": self.input_activation} if self.input_activation is not None else {}
        if self.finishes_itself:
            k.retention(projected, self.heads, self.dim, self.vdim, self.rot_dims, self.table, self.key_scale,
                        self.decay, self.eps, cache.state, ctx, out, at=at, out_at=out_at, out_scale=out_scale, **more)
            return
        width = self.heads * self.vdim
        raw = ctx.arena.take((projected.shape[0], width), torch.float32)
        k.retention(projected, self.heads, self.dim, self.vdim, self.rot_dims, self.table, self.key_scale,
                    self.decay, self.eps, cache.state, ctx, None, at=at, raw=raw, **more)
        if self.norm_over == "all_heads":
            k.norm_gate_rows(raw, self.norm_weight, self.eps, projected, at + 2 * self.heads * self.dim + width, self.gate,
                             out, out_at=out_at, out_scale=out_scale)
            return
        for head in range(self.heads):      # (head by head without a weight, another gate: a launch a head)
            k.norm_gate_rows(raw, None, self.eps, projected, at + 2 * self.heads * self.dim + width + head * self.vdim,
                             self.gate, out, out_at=out_at + head * self.vdim, out_scale=out_scale, x_at=head * self.vdim,
                             width=self.vdim)

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        tokens, dtype = x.shape[0], self.rt.dtype
        projected = ctx.arena.take((tokens, 2 * self.heads * (self.dim + self.vdim)), dtype)
        self.qkvg.forward(x, projected)
        gated = ctx.arena.take((tokens, self.heads * self.vdim), dtype)
        self.attend_columns(projected, 0, ctx, cache, writes_cache, gated, 0, 1.0)
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.out.forward(gated, out)


register_part("mixer", "retention", Retention)
