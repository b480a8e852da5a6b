"""The gated delta rule with a decay per key channel, behind short causal convolutions.

    q = W_q h, k = W_k h (kv_heads x head_dim), v = W_v h (heads x value_dim); head h reads q / k head h // (heads / kv_heads)
    each of q, k, v: a causal convolution over the last `taps` inputs per channel (no bias, zeros before the start), silu
    q, k <- x / sqrt(sum(x^2) + unit_eps) per head;  q <- q * head_dim^(-1/2)
    beta = sigmoid(W_b h) per head;   g = exp(-exp(A_log_h) * softplus(W_a2 (W_a1 h) + dt_bias))   (heads x head_dim)
    per head, S [head_dim, value_dim] from zero:  S <- g * S (row d times g_d);  u = beta (v - S^T k);  S <- S + k u^T;
                                                  o = S^T q            (the read-out sees the token's own write)
    out = W_o (concat_h(o_h / rms(o_h) * w) * sigmoid(W_g2 (W_g1 h)))   (w: `value_dim` weights shared by the heads)

What a request carries between steps lies in its slot as one float32 vector: S of every head (as [heads, value_dim,
head_dim]), then the convolutions' last taps - 1 inputs.  W_q, W_k, W_v, W_b, W_a1 and W_g1 are one product; the decays'
and the gates' second products leave their sums in float32; unit norms, sigmoids, softplus, exponentials, the state, its
sums and the norm of the outputs are float32.
"""

from __future__ import annotations

import torch

from ..weights.spec import BIAS, MATRIX, NORM, TensorSpec
from .base import Part, SlotState, register_part
from .linear import Linear


class GatedDeltaRule(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.heads, self.kv_heads = int(spec["heads"]), int(spec["kv_heads"])
        self.dim, self.vdim, self.taps = int(spec["head_dim"]), int(spec["value_dim"]), int(spec["taps"])
        self.decay_rank, self.gate_rank = int(spec["decay_rank"]), int(spec["gate_rank"])
        self.unit_eps, self.eps = float(spec["unit_eps"]), float(spec["eps"])
        self.name = spec.get("name", "mix")
        if self.heads % self.kv_heads:
            raise ValueError(f"heads {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.taps < 1:
            raise ValueError(f"a convolution has at least one tap, got {self.taps}")
        self.qk, self.vs = self.kv_heads * self.dim, self.heads * self.vdim
        self.conv_channels = 2 * self.qk + self.vs
        # (the convolutions' inputs first: the kernel reads the first columns of the stacked product)
        sizes = [self.qk, self.qk, self.vs, self.heads, self.decay_rank, self.gate_rank]
        self.into = Linear(runtime, self.hidden, sizes, ["q", "k", "v", "b", "a1", "g1"])
        self.beta_at = self.conv_channels
        self.decay_at, self.gate_at = self.beta_at + self.heads, self.beta_at + self.heads + self.decay_rank
        self.decay_up = Linear(runtime, self.decay_rank, [self.heads * self.dim], ["a2"])
        self.gate_up = Linear(runtime, self.gate_rank, [self.vs], ["g2"])
        self.out = Linear(runtime, self.vs, [self.hidden], ["o"])
        self.conv_weight = self.decay_bias = self.rate = self.norm_weight = None
        runtime.kernels.check_delta_rule_sizes(self.heads, self.kv_heads, self.dim, self.vdim)

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _own_specs(self, p):
        return [TensorSpec(p + "q.conv", (self.qk, self.taps), MATRIX), TensorSpec(p + "k.conv", (self.qk, self.taps), MATRIX),
                TensorSpec(p + "v.conv", (self.vs, self.taps), MATRIX), TensorSpec(p + "A_log", (self.heads,), BIAS),
                TensorSpec(p + "dt_bias", (self.heads * self.dim,), BIAS), TensorSpec(p + "norm", (self.vdim,), NORM)]

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return (self.into.tensors(p) + self.decay_up.tensors(p) + self.gate_up.tensors(p) + self.out.tensors(p)
                + self._own_specs(p))

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        for linear in (self.into, self.decay_up, self.gate_up, self.out):
            linear.load(fetch, p)
        q_conv, k_conv, v_conv, a_log, dt_bias, norm = (fetch(spec) for spec in self._own_specs(p))
        self.conv_weight = torch.cat((q_conv, k_conv, v_conv), dim=0).contiguous()
        self.rate = torch.exp(a_log.to(torch.float32)).contiguous()
        self.decay_bias = dt_bias.to(torch.float32).contiguous()
        self.norm_weight = norm.to(torch.float32).contiguous()

    def weight_bytes(self):
        return sum(linear.weight_bytes() for linear in (self.into, self.decay_up, self.gate_up, self.out))

    def cache_request(self):
        return SlotState((self.heads * self.dim * self.vdim + (self.taps - 1) * self.conv_channels,), torch.float32)

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        projected = ctx.arena.take((tokens, self.into.total_out), dtype)
        self.into.forward(x, projected)
        conv = ctx.arena.take((tokens, self.conv_channels), dtype)
        k.conv_silu(projected, self.conv_channels, self.conv_weight, None, cache.state, 0, ctx, conv,
                    conv_at=self.heads * self.dim * self.vdim)
        # the two low-rank branches' second products, their sums left in float32
        low = ctx.arena.take((tokens, self.decay_rank), dtype)
        k.copy_heads(projected[:, self.decay_at:self.decay_at + self.decay_rank].unsqueeze(1), low.view(tokens, 1, -1))
        decay_logits = ctx.arena.take((tokens, self.heads * self.dim), torch.float32)
        self.decay_up.forward(low, decay_logits)
        low = ctx.arena.take((tokens, self.gate_rank), dtype)
        k.copy_heads(projected[:, self.gate_at:self.gate_at + self.gate_rank].unsqueeze(1), low.view(tokens, 1, -1))
        gates = ctx.arena.take((tokens, self.vs), torch.float32)
        self.gate_up.forward(low, gates)
        gated = ctx.arena.take((tokens, self.vs), dtype)
        k.delta_rule(conv, projected, self.beta_at, decay_logits, self.decay_bias, self.rate, gates, self.norm_weight,
                     self.unit_eps, self.eps, self.dim ** -0.5, self.heads, self.kv_heads, self.dim, self.vdim, cache.state,
                     ctx, gated)
        return self.out.forward(gated, ctx.arena.take((tokens, self.hidden), dtype))


register_part("mixer", "gated_delta_rule", GatedDeltaRule)
