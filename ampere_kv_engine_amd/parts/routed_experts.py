"""A routed feed-forward: `experts` small feed-forwards of which every token uses `top`.

Two laws of choosing and weighting (`weights`):
    "softmax_all"     scores = softmax(W_r h) over all experts (float32); experts form `groups` equal groups of
                      neighbours; a group's score is its best expert's; only experts of the `groups_kept` best groups can
                      be chosen; the `top` best of those are, weighted by their own scores as they are.
    "softmax_chosen"  logits = W_r h (+ b_r); the `top` experts with the largest logits are chosen and weighted by the
                      softmax over their logits alone.
    "sigmoid_chosen"  scores = sigmoid(W_r h); the `top` experts with the largest scores are chosen and weighted by their
                      own scores as they are.
Forms of an expert (`activation`), none with biases:
    "relu_squared"    W_down relu(W_up h)^2
    "silu_gated"      W_down (silu(W_gate h) * (W_up h))
    "gelu"            W_down gelu(W_up h), the exact (erf) gelu
With `weight_on_input` the router's weight multiplies what the expert reads, not what it returns: expert(w h) - for an
expert without biases that is the activation of w (W_up h).
With `shared_size`, one more expert of that width which every token uses, added to the chosen experts' weighted sum -
weighted by sigmoid(w_sg . h), one number a token (`shared_gate`, the default), or as it is.

The experts' first matrices are stacked into one [experts * ff (+ shared), hidden] (gates, then ups, where an expert
has both) and their second ones side by side into one [hidden, experts * ff (+ shared)]: a step is the router (the
shared expert's gate is one more row of it), one product, the activation times the router's weight - exact zeros
for experts a token did not choose - and one product whose sum over all columns IS the weighted sum over the chosen
experts and the shared one.  Every launch depends on the step's shape alone (a recorded step replays it), and a
token's result on nothing but the token.
"""

from __future__ import annotations

import torch

from ..weights.spec import MATRIX, TensorSpec
from .base import Part, register_part
from .linear import Linear

ACTIVATIONS = ("relu_squared", "silu_gated", "gelu")
WEIGHTS = ("softmax_all", "softmax_chosen", "sigmoid_chosen")


class RoutedExperts(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden, self.ff = int(spec["hidden_size"]), int(spec["expert_size"])
        self.experts, self.top = int(spec["experts"]), int(spec["top"])
        self.groups, self.kept = int(spec.get("groups", 1)), int(spec.get("groups_kept", 1))
        self.activation = spec.get("activation", "relu_squared")
        self.weights = spec.get("weights", "softmax_all")
        self.shared = int(spec["shared_size"]) if spec.get("shared_size") else 0
        self.name = spec.get("name", "mlp")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"activation {self.activation!r} is not one of {ACTIVATIONS}")
        if self.weights not in WEIGHTS:
            raise ValueError(f"weights {self.weights!r} is not one of {WEIGHTS}")
        if self.experts % self.groups or not 0 < self.kept <= self.groups:
            raise ValueError(f"{self.experts} experts do not form {self.groups} equal groups of which {self.kept} are kept")
        if not 0 < self.top <= self.kept * (self.experts // self.groups):
            raise ValueError(f"{self.top} experts a token cannot be chosen from {self.kept} groups of {self.experts // self.groups}")
        if self.weights != "softmax_all" and self.groups != 1:
            raise ValueError("weights over the chosen experts alone know no groups")
        self.inside = bool(spec.get("weight_on_input", False))
        self.shared_gate = bool(spec.get("shared_gate", True)) and bool(self.shared)
        # which kernels take the step: the gated pair of Tukevik's experts, or one activation with the weight in or outside
        self.plain = self.activation == "gelu" or self.inside or self.weights == "sigmoid_chosen"
        if self.plain and (self.activation == "silu_gated" or self.weights != "sigmoid_chosen" or self.shared_gate):
            raise ValueError("experts weighted by their sigmoid scores are ungated, and so is the expert they share")
        if not self.plain and self.shared and (self.weights != "softmax_chosen" or self.activation != "silu_gated"):
            raise ValueError("a shared expert behind a gate comes with gated experts weighted by the softmax over the chosen")
        self.gated = self.activation == "silu_gated"
        first = [f"e{e}.up" for e in range(self.experts)] + (["shared.up"] if self.shared else [])
        sizes = [self.ff] * self.experts + ([self.shared] if self.shared else [])
        if self.gated:
            first = [name[:-2] + "gate" for name in first] + first
            sizes = sizes + sizes
        self.columns = self.experts * self.ff + self.shared
        self.up = Linear(runtime, self.hidden, sizes, first)
        self.down = Linear(runtime, self.columns, [self.hidden], ["down"])     # (adopted at load: side by side)
        # the router's logits are a product like any other, with float32 sums left as they are: what the file stores in
        # 16 bits is exact in the operands, so nothing of the logits is formed in less than 32 bits
        bias = "router.b" if spec.get("router_bias", False) else None
        if self.shared_gate:
            self.router = Linear(runtime, self.hidden, [self.experts, 1], ["router", "shared.sg"],
                                 bias_names=[bias, None] if bias else None)
        else:
            self.router = Linear(runtime, self.hidden, [self.experts], ["router"], bias_names=[bias] if bias else None)

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _down_specs(self, p):
        specs = [TensorSpec(f"{p}e{e}.down", (self.hidden, self.ff), MATRIX, library_copy=True) for e in range(self.experts)]
        if self.shared:
            specs.append(TensorSpec(f"{p}shared.down", (self.hidden, self.shared), MATRIX, library_copy=True))
        return specs

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.up.tensors(p) + self._down_specs(p) + self.router.tensors(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.up.load(fetch, p)
        self.down.adopt(torch.cat([fetch(spec) for spec in self._down_specs(p)], dim=1).contiguous())
        self.router.load(fetch, p)

    def weight_bytes(self):
        return self.up.weight_bytes() + self.down.weight_bytes() + self.router.weight_bytes()

    def forward(self, x, ctx):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        scored = self.experts + (1 if self.shared else 0)
        if self.plain:
            logits = ctx.arena.take((tokens, self.experts), torch.float32)
            self.router.forward(x, logits)
            gates = ctx.arena.take((tokens, scored), torch.float32)
            k.route_chosen(logits, gates, self.experts, self.top, law="sigmoid")      # (the shared expert's gate is 1)
            up = ctx.arena.take((tokens, self.columns), dtype)
            self.up.forward(x, up)
            act = ctx.arena.take((tokens, self.columns), dtype)
            k.gate_activation(up, gates, act, self.experts, self.ff, self.activation, self.inside)
            return self.down.forward(act, ctx.arena.take((tokens, self.hidden), dtype))
        logits = ctx.arena.take((tokens, scored), torch.float32)
        self.router.forward(x, logits)
        gates = ctx.arena.take((tokens, scored), torch.float32)
        if self.weights == "softmax_all":
            k.route(logits, gates, self.top, self.groups, self.kept)
        else:
            k.route_chosen(logits, gates, self.experts, self.top)
        up = ctx.arena.take((tokens, self.columns * (2 if self.gated else 1)), dtype)
        self.up.forward(x, up)
        act = ctx.arena.take((tokens, self.columns), dtype)
        if self.gated:
            k.gate_silu_mul(up, gates, act, self.experts, self.ff)
        else:
            k.gate_relu_squared(up, gates, act)
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.down.forward(act, out)


register_part("feed_forward", "routed_experts", RoutedExperts)
