"""Attention over a compressed latent, with a sliding window.

Per token the layer keeps one record [c | k_rot]: c = norm(W_dkv h)[:kv_rank] and the rotated last `rotated_dim`
outputs of the same product, a key part that every head shares.  Head h's key is [U_h c | k_rot], its value V_h c,
its query [q_h | rot(q_h')] from a latent of its own (c_q = norm(W_dq h), q = W_uq c_q).  Because keys and values are
linear in c, the heads attend the records themselves:

    score_h(i, j) = ((U_h^T q_h(i)) . c_j + rot(q_h'(i)) . k_rot(j)) * scale          out_h(i) = V_h sum_j p_j c_j

so nothing but the records is ever read from the cache, for prompts and single tokens alike.  Query i sees the keys
j with 0 <= i - j < window.  A layer may have no down-projection of its own and read another layer's records
(`own_latent = False`, with the run order naming that layer's cache); the pages are then kept for the widest window
among the readers (`cache_window`).  Norms, angles, scores, softmax weights and the weighted sums are float32.
Without a window every earlier key is seen.  `position` (a `rope_scaled` specification) replaces the plain rotation of
`rotary_base`: stretched frequencies, a factor on cos and sin, pairs in halves or interleaved.  With `gate` the heads'
outputs are multiplied, value by value, with sigmoid(W_g h) before the output product (tensor `g`, stacked with the
down-projections: it reads the same input).
"""

from __future__ import annotations

import torch

from ..config.specs import part
from ..weights.spec import MATRIX, NORM, TensorSpec
from .base import PagedKV, Part, build_part, register_part
from .linear import Linear


class LatentAttention(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.heads, self.dim, self.rot = int(spec["heads"]), int(spec["head_dim"]), int(spec["rotated_dim"])
        self.vdim, self.kv_rank, self.q_rank = int(spec["value_dim"]), int(spec["kv_rank"]), int(spec["q_rank"])
        self.scale, self.eps = float(spec["scale"]), float(spec["eps"])
        self.window = int(spec["window"]) if spec.get("window") is not None else None
        cache_window = spec.get("cache_window", self.window)
        self.cache_window = int(cache_window) if cache_window is not None else None
        if self.window is not None and (self.cache_window is None or self.cache_window < self.window) and self.window > 0:
            if self.cache_window is not None:
                raise ValueError(f"the cache keeps {self.cache_window} tokens, fewer than the window of {self.window}")
        self.rot_dims = int(spec.get("rotary_dims", self.rot))
        self.own_latent = bool(spec.get("own_latent", True))
        self.name = spec.get("name", "mix")
        if self.rot_dims % 2 or self.rot_dims > self.rot:
            raise ValueError(f"{self.rot_dims} rotated dimensions of a key part of {self.rot}: must be even and fit")
        self.record = self.kv_rank + self.rot
        down_outs, down_names = [self.q_rank], ["dq"]
        if self.own_latent:
            down_outs.append(self.record)
            down_names.append("dkv")
        self.gate = bool(spec.get("gate", False))
        if self.gate:
            down_outs.append(self.heads * self.vdim)
            down_names.append("g")
        self.down = Linear(runtime, self.hidden, down_outs, down_names)
        self.up_q = Linear(runtime, self.q_rank, [self.heads * (self.dim + self.rot)], ["uq"])
        self.out = Linear(runtime, self.heads * self.vdim, [self.hidden], ["o"])
        if spec.get("position") is not None:
            self.position = build_part("position", spec["position"], runtime)
            if self.position.dims != self.rot_dims:
                raise ValueError(f"the rotation turns {self.position.dims} dimensions, the layer says {self.rot_dims}")
        else:
            self.position = build_part("position", part("rope_half", head_dim=self.rot_dims, theta=float(spec["rotary_base"])),
                                       runtime)
        self.interleaved = bool(getattr(self.position, "interleaved", False))
        # where the kernel set has a matrix-core kernel for these sizes the layer keeps the latents twice: inside the
        # records, and once more with the keys contiguous, as that kernel's second product reads them
        # (the copy is kept by the layer that writes the records, for whichever of their readers has such a kernel:
        # `reader_heads`, the head counts of all layers that read this layer's cache)
        fits = lambda heads: bool(runtime.kernels.latent_on_matrix_cores(int(heads), self.kv_rank, self.record,
                                                                         runtime.page_size, runtime.dtype))
        self.on_matrix_cores = fits(self.heads)
        self.keeps_turned = any(fits(heads) for heads in spec.get("reader_heads", (self.heads,)))
        self.q_norm_weight = self.kv_norm_weight = None
        self.key_up = self.value_up = None      # [heads, dim, kv_rank] and [heads, kv_rank, vdim], as the per-head products read them
        self._bytes = 0

    # ---- weights --------------------------------------------------------------------------------------------------
    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _own_specs(self, p):
        specs = [TensorSpec(p + "dq.norm", (self.q_rank,), NORM),
                 TensorSpec(p + "uk", (self.heads * self.dim, self.kv_rank), MATRIX),
                 TensorSpec(p + "uv", (self.heads * self.vdim, self.kv_rank), MATRIX)]
        if self.own_latent:
            specs.append(TensorSpec(p + "dkv.norm", (self.kv_rank,), NORM))
        return specs

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.down.tensors(p) + self.up_q.tensors(p) + self.out.tensors(p) + self._own_specs(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.down.load(fetch, p)
        self.up_q.load(fetch, p)
        self.out.load(fetch, p)
        specs = self._own_specs(p)
        self.q_norm_weight = fetch(specs[0]).to(torch.float32).contiguous()
        key_up, value_up = fetch(specs[1]), fetch(specs[2])
        self.key_up = key_up.view(self.heads, self.dim, self.kv_rank).contiguous()
        self.value_up = value_up.view(self.heads, self.vdim, self.kv_rank).transpose(1, 2).contiguous()
        if self.own_latent:
            self.kv_norm_weight = fetch(specs[3]).to(torch.float32).contiguous()
        self._bytes = (self.down.weight_bytes() + self.up_q.weight_bytes() + self.out.weight_bytes()
                       + (key_up.numel() + value_up.numel()) * key_up.element_size())

    def weight_bytes(self):
        return self._bytes

    # ---- cache ------------------------------------------------------------------------------------------------------
    def cache_request(self):
        """One record per token and no values: what a head multiplies its weights with is the record's first part -
        kept a second time in the values' layout where the matrix cores read it."""
        return PagedKV(1, self.record, self.cache_window, value_dim=self.kv_rank if self.keeps_turned else 0)

    # ---- one step ---------------------------------------------------------------------------------------------------
    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        meta = ctx.paged[cache.group]
        if writes_cache != self.own_latent:
            raise ValueError("a layer writes records exactly when it has a down-projection of its own")
        if cache.k.shape[3] != self.record:
            raise ValueError(f"the cache holds records of {cache.k.shape[3]}, this layer reads {self.record}")
        down = ctx.arena.take((tokens, self.down.total_out), dtype)
        self.down.forward(x, down)
        cq = ctx.arena.take((tokens, self.q_rank), dtype)
        turned = cache.v if self.on_matrix_cores else None
        k.latent_encode(down, self.q_rank, self.kv_rank, self.rot, self.rot_dims, self.q_norm_weight, self.kv_norm_weight,
                        self.eps, self.position.table, ctx.positions, meta.slot_map, cq, cache.k if writes_cache else None,
                        latents_t=cache.v if writes_cache else None, **self._pairs())
        q = ctx.arena.take((tokens, self.heads * (self.dim + self.rot)), dtype)
        self.up_q.forward(cq, q)
        between = dtype if turned is not None else torch.float32      # the matrix cores take their queries in bfloat16
        q_abs = ctx.arena.take((tokens, self.heads, self.record), between)
        k.heads_linear(q.view(tokens, self.heads, self.dim + self.rot), self.dim + self.rot, self.key_up, q_abs, self.record)
        k.rotate_queries(q, self.heads, self.dim, self.rot, self.rot_dims, self.position.table, ctx.positions, q_abs,
                         self.kv_rank, **self._pairs())
        mixed = ctx.arena.take((tokens, self.heads, self.kv_rank), between)
        k.latent_attend(q_abs, cache.k, ctx, meta, self.heads, self.kv_rank, self.scale, self.window, mixed, latents_t=turned)
        values = ctx.arena.take((tokens, self.heads, self.vdim), dtype)
        k.heads_linear(mixed, self.kv_rank, self.value_up, values, self.vdim)
        values = values.view(tokens, self.heads * self.vdim)
        if self.gate:
            gated = ctx.arena.take((tokens, self.heads * self.vdim), dtype)
            k.norm_gate_rows(values, None, None, down, self.down.total_out - self.heads * self.vdim, "sigmoid", gated)
            values = gated
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.out.forward(values, out)

    def _pairs(self):
        return {"interleaved": True} if self.interleaved else {}


register_part("mixer", "latent_attention", LatentAttention)
