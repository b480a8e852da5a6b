"""A test double for the engine's kernel set, written with plain torch operations.

It exists so that the host side of the engine (batch layout, block tables, page reuse, scheduling, replay)
can be exercised where there is no GPU.  It is handed to `Engine(..., kernels=TorchKernels())` by tests only;
the product never constructs it and has no fallback to it.  Each method states the contract of the HIP
kernel of the same name; the GPU tests hold the HIP kernels to these same contracts.
"""

from __future__ import annotations

import math

import numpy as np
import torch

from ampere_kv_engine_amd.parts.base import KernelSet


def _round(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    return x.to(dtype)


class TorchKernels(KernelSet):
    name = "torch-double"

    def __init__(self, fold_rows: int = 0, fold_many_rows: int = 0, rows_left: bool = False):
        """`fold_rows`: steps of up to this many rows let a branch's last product add itself to the residual sum and
        the next product norm its rows from the sums of squares left there, as the HIP kernel set does in decode
        steps (0: never).  `fold_many_rows`: steps of more rows, up to this many, do the same the way the HIP
        kernel set's mid-size products do: the adding product leaves the new rows times the next norm's weight, and
        the reading product divides its results by the rows' root mean square."""
        self.fold_rows = fold_rows
        self.fold_many_rows = fold_many_rows
        # steps of up to `fold_rows` rows too: the adding product leaves the rows times the next norm's weight where it
        # is told that weight, and the reader scales its results (what the HIP kernel set's decode products do)
        self.rows_left = rows_left

    def check_attention_sizes(self, q_heads, kv_heads, head_dim, page_size):
        if q_heads % kv_heads:
            raise ValueError("q_heads must be a multiple of kv_heads")

    # ---- token-wise ------------------------------------------------------------------------------------
    def embed(self, ids, table, out, ctx=None):
        """An id of -1 stands for the token chosen last for the row's request (word 1 of its slot)."""
        ids = ids.long().clone()
        words = getattr(ctx, "slot_words", None) if ctx is not None else None
        if words is not None:
            last = words[ctx.seq_slots.long()[ctx.seq_of_token.long()], 1].long()
            ids = torch.where(ids == -1, last, ids)
        out.copy_(table[ids].float())

    def step_prologue(self, ctx):
        """state[offset] = value for the step's (offset, value) pairs; word 0 of every request's slot = its length."""
        count = int(ctx.patch_count[0])
        assert count <= ctx.patch_room
        pairs = ctx.patches[:2 * count].view(count, 2).long()
        ctx.slot_state[pairs[:, 0]] = pairs[:, 1].int()
        ctx.slot_words[ctx.seq_slots.long(), 0] = ctx.seq_lens

    def add_rmsnorm(self, stream, delta, weight, eps, out):
        if delta is not None:
            stream += delta.float()
        normed = stream * torch.rsqrt((stream * stream).mean(-1, keepdim=True) + eps)
        out.copy_(_round(_round(normed, out.dtype).float() * weight, out.dtype))

    def rmsnorm(self, x, weight, eps, out):
        xf = x.float()
        normed = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
        out.copy_(_round(_round(normed, out.dtype).float() * weight, out.dtype))

    def rmsnorm_heads(self, x, weight, eps, out):
        self.rmsnorm(x, weight, eps, out)

    def copy_heads(self, x, out):
        out.copy_(x)

    def gather_rows(self, stream, pending, rows, out):
        picked = stream[rows.long()]
        if pending is not None:
            picked = picked + pending[rows.long()].float()
        out.copy_(picked)

    def prepare_linear(self, matrix):
        return matrix

    def linear(self, x, weight, out, bias=None):
        y = x.float() @ weight.float().T
        out.copy_((y if bias is None else y + bias.float()).to(out.dtype))

    def prepare_gated_linear(self, gate, up):
        return (gate, up)

    # ---- the residual sum and the norm inside the products (decode steps) -------------------------------
    def folds_norm(self, rows, hidden, dtype):
        return 0 < rows <= max(self.fold_rows, self.fold_many_rows) and dtype == torch.bfloat16

    def adds_to_stream(self, rows, weight, dtype, gain=None):
        if not isinstance(weight, torch.Tensor) or dtype != torch.bfloat16:
            return False
        if 0 < rows <= self.fold_rows:
            return True
        return gain is not None and rows <= self.fold_many_rows

    def add_to_stream(self, x, weight, stream, arena, bias=None, gain=None):
        from ampere_kv_engine_amd.parts.base import StreamSums
        rows, outs = x.shape[0], weight.shape[0]
        if rows <= self.fold_rows:
            sums = arena.take(((outs + 15) // 16, 16), torch.float32)
            self.linear_adds(x, weight, stream, sums, bias=bias)
            if not self.rows_left or gain is None:
                return StreamSums(sums)
            left = arena.take((rows, outs), x.dtype)
            left.copy_((stream * gain).to(x.dtype))
            return StreamSums(sums, rows=left, gain=gain)
        # many rows: the new rows times the next norm's weight, and three groups of partial sums per row
        y = torch.empty(rows, outs, dtype=x.dtype)
        self.linear(x, weight, y, bias)
        stream += y.float()
        sums = arena.take((3, (rows + 15) // 16 * 16), torch.float32)
        sums.zero_()
        for group, columns in enumerate(torch.arange(outs).chunk(3)):
            sums[group, :rows] = (stream[:, columns] ** 2).sum(-1)
        left = arena.take((rows, outs), x.dtype)
        left.copy_((stream * gain).to(x.dtype))
        return StreamSums(sums, rows=left, gain=gain)

    def scales_rows_in_product(self, rows, weight, dtype, sums):
        return sums.rows is not None and 0 < rows <= max(self.fold_rows, self.fold_many_rows) and dtype == torch.bfloat16

    def linear_rowscaled(self, x, sums, eps, weight, out, bias=None):
        rows, k = x.shape
        scale = torch.rsqrt(sums.sum(0)[:rows, None] / k + eps)
        if isinstance(weight, tuple):
            g, u = x.float() @ weight[0].float().T * scale, x.float() @ weight[1].float().T * scale
            out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))
        else:
            y = x.float() @ weight.float().T * scale
            out.copy_((y if bias is None else y + bias.float()).to(out.dtype))

    def norms_rows_in_product(self, rows, weight, dtype):
        matrix = weight[0] if isinstance(weight, tuple) else weight
        return isinstance(matrix, torch.Tensor) and self.folds_norm(rows, matrix.shape[1], dtype)

    def linear_adds(self, x, weight, stream, sums, bias=None):
        y = torch.empty(x.shape[0], weight.shape[0], dtype=x.dtype)
        self.linear(x, weight, y, bias)
        stream += y.float()
        rows, outs = stream.shape
        padded = torch.zeros(rows, sums.shape[0] * 16)
        padded[:, :outs] = stream
        sums.zero_()
        sums[:, :rows] = (padded * padded).view(rows, -1, 16).sum(-1).T

    def linear_scaled(self, stream, sums, norm_weight, eps, weight, out, bias=None):
        rows, k = stream.shape
        scale = torch.rsqrt(sums.sum(0)[:rows, None] / k + eps)
        normed = _round(_round(stream * scale, out.dtype).float() * norm_weight, out.dtype)
        if isinstance(weight, tuple):
            self.gated_linear(normed, weight, out)
        else:
            self.linear(normed, weight, out, bias)

    def gated_scratch(self, weight, rows, dtype):
        return None

    def gated_linear(self, x, weight, out, scratch=None):
        g, u = x.float() @ weight[0].float().T, x.float() @ weight[1].float().T
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    def swiglu(self, gate_up, out):
        inter = out.shape[-1]
        g, u = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    # ---- position ----------------------------------------------------------------------------------------
    def rope_table(self, inv_freq, table):
        positions = torch.arange(table.shape[0], dtype=torch.float32, device=table.device)
        angles = positions[:, None] * inv_freq[None, :].float()
        table[..., 0] = angles.cos()
        table[..., 1] = angles.sin()

    def _rotate(self, x, positions, table):
        half = x.shape[-1] // 2
        cs = table[positions.long()]                      # [N, d/2, 2]
        cos, sin = cs[:, None, :, 0], cs[:, None, :, 1]
        lo, hi = x[..., :half].float(), x[..., half:].float()
        return torch.cat((lo * cos - hi * sin, hi * cos + lo * sin), dim=-1)

    def rope(self, x, positions, table):
        x.copy_(self._rotate(x, positions, table).to(x.dtype))

    # ---- cache ---------------------------------------------------------------------------------------------
    def kv_write(self, k, v, slot_map, k_pages, v_pages):
        pages, kv_heads, page_size, d = k_pages.shape
        slots = slot_map.long()
        k_pages[slots // page_size, :, slots % page_size] = k          # keys   [pages, kv_heads, page_size, d]
        v_pages[slots // page_size, :, :, slots % page_size] = v       # values [pages, kv_heads, d, page_size]

    def qk_norm_rope_write(self, qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages,
                           q_out, q_heads, kv_heads, head_dim):
        n = qkv.shape[0]
        q_size, kv_size = q_heads * head_dim, kv_heads * head_dim
        q = qkv[:, :q_size].reshape(n, q_heads, head_dim).float()
        k = qkv[:, q_size:q_size + kv_size].reshape(n, kv_heads, head_dim).float()
        v = qkv[:, q_size + kv_size:].reshape(n, kv_heads, head_dim)
        dtype = qkv.dtype
        if q_weight is not None:
            q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps)
            q = _round(q, dtype).float() * q_weight
            k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps)
            k = _round(k, dtype).float() * k_weight
        if table is not None:
            q = self._rotate(_round(q, dtype), positions, table)
            k = self._rotate(_round(k, dtype), positions, table)
        q_out.copy_(q.reshape(n, q_size).to(dtype))
        if slot_map is not None:
            self.kv_write(k.to(dtype), v, slot_map, k_pages, v_pages)

    def encode_and_attend(self, qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q, ctx,
                          meta, q_heads, kv_heads, head_dim, scale, window, out):
        self.qk_norm_rope_write(qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q,
                                q_heads, kv_heads, head_dim)
        self.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out)

    def attention(self, q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out):
        page_size = k_pages.shape[2]
        group = q_heads // kv_heads
        table = meta.block_table.cpu()
        if getattr(meta, "rows", None) is not None:          # the persistent table: a row per slot
            table = table[meta.rows.cpu().long()]
        for r in range(ctx.num_seqs):
            first, last = ctx.host_q_start[r], ctx.host_q_start[r + 1]
            length = ctx.host_seq_lens[r]
            history = length - (last - first)
            lowest = 0 if window is None else max(0, history - window + 1)
            key_pos = torch.arange(lowest, length)
            pages = table[r][key_pos // page_size].long()
            assert (pages >= 0).all(), "attention would read a page that was given back"
            keys = k_pages[pages, :, key_pos % page_size].float()        # [S, kv_heads, d]
            values = v_pages[pages, :, :, key_pos % page_size].float()
            qs = q[first:last].reshape(last - first, q_heads, head_dim).float()
            q_pos = history + torch.arange(last - first)
            visible = key_pos[None, :] <= q_pos[:, None]
            if window is not None:
                visible &= key_pos[None, :] > q_pos[:, None] - window
            merged = torch.empty_like(qs)
            for head in range(q_heads):          # a head at a time: long histories' scores of all heads need not fit
                scores = (qs[:, head] @ keys[:, head // group].T) * scale
                scores = scores.masked_fill(~visible, -math.inf)
                merged[:, head] = scores.softmax(-1) @ values[:, head // group]
            out[first:last] = merged.reshape(last - first, q_heads * head_dim).to(out.dtype)

    # ---- designs with float32 norms: pair embedding, norm before and after, latent attention, scan, routing ------------
    def embed_pairs(self, ids, table, pairs, buckets, mul_prev, mul_cur, out, ctx):
        """out[n] = table[id] + pairs[row]; row = (previous * mul_prev + id * mul_cur) mod buckets, `buckets` at position
        0; the previous id of a portion's first token is word 7 of the request's slot, which then takes the portion's
        last id."""
        words = ctx.slot_words
        slots = ctx.seq_slots.long()[ctx.seq_of_token.long()]
        cur = ids.long().clone()
        cur = torch.where(cur == -1, words[slots, 1].long(), cur)
        prev = torch.roll(cur, 1)
        starts = ctx.q_start.long()[:-1]
        prev[starts] = words[ctx.seq_slots.long(), 7].long()
        rows = (prev * mul_prev + cur * mul_cur) % buckets
        rows = torch.where(ctx.positions.long() == 0, torch.full_like(rows, buckets), rows)
        out.copy_(table[cur].float() + pairs[rows].float())
        words[ctx.seq_slots.long(), 7] = cur[ctx.q_start.long()[1:] - 1].int()

    def norm_add_norm(self, stream, delta, post_weight, post_eps, pre_weight, pre_eps, out, delta_scale=1.0, offset=None,
                      delta2=None):
        if delta is not None:
            d = (delta.float() + delta2.float() if delta2 is not None else delta.float()) * delta_scale
            if post_weight is not None:
                d = d * torch.rsqrt((d * d).mean(-1, keepdim=True) + post_eps) * post_weight
            stream += d
        if offset is not None:
            stream += offset
        if out is not None:
            out.copy_((stream * torch.rsqrt((stream * stream).mean(-1, keepdim=True) + pre_eps) * pre_weight).to(out.dtype))

    def embed_add(self, ids, table, out, ctx=None):
        """out[n] += table[id]; an id of -1 is the token chosen last for the row's request."""
        rows = torch.empty_like(out)
        self.embed(ids, table, rows, ctx)
        out += rows

    def norm_gate_rows(self, x, weight, eps, gates, gate_at, gate, out, out_at=0, out_scale=1.0, x_at=0, width=None):
        width = x.shape[1] - x_at if width is None else width
        v = x[:, x_at:x_at + width].float()
        if eps is not None:
            v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps)
        if weight is not None:
            v = v * weight
        if gate is not None:
            g = gates[:, gate_at:gate_at + width].float()
            v = v * (torch.sigmoid(g) if gate == "sigmoid" else g * torch.sigmoid(g))
        out[:, out_at:out_at + width] = (v * out_scale).to(out.dtype)

    def embed_normed(self, ids, table, weight, eps, out, ctx=None):
        """out[n] = table[id] / rms(table[id]) * weight; an id of -1 is the token chosen last for the row's request."""
        self.embed(ids, table, out, ctx)
        out.copy_(out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps) * weight)

    def gated_activation(self, gate_up, out, activation):
        inter = out.shape[1]
        gate, up = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        if activation == "gelu_tanh":
            act = 0.5 * gate * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (gate + 0.044715 * gate ** 3)))
        else:
            act = gate * torch.sigmoid(gate)
        out.copy_((act * up).to(out.dtype))

    def difference_norm_gate(self, maps, lam, eps, after, gates, gate_at, heads, vdim, out):
        n = maps.shape[0]
        both = maps.float().view(n, heads, 2, vdim)
        o = both[:, :, 0] - lam.float() * both[:, :, 1]
        o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * after
        gate = torch.sigmoid(gates[:, gate_at:gate_at + heads * vdim].float()).view(n, heads, vdim)
        out.copy_((o * gate).reshape(n, heads * vdim).to(out.dtype))

    def check_delta_rule_sizes(self, heads, groups, dim, vdim):
        assert heads % groups == 0

    def delta_rule(self, conv, beta_logits, beta_at, decay_logits, decay_bias, rate, gates, norm_weight, unit_eps, norm_eps,
                   q_scale, heads, groups, dim, vdim, state, ctx, out):
        """S of a request lies at the start of its slot as [heads, vdim, dim]."""
        n = conv.shape[0]
        x = conv.float()
        qk = groups * dim
        q, k = x[:, :qk].reshape(n, groups, dim), x[:, qk:2 * qk].reshape(n, groups, dim)
        v = x[:, 2 * qk:].reshape(n, heads, vdim)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * q_scale
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)
        share = heads // groups
        q, k = q.repeat_interleave(share, dim=1), k.repeat_interleave(share, dim=1)
        beta = torch.sigmoid(beta_logits[:, beta_at:beta_at + heads].float())
        g = torch.exp(-rate[None, :, None] * torch.nn.functional.softplus(
            (decay_logits + decay_bias).view(n, heads, dim), threshold=20.0))
        for r in range(ctx.num_seqs):
            first, last, slot = ctx.host_q_start[r], ctx.host_q_start[r + 1], ctx.host_seq_slots[r]
            S = state[slot, :heads * dim * vdim].view(heads, vdim, dim).transpose(1, 2).clone()      # [heads, dim, vdim]
            for t in range(first, last):
                S = g[t][:, :, None] * S
                u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
                S = S + k[t][:, :, None] * u[:, None, :]
                o = torch.einsum("hdv,hd->hv", S, q[t])
                o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + norm_eps) * norm_weight
                out[t] = (o * torch.sigmoid(gates[t].view(heads, vdim))).reshape(-1).to(out.dtype)
            state[slot, :heads * dim * vdim] = S.transpose(1, 2).reshape(-1)

    @staticmethod
    def _turn(x, positions, table, rot_dims, interleaved=False):
        """x [..., tokens, heads, rot] float: the first rot_dims dimensions rotated by the table's angles, pair i being
        dimensions (i, i + rot_dims / 2) - or (2 i, 2 i + 1) where the pairs are interleaved."""
        half = rot_dims // 2
        cos = table[positions.long(), :, 0][:, None, :]
        sin = table[positions.long(), :, 1][:, None, :]
        if interleaved:
            u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
            turned = torch.stack((u * cos - v * sin, v * cos + u * sin), dim=-1).flatten(-2)
            return torch.cat((turned, x[..., rot_dims:]), dim=-1)
        u, v = x[..., :half], x[..., half:rot_dims]
        return torch.cat((u * cos - v * sin, v * cos + u * sin, x[..., rot_dims:]), dim=-1)

    def latent_encode(self, down, q_rank, kv_rank, rot, rot_dims, q_weight, kv_weight, eps, table, positions, slot_map,
                      cq, records, latents_t=None, interleaved=False):
        d = down.float()
        ql = d[:, :q_rank]
        cq.copy_((ql * torch.rsqrt((ql * ql).mean(-1, keepdim=True) + eps) * q_weight).to(cq.dtype))
        if records is None:
            return
        c = d[:, q_rank:q_rank + kv_rank]
        c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * kv_weight
        key = self._turn(d[:, None, q_rank + kv_rank:q_rank + kv_rank + rot], positions, table, rot_dims, interleaved)[:, 0]
        flat = records.view(-1, kv_rank + rot)
        flat[slot_map.long()] = torch.cat((c, key), dim=-1).to(records.dtype)

    def rotate_queries(self, q, heads, dim, rot, rot_dims, table, positions, q_abs, at, interleaved=False):
        part = q.float().view(q.shape[0], heads, dim + rot)[..., dim:]
        q_abs[..., at:at + rot] = self._turn(part, positions, table, rot_dims, interleaved)

    def heads_linear(self, x, x_width, weight, y, y_width):
        heads, ins, outs = weight.shape
        y[..., :outs] = torch.einsum("thi,hio->tho", x[..., :ins].float(), weight.float()).to(y.dtype)

    def latent_attend(self, q_abs, records, ctx, meta, heads, kv_rank, scale, window, out, latents_t=None):
        page_size = records.shape[2]
        table = meta.block_table.cpu()
        if getattr(meta, "rows", None) is not None:
            table = table[meta.rows.cpu().long()]
        positions = ctx.positions.cpu().long()
        for r in range(ctx.num_seqs):
            first, last = ctx.host_q_start[r], ctx.host_q_start[r + 1]
            for n in range(first, last):
                pos = int(positions[n])
                lowest = 0 if window is None else max(0, pos - window + 1)
                key_pos = torch.arange(lowest, pos + 1)
                pages = table[r][key_pos // page_size].long()
                assert (pages >= 0).all(), "attention would read a page that was given back"
                recs = records[pages, 0, key_pos % page_size].float()           # [S, width]
                weights = ((q_abs[n] @ recs.T) * scale).softmax(-1)             # [heads, S]
                out[n] = weights @ recs[:, :kv_rank]

    def conv_silu(self, xz, channels, weight, bias, state, n_state, ctx, out, activation="silu", conv_at=None):
        taps = weight.shape[1]
        if conv_at is None:
            conv_at = channels * n_state
        conv_end = conv_at + (taps - 1) * channels
        for r in range(ctx.num_seqs):
            first, last, slot = ctx.host_q_start[r], ctx.host_q_start[r + 1], ctx.host_seq_slots[r]
            kept = state[slot, conv_at:conv_end].view(taps - 1, channels)
            seen = torch.cat((kept, xz[first:last, :channels].float()), dim=0)
            for t in range(last - first):
                acc = (seen[t:t + taps] * weight.float().T).sum(0) + (bias.float() if bias is not None else 0.0)
                out[first + t] = (acc * torch.sigmoid(acc) if activation == "silu" else acc).to(out.dtype)
            state[slot, conv_at:conv_end] = seen[seen.shape[0] - (taps - 1):].reshape(-1)

    def selective_scan(self, x, dt, bc, xz, a, d, state, taps, ctx, out):
        channels, n_state = a.shape
        dt.copy_(torch.nn.functional.softplus(dt, threshold=20.0))          # (taken in place, as the kernel does)
        for r in range(ctx.num_seqs):
            first, last, slot = ctx.host_q_start[r], ctx.host_q_start[r + 1], ctx.host_seq_slots[r]
            S = state[slot, :channels * n_state].view(channels, n_state).clone()
            for t in range(first, last):
                step = dt[t]
                xv = x[t].float()
                S = torch.exp(step[:, None] * a) * S + (step * xv)[:, None] * bc[t, None, :n_state]
                y = S @ bc[t, n_state:] + d * xv
                z = xz[t, channels:].float()
                out[t] = (y * z * torch.sigmoid(z)).to(out.dtype)
            state[slot, :channels * n_state] = S.reshape(-1)

    def route(self, logits, gates, top, groups, keep):
        scores = logits.softmax(-1)
        tokens, experts = scores.shape
        best = scores.view(tokens, groups, experts // groups).amax(-1)
        allowed = torch.zeros(tokens, groups, dtype=torch.bool)
        allowed.scatter_(1, best.topk(keep, dim=-1).indices, True)
        allowed = allowed[:, :, None].expand(tokens, groups, experts // groups).reshape(tokens, experts)
        chosen = scores.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
        gates.zero_()
        gates.scatter_(1, chosen, scores.gather(1, chosen))

    def gate_relu_squared(self, up, gates, act):
        tokens, experts = gates.shape
        u = torch.relu(up.float()).view(tokens, experts, -1) ** 2
        act.copy_((u * gates[:, :, None]).view(tokens, -1).to(act.dtype))

    # ---- attention with a softcap, chunks, a sink and a gate per head; retention; gated linear recurrence ----------------
    def check_gated_attention_sizes(self, q_heads, kv_heads, dim, vdim, page_size):
        assert q_heads % kv_heads == 0

    def check_retention_sizes(self, heads, dim, vdim):
        pass

    def unit_norm_write(self, projected, q_heads, kv_heads, dim, vdim, eps, slot_map, k_pages, v_pages, q_out, at=0, maps=1,
                        table=None, rot_dims=0, positions=None, q_weight=None, k_weight=None, whole=False, interleaved=False):
        projected = projected[:, at:]
        n = projected.shape[0]
        q_size, k_size, v_size = q_heads * maps * dim, kv_heads * maps * dim, kv_heads * vdim
        q = projected[:, :q_size].reshape(n, q_heads * maps, dim).float()
        k = projected[:, q_size:q_size + k_size].reshape(n, kv_heads * maps, dim).float()
        v = projected[:, q_size + k_size:q_size + k_size + v_size].reshape(n, kv_heads, vdim)
        if eps is not None:
            over = (-2, -1) if whole else -1        # (`whole`: one root mean square for all of a token's query vectors)
            q = q * torch.rsqrt((q * q).mean(over, keepdim=True) + eps)
            k = k * torch.rsqrt((k * k).mean(over, keepdim=True) + eps)
        if q_weight is not None:
            q = q * q_weight.view(q_heads * maps, dim)
        if k_weight is not None:
            k = k * k_weight.view(kv_heads * maps, dim)
        if table is not None:
            q, k = self._turn(q, positions, table, rot_dims, interleaved), self._turn(k, positions, table, rot_dims, interleaved)
        q_out.copy_(q.reshape(n, q_size).to(q_out.dtype))
        if slot_map is not None:
            page_size = k_pages.shape[2]
            slots = slot_map.long()
            k_pages[slots // page_size, :, slots % page_size] = k.reshape(n, kv_heads, maps * dim).to(k_pages.dtype)
            v_pages[slots // page_size, :, :, slots % page_size] = v.to(v_pages.dtype)

    def gated_attention(self, q, k_pages, v_pages, gates, gate_at, ctx, meta, q_heads, kv_heads, dim, vdim, scale, softcap,
                        chunk, window, sink, out, out_at=0, out_scale=1.0, sink_logits=None, maps=1, keep_first=0):
        """`maps` > 1: a head has `maps` query vectors; vector number m of a head reads the m-th `dim` columns of its key
        head's record and the head's values.  `sink_logits`: the sink's term is exp(sink_logits[head])."""
        page_size = k_pages.shape[2]
        q_heads = q_heads * maps          # (from here on: query vectors)
        group = q_heads // kv_heads
        table = meta.block_table.cpu()
        if getattr(meta, "rows", None) is not None:
            table = table[meta.rows.cpu().long()]
        for r in range(ctx.num_seqs):
            first, last = ctx.host_q_start[r], ctx.host_q_start[r + 1]
            length = ctx.host_seq_lens[r]
            history = length - (last - first)
            lowest = 0
            if window is not None:
                lowest = max(lowest, history - window + 1)
            if chunk is not None:
                lowest = max(lowest, history // chunk * chunk)
            key_pos = torch.arange(lowest, length)
            if keep_first and lowest > 0:       # the request's first keys stay visible behind the window
                key_pos = torch.cat((torch.arange(0, min(keep_first, lowest)), key_pos))
            pages = table[r][key_pos // page_size].long()
            assert (pages >= 0).all(), "attention would read a page that was given back"
            keys = k_pages[pages, :, key_pos % page_size].float()        # [S, kv_heads, dim]
            values = v_pages[pages, :, :, key_pos % page_size].float()   # [S, kv_heads, vdim]
            qs = q[first:last].reshape(last - first, q_heads, dim).float()
            q_pos = history + torch.arange(last - first)
            visible = key_pos[None, :] <= q_pos[:, None]
            if window is not None:
                visible &= (key_pos[None, :] > q_pos[:, None] - window) | (key_pos[None, :] < keep_first)
            if chunk is not None:
                visible &= (key_pos[None, :] // chunk) == (q_pos[:, None] // chunk)
            merged = torch.empty(last - first, q_heads, vdim)
            for head in range(q_heads):
                record = keys[:, head // group]
                scores = (qs[:, head] @ record[:, head % maps * dim:head % maps * dim + dim].T) * scale
                if softcap is not None:
                    scores = softcap * torch.tanh(scores / softcap)
                scores = scores.masked_fill(~visible, -math.inf)
                top = scores.amax(-1, keepdim=True)
                sunk = float(sink_logits[head]) if sink_logits is not None else 0.0
                if sink:
                    top = top.clamp(min=sunk)
                weights = torch.exp(scores - top)
                total = weights.sum(-1, keepdim=True) + (torch.exp(sunk - top) if sink else 0.0)
                merged[:, head] = (weights / total) @ values[:, head // group]
            if gates is not None:
                merged = merged * torch.sigmoid(gates[first:last, gate_at:gate_at + q_heads].float())[:, :, None]
            out[first:last, out_at:out_at + q_heads * vdim] = (merged.reshape(last - first, q_heads * vdim) * out_scale).to(out.dtype)

    def retention(self, projected, heads, dim, vdim, rot_dims, table, key_scale, decay, eps, state, ctx, out, at=0, out_at=0,
                  out_scale=1.0, input_activation=None, raw=None):
        n = projected.shape[0]
        qk, vs = heads * dim, heads * vdim
        p = projected[:, at:].float()
        q, k = p[:, :qk].reshape(n, heads, dim), p[:, qk:2 * qk].reshape(n, heads, dim)
        v, g = p[:, 2 * qk:2 * qk + vs].reshape(n, heads, vdim), p[:, 2 * qk + vs:2 * qk + 2 * vs]
        if input_activation == "silu":
            q, k, v = q * torch.sigmoid(q), k * torch.sigmoid(k), v * torch.sigmoid(v)
        if rot_dims:
            q, k = self._turn(q, ctx.positions, table, rot_dims), self._turn(k, ctx.positions, table, rot_dims)
        k = k * key_scale
        for r in range(ctx.num_seqs):
            first, last, slot = ctx.host_q_start[r], ctx.host_q_start[r + 1], ctx.host_seq_slots[r]
            S = state[slot].view(heads, dim, vdim).clone()
            for t in range(first, last):
                S = decay.float()[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
                o = torch.einsum("hdv,hd->hv", S, q[t])
                if raw is not None:
                    raw[t] = o.reshape(-1)
                    continue
                o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps)
                gate = g[t]
                out[t, out_at:out_at + vs] = (o.reshape(-1) * gate * torch.sigmoid(gate) * out_scale).to(out.dtype)
            state[slot] = S.reshape(-1)

    def scaled_sum(self, a, scale_a, b, scale_b, out):
        out.copy_((a.float() * scale_a + b.float() * scale_b).to(out.dtype))

    def gated_linear_scan(self, u, gates, gate_bias, rate, xy, blocks, state, taps, ctx, out):
        tokens, width = u.shape
        bw = width // blocks
        z = gates.float() + gate_bias[None]
        r = torch.sigmoid(z[..., :bw]).reshape(tokens, width)
        i = torch.sigmoid(z[..., bw:]).reshape(tokens, width)
        a = torch.exp(rate * r)
        fed = torch.sqrt(-torch.expm1(2.0 * rate * r)) * i * u.float()        # (1 - a^2, without the difference of squares)
        y = xy[:, width:].float()
        y = 0.5 * y * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (y + 0.044715 * y ** 3)))
        for s in range(ctx.num_seqs):
            first, last, slot = ctx.host_q_start[s], ctx.host_q_start[s + 1], ctx.host_seq_slots[s]
            S = state[slot, :width].clone()
            for t in range(first, last):
                S = a[t] * S + fed[t]
                out[t] = (S * y[t]).to(out.dtype)
            state[slot, :width] = S

    def route_chosen(self, logits, gates, experts, top, law="softmax"):
        values, chosen = logits[:, :experts].topk(top, dim=-1)
        gates.zero_()
        if law == "sigmoid":
            gates[:, :experts].scatter_(1, chosen, torch.sigmoid(values))
            gates[:, experts:] = 1.0
            return
        gates[:, :experts].scatter_(1, chosen, values.softmax(-1))
        if logits.shape[1] > experts:
            gates[:, experts:] = torch.sigmoid(logits[:, experts:])

    def gate_activation(self, up, gates, act, experts, ff, activation, inside):
        columns = act.shape[1]
        weight = gates[:, :experts].repeat_interleave(ff, dim=1)
        if columns > experts * ff:
            weight = torch.cat((weight, gates[:, experts:experts + 1].expand(-1, columns - experts * ff)), dim=1)
        f = {"gelu": lambda z: 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0))),
             "gelu_tanh": lambda z: 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3))),
             "silu": lambda z: z * torch.sigmoid(z),
             "relu_squared": lambda z: torch.relu(z) ** 2}[activation]
        z = up.float()
        value = f(weight * z) if inside else weight * f(z)
        act.copy_(torch.where(weight != 0, value, torch.zeros_like(value)).to(act.dtype))

    def gate_silu_mul(self, gate_up, gates, act, experts, ff):
        columns = act.shape[1]
        g, u = gate_up[:, :columns].float(), gate_up[:, columns:].float()
        weight = gates[:, :experts].repeat_interleave(ff, dim=1)
        if columns > experts * ff:
            weight = torch.cat((weight, gates[:, experts:experts + 1].expand(-1, columns - experts * ff)), dim=1)
        act.copy_((weight * (g * torch.sigmoid(g) * u)).to(act.dtype))

    # ---- sampling -----------------------------------------------------------------------------------------
    def sample(self, logits, temperature, seeds, draws, out):
        """temperature 0: the largest logit, ties to the lowest id.  Otherwise the Gumbel-max draw
        argmax(logits / t - log(-log(u))), u from Philox-4x32-10 keyed by the seed with counter (id, draw).
        A row with a NaN, or with nothing above -infinity, gives -1."""
        for row in range(logits.shape[0]):
            if torch.isnan(logits[row]).any() or not (logits[row] > -math.inf).any():
                out[row] = -1
                continue
            t = float(temperature[row]) if temperature is not None else 0.0
            scores = logits[row].double()
            if t > 0:
                seed = int(seeds[row])
                bits = philox_first(np.arange(logits.shape[1]), int(draws[row]), seed & 0xFFFFFFFF, seed >> 32)
                u = ((bits >> np.uint64(8)).astype(np.float64) + 0.5) * 2.0 ** -24
                scores = scores / t - torch.from_numpy(np.log(-np.log(u)))
            best = scores.max()
            out[row] = int((scores == best).nonzero()[0])

    def argmax(self, logits, out):
        self.sample(logits, None, None, None, out)

    def sample_slots(self, logits, ctx, out):
        """`sample` with every row's temperature (word 2, float bits), seed (words 3 and 4) and draw count (word 5)
        read from its request's slot; the chosen token goes to word 1 and the draw count rises by one."""
        words = ctx.slot_words
        slots = ctx.seq_slots.long()[ctx.seq_of_token.long()[ctx.logit_rows.long()]]
        assert len(set(slots.tolist())) == len(slots), "two wanted rows of one request"
        state = words[slots].cpu()
        temperature = state[:, 2].contiguous().view(torch.float32)
        seeds = (state[:, 3].long() & 0xFFFFFFFF) | ((state[:, 4].long() & 0xFFFFFFFF) << 32)
        chosen = torch.empty(len(slots), dtype=torch.int32)
        self.sample(logits.cpu(), temperature, seeds, state[:, 5], chosen)
        out.copy_(chosen)
        words[slots, 1] = chosen.to(words.device)
        words[slots, 5] += 1


def philox_first(c0, c1, k0, k1):
    """First output word of Philox-4x32-10 for counters (c0, c1, 0, 0) and key (k0, k1); c0 may be an array."""
    c0 = np.asarray(c0, dtype=np.uint64)
    c1 = np.full_like(c0, np.uint64(c1))
    c2, c3 = np.zeros_like(c0), np.zeros_like(c0)
    k0, k1 = np.uint64(k0), np.uint64(k1)
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0, p1 = np.uint64(0xD2511F53) * c0, np.uint64(0xCD9E8D57) * c2
        c0, c1, c2, c3 = (((p1 >> np.uint64(32)) ^ c1 ^ k0) & mask, p1 & mask,
                          ((p0 >> np.uint64(32)) ^ c3 ^ k1) & mask, p0 & mask)
        k0, k1 = (k0 + np.uint64(0x9E3779B9)) & mask, (k1 + np.uint64(0xBB67AE85)) & mask
    return c0
