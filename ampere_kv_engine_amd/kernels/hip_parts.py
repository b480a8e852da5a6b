"""Wrappers over the second kernel library (`csrc/api_parts.h`): the token-wise kernels, mixers and routed feed-forward
of designs whose norms and residual sum are float32 throughout.  `HipKernels` inherits them; the library is compiled
and loaded when a model first asks for one of them.  As everywhere in the kernel set, shapes, dtypes, contiguity and
devices are checked on the host before a launch."""

from __future__ import annotations

import ctypes

import torch

from ..csrc.build import ensure_parts

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _long(value: int):
    return ctypes.c_long(int(value))


def _ptr_at(t, column: int):
    """Where column `column` of the first row of a dense [rows, width] tensor lies."""
    return ctypes.c_void_p(t.data_ptr() + int(column) * t.element_size())


class PartsKernels:
    """Mixed into `HipKernels` (which provides `_dense`, `_check`, `_stream`, `device`)."""

    _parts_lib = None

    def _parts(self):
        if self._parts_lib is None:
            from ..cache import slots
            from .hip import KernelError
            path = ensure_parts()
            try:
                lib = ctypes.CDLL(path)
            except OSError as error:
                raise KernelError(f"the kernel library {path} could not be loaded: {error}") from error
            for name in ("akv_embed_pairs", "akv_note_fed_tokens", "akv_norm_add_norm", "akv_latent_encode",
                         "akv_rotate_queries", "akv_heads_linear", "akv_latent_attend", "akv_latent_attend_mfma", "akv_conv_silu",
                         "akv_conv_state_update", "akv_selective_scan", "akv_route", "akv_gate_relu_squared",
                         "akv_parts_slot_layout", "akv_conv_taps", "akv_scaled_sum", "akv_unit_norm_write",
                         "akv_gated_attention_rows", "akv_gated_attention_tiles", "akv_retention", "akv_retention_chunked", "akv_gated_linear_scan", "akv_route_chosen",
                         "akv_gate_silu_mul", "akv_embed_normed", "akv_gated_activation", "akv_difference_norm_gate",
                         "akv_delta_rule", "akv_embed_rows", "akv_norm_gate_rows", "akv_gate_activation"):
                getattr(lib, name).restype = ctypes.c_int
            lib.akv_delta_rule_workspace.restype = ctypes.c_long
            layout = (ctypes.c_int * 3)()
            lib.akv_parts_slot_layout(layout)
            if tuple(layout) != (slots.SLOT_WORDS, slots.WORD_LAST_TOKEN, slots.WORD_FED_TOKEN):
                raise KernelError(f"the kernel library lays a request's slot out as {tuple(layout)} (words, last token, "
                                  "fed token); the host otherwise")
            self._parts_lib = lib
            self.parts_library_path = path
        return self._parts_lib

    def _code_of(self, t: torch.Tensor) -> int:
        from .hip import KernelError
        try:
            return _DTYPE_CODE[t.dtype]
        except KeyError:
            raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None

    def _refuse(self, message: str):
        from .hip import KernelError
        raise KernelError(message)

    def _step_arrays(self, ctx, tokens: int):
        self._dense(ctx.seq_of_token, "seq_of_token", torch.int32, (tokens,))
        self._dense(ctx.q_start, "q_start", torch.int32, (ctx.num_seqs + 1,))
        self._dense(ctx.seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
        self._dense(ctx.positions, "positions", torch.int32, (tokens,))
        if ctx.host_q_start[-1] != tokens:
            self._refuse("the step's request boundaries do not end at its last token")

    # ---- token-wise ------------------------------------------------------------------------------------------------------
    def embed_pairs(self, ids, table, pairs, buckets: int, mul_prev: int, mul_cur: int, out, ctx) -> None:
        """out[n] = table[id] + pairs[(previous id * mul_prev + id * mul_cur) mod buckets] (row `buckets` for a request's
        first token); the id a request was fed last is kept in its slot for the next step's first pair."""
        lib = self._parts()
        tokens = ids.shape[0]
        vocab, hidden = table.shape
        self._dense(ids, "ids", torch.int32, (tokens,))
        self._dense(table, "table")
        self._dense(pairs, "pairs", table.dtype, (buckets + 1, hidden))
        self._dense(out, "out", torch.float32, (tokens, hidden))
        words = getattr(ctx, "slot_words", None)
        if words is None:
            self._refuse("an embedding of token pairs needs the requests' slots (the token each was fed last)")
        self._dense(words, "slot_words", torch.int32)
        self._step_arrays(ctx, tokens)
        if max(ctx.host_seq_slots) >= words.shape[0]:
            self._refuse("a request's slot lies outside the slot words")
        self._check(lib.akv_embed_pairs(_ptr(ids), _ptr(table), _ptr(pairs), self._code_of(table), _ptr(out), tokens, hidden,
                                        vocab, _long(buckets), _long(mul_prev), _long(mul_cur), _ptr(ctx.seq_of_token),
                                        _ptr(ctx.q_start), _ptr(ctx.positions), _ptr(ctx.seq_slots), _ptr(words),
                                        self._stream()), "embed_pairs")
        self._check(lib.akv_note_fed_tokens(_ptr(ids), _ptr(ctx.q_start), _ptr(ctx.seq_slots), _ptr(words), ctx.num_seqs,
                                            self._stream()), "note_fed_tokens")

    def norm_add_norm(self, stream, delta, post_weight, post_eps, pre_weight, pre_eps, out, delta_scale: float = 1.0,
                      offset=None, delta2=None) -> None:
        """stream (float32) += delta / rms(delta) * post_weight (+= delta_scale * delta where `post_weight` is None; nothing
        where `delta` is None); then stream += offset (a float32 vector, the same on every row) where there is one; then,
        where `out` is given, out = stream / rms(stream) * pre_weight.  Float32 up to the one rounding of a stored result.
        `delta2` (beside a `delta` that is not normed): a second branch, stream += delta_scale * (delta + delta2)."""
        tokens, hidden = stream.shape
        self._dense(stream, "stream", torch.float32)
        dtype = None
        if delta is not None:
            self._dense(delta, "delta", None, (tokens, hidden))
            dtype = delta.dtype
        if delta2 is not None:
            if delta is None or post_weight is not None:
                self._refuse("a second branch comes beside a first one that is added as it is")
            self._dense(delta2, "delta2", delta.dtype, (tokens, hidden))
        if out is not None:
            self._dense(out, "out", dtype, (tokens, hidden))
            self._dense(pre_weight, "pre_weight", torch.float32, (hidden,))
            dtype = out.dtype
        if post_weight is not None:
            self._dense(post_weight, "post_weight", torch.float32, (hidden,))
        if offset is not None:
            self._dense(offset, "offset", torch.float32, (hidden,))
            dtype = dtype or torch.float32
        if dtype is None:
            return
        self._check(self._parts().akv_norm_add_norm(_ptr(stream), _ptr(delta), _ptr(post_weight), ctypes.c_float(post_eps),
                                                    _ptr(pre_weight), ctypes.c_float(pre_eps), _ptr(out), _DTYPE_CODE[dtype],
                                                    tokens, hidden, ctypes.c_float(delta_scale), _ptr(offset), _ptr(delta2),
                                                    self._stream()),
                    "norm_add_norm")

    def embed_add(self, ids, table, out, ctx=None) -> None:
        """out[n] += table[id], float32: the embedding's rows added to a residual sum that already holds something.  With
        the step's context an id of -1 is the token chosen last for the row's request."""
        tokens = ids.shape[0]
        self._dense(ids, "ids", torch.int32, (tokens,))
        self._dense(table, "table")
        vocab, hidden = table.shape
        self._dense(out, "out", torch.float32, (tokens, hidden))
        words = getattr(ctx, "slot_words", None) if ctx is not None else None
        seq_of_token = seq_slots = None
        if words is not None:
            seq_of_token, seq_slots = ctx.seq_of_token, ctx.seq_slots
            self._dense(words, "slot_words", torch.int32)
            self._dense(seq_of_token, "seq_of_token", torch.int32, (tokens,))
            self._dense(seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
            if max(ctx.host_seq_slots) >= words.shape[0]:
                self._refuse("a request's slot lies outside the slot words")
        self._check(self._parts().akv_embed_rows(_ptr(ids), _ptr(table), self._code_of(table), _ptr(out), tokens, hidden, vocab,
                                                 1, _ptr(seq_of_token), _ptr(seq_slots), _ptr(words), self._stream()),
                    "embed_add")

    GATE_ACTS = {None: 0, "sigmoid": 1, "silu": 2}

    def norm_gate_rows(self, x, weight, eps, gates, gate_at: int, gate: str | None, out, out_at: int = 0,
                       out_scale: float = 1.0, x_at: int = 0, width: int | None = None) -> None:
        """Columns x_at .. x_at + width of `x` (float32, or `out`'s dtype; default: all of them) -> columns out_at .. of
        `out`: the row divided by its root mean square over all `width` columns (eps inside the root; `eps` None: not
        normed), times `weight` (float32 [width], may be None), times sigmoid or silu (`gate`) of columns gate_at .. of
        `gates`, times `out_scale`.  Float32 up to the one rounding."""
        tokens = x.shape[0]
        self._dense(x, "x")
        self._dense(out, "out")
        if width is None:
            width = x.shape[1] - x_at
        if x.dim() != 2 or x_at < 0 or x_at + width > x.shape[1] or width <= 0:
            self._refuse(f"x must be [tokens, at least {x_at + width}], got {tuple(x.shape)}")
        if x.dtype != torch.float32 and x.dtype != out.dtype:
            self._refuse(f"x must be float32 or {out.dtype}, got {x.dtype}")
        if out.dim() != 2 or out.shape[0] != tokens or out_at < 0 or out_at + width > out.shape[1]:
            self._refuse(f"out must be [tokens, at least {out_at + width}], got {tuple(out.shape)}")
        if weight is not None:
            self._dense(weight, "weight", torch.float32, (width,))
        if gate not in self.GATE_ACTS:
            self._refuse(f"a gate is 'sigmoid', 'silu' or None, not {gate!r}")
        gate_stride = 0
        if gate is not None:
            self._dense(gates, "gates", out.dtype)
            if gates.dim() != 2 or gates.shape[0] != tokens or gate_at < 0 or gate_at + width > gates.shape[1]:
                self._refuse(f"gates must be [tokens, at least {gate_at + width}], got {tuple(gates.shape)}")
            gate_stride = gates.shape[1]
        self._check(self._parts().akv_norm_gate_rows(
            _ptr_at(x, x_at), self._code_of(x), _long(x.shape[1]), width, 0 if eps is None else 1, _ptr(weight),
            ctypes.c_float(eps if eps is not None else 0.0), _ptr_at(gates, gate_at) if gate is not None else ctypes.c_void_p(0),
            _long(gate_stride), self.GATE_ACTS[gate], _ptr_at(out, out_at), self._code_of(out), _long(out.shape[1]),
            ctypes.c_float(out_scale), _long(tokens), self._stream()), "norm_gate_rows")

    def embed_normed(self, ids, table, weight, eps: float, out, ctx=None) -> None:
        """out[n] = table[id] / rms(table[id]) * weight, float32: an embedding whose rows are normed before the first layer.
        With the step's context an id of -1 is the token chosen last for the row's request."""
        tokens = ids.shape[0]
        self._dense(ids, "ids", torch.int32, (tokens,))
        self._dense(table, "table")
        vocab, hidden = table.shape
        self._dense(weight, "weight", torch.float32, (hidden,))
        self._dense(out, "out", torch.float32, (tokens, hidden))
        words = getattr(ctx, "slot_words", None) if ctx is not None else None
        seq_of_token = seq_slots = None
        if words is not None:
            seq_of_token, seq_slots = ctx.seq_of_token, ctx.seq_slots
            self._dense(words, "slot_words", torch.int32)
            self._dense(seq_of_token, "seq_of_token", torch.int32, (tokens,))
            self._dense(seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
            if max(ctx.host_seq_slots) >= words.shape[0]:
                self._refuse("a request's slot lies outside the slot words")
        self._check(self._parts().akv_embed_normed(_ptr(ids), _ptr(table), self._code_of(table), _ptr(weight),
                                                   ctypes.c_float(eps), _ptr(out), tokens, hidden, vocab, _ptr(seq_of_token),
                                                   _ptr(seq_slots), _ptr(words), self._stream()), "embed_normed")

    GATED_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}

    def gated_activation(self, gate_up, out, activation: str) -> None:
        """out [tokens, inter] = act(gate_up[:, :inter]) * gate_up[:, inter:], in float32 with one rounding."""
        tokens, inter = out.shape
        self._dense(out, "out")
        self._dense(gate_up, "gate_up", out.dtype, (tokens, 2 * inter))
        if activation not in self.GATED_ACTIVATIONS:
            self._refuse(f"a gated feed-forward's activation is one of {sorted(self.GATED_ACTIVATIONS)}, not {activation!r}")
        self._check(self._parts().akv_gated_activation(_ptr(gate_up), _ptr(out), self._code_of(out), _long(tokens), inter,
                                                       self.GATED_ACTIVATIONS[activation], self._stream()), "gated_activation")

    def difference_norm_gate(self, maps, lam, eps: float, after: float, gates, gate_at: int, heads: int, vdim: int, out) -> None:
        """maps [tokens, heads * 2 * vdim] (per head: map 1, map 2) -> out [tokens, heads * vdim] = (a1 - lam a2) /
        rms(a1 - lam a2) * after * sigmoid(gates[:, gate_at + h * vdim + i]); `lam`: one float32 on the device."""
        tokens = maps.shape[0]
        self._dense(maps, "maps", None, (tokens, heads * 2 * vdim))
        self._dense(out, "out", maps.dtype, (tokens, heads * vdim))
        self._dense(lam, "lam", torch.float32, (1,))
        self._dense(gates, "gates", maps.dtype)
        if gates.dim() != 2 or gates.shape[0] != tokens or gate_at < 0 or gate_at + heads * vdim > gates.shape[1]:
            self._refuse(f"gates must be [tokens, at least {gate_at + heads * vdim}], got {tuple(gates.shape)}")
        self._check(self._parts().akv_difference_norm_gate(
            _ptr(maps), _ptr(lam), ctypes.c_float(eps), ctypes.c_float(after), _ptr(gates), _long(gates.shape[1]),
            _long(gate_at), _ptr(out), self._code_of(maps), _long(tokens), heads, vdim, self._stream()), "difference_norm_gate")

    def scaled_sum(self, a, scale_a: float, b, scale_b: float, out) -> None:
        """out = a * scale_a + b * scale_b, in float32 with one rounding (`out` may be `a` or `b`)."""
        self._dense(a, "a")
        self._dense(b, "b", a.dtype, tuple(a.shape))
        self._dense(out, "out", a.dtype, tuple(a.shape))
        self._check(self._parts().akv_scaled_sum(_ptr(a), ctypes.c_float(scale_a), _ptr(b), ctypes.c_float(scale_b), _ptr(out),
                                                 self._code_of(a), _long(a.numel()), self._stream()), "scaled_sum")

    # ---- attention over a compressed latent --------------------------------------------------------------------------
    MATRIX_CORE_LATENTS = (128, 256, 512)

    def latent_on_matrix_cores(self, heads: int, kv_rank: int, width: int, page_size: int, dtype) -> bool:
        """Whether `latent_attend` has a matrix-core kernel for these sizes.  It reads a second copy of the latents with
        the keys contiguous, which the layer then keeps beside the records (`latent_encode(..., latents_t=)`)."""
        return (dtype == torch.bfloat16 and heads % 16 == 0 and width % 32 == 0 and kv_rank in self.MATRIX_CORE_LATENTS
                and page_size % 8 == 0)

    def latent_encode(self, down, q_rank, kv_rank, rot, rot_dims, q_weight, kv_weight, eps, table, positions, slot_map,
                      cq, records, latents_t=None, interleaved: bool = False) -> None:
        """down [tokens, q_rank (+ kv_rank + rot)] -> cq = norm(q latent); with `records` [pages, 1, page, kv_rank + rot]
        also the token's record: norm(kv latent), then the key part with its first `rot_dims` dimensions rotated; with
        `latents_t` [pages, 1, kv_rank, page] the normed latent once more, keys contiguous.  A rotation pair is dimensions
        (i, i + rot_dims / 2), or (2 i, 2 i + 1) with `interleaved`."""
        tokens = down.shape[0]
        writes = records is not None
        self._dense(down, "down")
        if down.dim() != 2 or down.shape[1] < q_rank + (kv_rank + rot if writes else 0):
            self._refuse(f"down must be [tokens, at least {q_rank + (kv_rank + rot if writes else 0)}], got {tuple(down.shape)}")
        self._dense(cq, "cq", down.dtype, (tokens, q_rank))
        self._dense(q_weight, "q_weight", torch.float32, (q_rank,))
        self._dense(positions, "positions", torch.int32, (tokens,))
        slots = 0
        if writes:
            self._dense(records, "records", down.dtype)
            if records.dim() != 4 or records.shape[1] != 1 or records.shape[3] != kv_rank + rot:
                self._refuse(f"records must be [pages, 1, page, {kv_rank + rot}], got {tuple(records.shape)}")
            slots = records.shape[0] * records.shape[2]
            self._dense(kv_weight, "kv_weight", torch.float32, (kv_rank,))
            self._dense(slot_map, "slot_map", torch.int32, (tokens,))
            self._dense(table, "table", torch.float32)
            if table.dim() != 3 or table.shape[1] != rot_dims // 2 or table.shape[2] != 2:
                self._refuse(f"the rotation table must be [positions, {rot_dims // 2}, 2], got {tuple(table.shape)}")
            if latents_t is not None:
                self._dense(latents_t, "latents_t", down.dtype, (records.shape[0], 1, kv_rank, records.shape[2]))
        self._check(self._parts().akv_latent_encode(
            _ptr(down), self._code_of(down), tokens, q_rank, kv_rank, rot, rot_dims, _ptr(q_weight), _ptr(kv_weight),
            ctypes.c_float(eps), _ptr(table) if writes else ctypes.c_void_p(0), table.shape[0] if writes else 0,
            _ptr(positions), _ptr(slot_map) if writes else ctypes.c_void_p(0), _ptr(cq),
            _ptr(records) if writes else ctypes.c_void_p(0), _long(slots),
            _ptr(latents_t) if writes and latents_t is not None else ctypes.c_void_p(0),
            records.shape[2] if writes else 0, 1 if interleaved else 0, _long(down.shape[1]), self._stream()), "latent_encode")

    def rotate_queries(self, q, heads, dim, rot, rot_dims, table, positions, q_abs, at, interleaved: bool = False) -> None:
        """q [tokens, heads * (dim + rot)] -> q_abs[:, :, at:at + rot] (float32, or bfloat16 like q): every head's last
        `rot` dimensions, the first `rot_dims` of them rotated by the token's position."""
        tokens = q.shape[0]
        self._dense(q, "q", None, (tokens, heads * (dim + rot)))
        self._dense(q_abs, "q_abs")
        if q_abs.dtype != torch.float32 and q_abs.dtype != q.dtype:
            self._refuse(f"q_abs must be float32 or {q.dtype}, got {q_abs.dtype}")
        if q_abs.dim() != 3 or q_abs.shape[0] != tokens or q_abs.shape[1] != heads or at + rot > q_abs.shape[2]:
            self._refuse(f"q_abs must be [tokens, heads, at least {at + rot}], got {tuple(q_abs.shape)}")
        self._dense(table, "table", torch.float32)
        if table.dim() != 3 or table.shape[1] != rot_dims // 2 or table.shape[2] != 2:
            self._refuse(f"the rotation table must be [positions, {rot_dims // 2}, 2], got {tuple(table.shape)}")
        self._dense(positions, "positions", torch.int32, (tokens,))
        self._check(self._parts().akv_rotate_queries(_ptr(q), self._code_of(q), _long(tokens), heads, dim, rot, rot_dims,
                                                     _ptr(table), table.shape[0], _ptr(positions), _ptr(q_abs),
                                                     self._code_of(q_abs), q_abs.shape[2], at, 1 if interleaved else 0,
                                                     self._stream()),
                    "rotate_queries")

    def heads_linear(self, x, x_width: int, weight, y, y_width: int) -> None:
        """y[t, h, :outs] = x[t, h, :ins] W[h] for W [heads, ins, outs]: `x` is [tokens, heads, x_width] and `y`
        [tokens, heads, y_width], of which the product reads the first `ins` and writes the first `outs` of every head."""
        heads, ins, outs = weight.shape
        tokens = x.shape[0]
        self._dense(weight, "weight")
        self._dense(x, "x", None, (tokens, heads, x_width))
        self._dense(y, "y", None, (tokens, heads, y_width))
        if ins > x_width or outs > y_width:
            self._refuse(f"a product of {ins} -> {outs} per head does not fit rows of {x_width} and {y_width}")
        above = getattr(self, "library_products_above", None)
        if (above is not None and tokens > above and x.dtype == weight.dtype == y.dtype == torch.bfloat16):
            # as with the plain products: many rows of bfloat16 go to the BLAS library, one batched product over the heads
            torch.bmm(x[:, :, :ins].transpose(0, 1), weight, out=self._heads_scratch(heads, tokens, outs))
            y[:, :, :outs].copy_(self._heads_scratch(heads, tokens, outs).transpose(0, 1))
            return
        self._check(self._parts().akv_heads_linear(
            _ptr(x), self._code_of(x), _long(heads * x_width), _long(x_width), _ptr(weight), self._code_of(weight), _ptr(y),
            self._code_of(y), _long(heads * y_width), _long(y_width), tokens, heads, ins, outs, self._stream()),
            "heads_linear")

    def _heads_scratch(self, heads: int, tokens: int, outs: int) -> torch.Tensor:
        """Where a batched product over the heads leaves [heads, tokens, outs] before it is laid out by token."""
        need = heads * tokens * outs
        held = self.__dict__.get("_heads_buffer")
        if held is None or held.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                self._refuse("a recorded step needs more room for a product over the heads than the steps before it")
            self.__dict__.setdefault("_heads_outgrown", []).append(held)
            held = self.__dict__["_heads_buffer"] = torch.empty(max(need, 1 << 22), dtype=torch.bfloat16, device=self.device)
        return held[:need].view(heads, tokens, outs)

    LATENT_WAVES = 1024             # steps of few tokens cut every token's keys into runs until about so many waves work
    LATENT_MIN_RUN = 64
    LATENT_MAX_RUNS = 64

    def _latent_runs(self, tiles: int, kv_rank: int, span: int):
        """(keys per run, runs, workspace) for a launch of `tiles` waves whose tokens see at most `span` keys: one run
        where the tiles alone fill the device; else runs of a size that depends on the step's shape and the span's bound
        only - a recorded step is cut as the same step run eagerly."""
        if tiles * 2 >= self.LATENT_WAVES or span <= self.LATENT_MIN_RUN:
            return 0, 1, None
        wanted = max(self.LATENT_WAVES // tiles, 1)
        segment = max((span + wanted - 1) // wanted, self.LATENT_MIN_RUN)
        segment = (segment + 31) // 32 * 32
        segments = (span + segment - 2) // segment + 1            # the most runs that a span of keys can touch
        while segments > self.LATENT_MAX_RUNS:
            segment *= 2
            segments = (span + segment - 2) // segment + 1
        if segments <= 1:
            return 0, 1, None
        need = tiles * segments * 16 * (kv_rank + 2)
        held = self.__dict__.get("_latent_parts")
        if held is None or held.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                self._refuse("a recorded step needs more room for the runs' shares than the steps before it")
            self.__dict__.setdefault("_latent_outgrown", []).append(held)
            held = self.__dict__["_latent_parts"] = torch.empty(max(need, 1 << 22), dtype=torch.float32, device=self.device)
        return segment, segments, held

    def latent_attend(self, q_abs, records, ctx, meta, heads, kv_rank, scale, window, out, latents_t=None) -> None:
        """Every head of every token attends the records [kv_rank + rot] of its request's last `window` tokens (all,
        if None): softmax((q_abs . record) * scale), then the weighted sum of the records' first kv_rank dimensions
        -> out [tokens, heads, kv_rank].  q_abs and out are float32 - or, with `latents_t` (the layer's second copy of
        the latents, see `latent_on_matrix_cores`), bfloat16: the matrix-core kernel."""
        tokens, width = q_abs.shape[0], q_abs.shape[2]
        mfma = latents_t is not None
        self._dense(q_abs, "q_abs", torch.bfloat16 if mfma else torch.float32, (tokens, heads, width))
        self._dense(out, "out", q_abs.dtype, (tokens, heads, kv_rank))
        self._dense(records, "records")
        if records.dim() != 4 or records.shape[1] != 1 or records.shape[3] != width:
            self._refuse(f"records must be [pages, 1, page, {width}], got {tuple(records.shape)}")
        self._dense(meta.block_table, "block_table", torch.int32)
        if meta.block_table.dim() != 2 or meta.block_table.shape[1] != meta.width:
            self._refuse("the block table does not have the width the step names")
        self._step_arrays(ctx, tokens)
        if meta.rows is not None:
            self._dense(meta.rows, "table rows", torch.int32, (ctx.num_seqs,))
            if max(ctx.host_seq_slots) >= meta.block_table.shape[0]:
                self._refuse("a request's slot lies outside the block table")
        elif ctx.num_seqs > meta.block_table.shape[0]:
            self._refuse("the block table has fewer rows than the step has requests")
        if ctx.max_seq_len > meta.width * records.shape[2]:
            self._refuse("a request is longer than its row of the block table")
        if mfma:
            if not self.latent_on_matrix_cores(heads, kv_rank, width, records.shape[2], records.dtype):
                self._refuse("the matrix-core attention over latents does not take these sizes")
            self._dense(latents_t, "latents_t", torch.bfloat16, (records.shape[0], 1, kv_rank, records.shape[2]))
            segment, segments, parts = self._latent_runs(tokens * heads // 16, kv_rank,
                                                         int(window) if window is not None else ctx.max_seq_len)
            self._check(self._parts().akv_latent_attend_mfma(
                _ptr(q_abs), _ptr(records), _ptr(latents_t), _ptr(ctx.seq_of_token), _ptr(ctx.positions),
                _ptr(meta.block_table), _ptr(meta.rows), meta.width, _ptr(out), tokens, heads, kv_rank, width,
                records.shape[2], _long(records.shape[0]), ctypes.c_float(scale), int(window) if window is not None else 0,
                segment, segments, _ptr(parts), 1 if ctx.num_seqs == 1 else 0, self._stream()),
                "latent_attend on the matrix cores")
            return
        self._check(self._parts().akv_latent_attend(
            _ptr(q_abs), _ptr(records), self._code_of(records), _ptr(ctx.seq_of_token), _ptr(ctx.positions),
            _ptr(meta.block_table), _ptr(meta.rows), meta.width, _ptr(out), tokens, heads, kv_rank, width, records.shape[2],
            _long(records.shape[0]), ctypes.c_float(scale), int(window) if window is not None else 0, self._stream()),
            "latent_attend")

    # ---- selective scan ------------------------------------------------------------------------------------------------
    def _scan_state(self, state, ctx, channels, n_state, taps):
        self._dense(state, "state", torch.float32)
        need = channels * n_state + (taps - 1) * channels
        if state.dim() != 2 or state.shape[1] != need:
            self._refuse(f"the scan's state must be [slots, {need}], got {tuple(state.shape)}")
        if max(ctx.host_seq_slots) >= state.shape[0]:
            self._refuse("a request's slot lies outside the state")

    def conv_silu(self, xz, channels, weight, bias, state, n_state, ctx, out, activation: str = "silu", conv_at=None) -> None:
        """out[t, c] = silu(bias[c] + sum_k weight[c, k] * x[t - (taps - 1 - k), c]) over the first `channels` columns
        of `xz` (with `activation="none"` the sum as it is; `bias` None: none); inputs before a portion come from the
        request's state (zeros before its first token).  Afterwards the state holds the last taps - 1 inputs of every
        request of the step.  The inputs lie in the state from element `conv_at` on (default: after `channels * n_state`
        elements, and the state holds nothing else)."""
        tokens, taps = xz.shape[0], weight.shape[1]
        self._dense(xz, "xz")
        if xz.dim() != 2 or xz.shape[1] < channels:
            self._refuse(f"xz must be [tokens, at least {channels}], got {tuple(xz.shape)}")
        self._dense(weight, "weight", None, (channels, taps))
        if bias is not None:
            self._dense(bias, "bias", weight.dtype, (channels,))
        self._dense(out, "out", xz.dtype, (tokens, channels))
        if conv_at is None:
            self._scan_state(state, ctx, channels, n_state, taps)
            conv_at = channels * n_state
        else:
            self._dense(state, "state", torch.float32)
            if state.dim() != 2 or conv_at < 0 or state.shape[1] < conv_at + (taps - 1) * channels:
                self._refuse(f"the state must hold {(taps - 1) * channels} inputs from element {conv_at} on, got {tuple(state.shape)}")
            if max(ctx.host_seq_slots) >= state.shape[0]:
                self._refuse("a request's slot lies outside the state")
        self._step_arrays(ctx, tokens)
        lib = self._parts()
        if activation not in ("silu", "none"):
            self._refuse(f"the convolution's activation is 'silu' or 'none', not {activation!r}")
        self._check(lib.akv_conv_taps(_ptr(xz), _long(xz.shape[1]), self._code_of(xz), _ptr(weight), _ptr(bias),
                                      self._code_of(weight), _ptr(state), _long(state.shape[1]), _long(conv_at),
                                      _ptr(ctx.seq_of_token), _ptr(ctx.q_start), _ptr(ctx.seq_slots), _ptr(out), tokens,
                                      channels, taps, 1 if activation == "silu" else 0, self._stream()), "conv_taps")
        if taps > 1:
            self._check(lib.akv_conv_state_update(_ptr(xz), _long(xz.shape[1]), self._code_of(xz), _ptr(state),
                                                  _long(state.shape[1]), _long(conv_at), _ptr(ctx.q_start), _ptr(ctx.seq_slots),
                                                  ctx.num_seqs, channels, taps, self._stream()), "conv_state_update")

    # ---- the gated delta rule --------------------------------------------------------------------------------------------
    def check_delta_rule_sizes(self, heads: int, groups: int, dim: int, vdim: int) -> None:
        if heads % groups or not 0 < dim <= 2048 or vdim <= 0:
            self._refuse(f"the delta rule takes heads that are a multiple of the key heads and keys up to 2048 wide, not "
                         f"{heads} / {groups} heads of {dim}")

    def delta_rule(self, conv, beta_logits, beta_at: int, decay_logits, decay_bias, rate, gates, norm_weight, unit_eps: float,
                   norm_eps: float, q_scale: float, heads: int, groups: int, dim: int, vdim: int, state, ctx, out) -> None:
        """conv [tokens, 2 * groups * dim + heads * vdim]: q, k and v after their convolutions and activations.  q and k
        become unit vectors per head (x / sqrt(sum x^2 + unit_eps); q times q_scale); beta = sigmoid(beta_logits[:, beta_at +
        h]); g = exp(-rate[h] * softplus(decay_logits[t, h, d] + decay_bias[h, d])).  Per request and head, token after
        token: S <- g S (rows are key channels); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  out [tokens, heads * vdim]
        = o / rms(o) * norm_weight * sigmoid(gates).  S lies at the start of the request's slot of `state`, float32, as
        [heads, vdim, dim]."""
        tokens = conv.shape[0]
        width = 2 * groups * dim + heads * vdim
        self._dense(conv, "conv", None, (tokens, width))
        self._dense(beta_logits, "beta_logits", conv.dtype)
        if beta_logits.dim() != 2 or beta_logits.shape[0] != tokens or beta_at < 0 or beta_at + heads > beta_logits.shape[1]:
            self._refuse(f"beta_logits must be [tokens, at least {beta_at + heads}], got {tuple(beta_logits.shape)}")
        self._dense(decay_logits, "decay_logits", torch.float32, (tokens, heads * dim))
        self._dense(decay_bias, "decay_bias", torch.float32, (heads * dim,))
        self._dense(rate, "rate", torch.float32, (heads,))
        self._dense(gates, "gates", torch.float32, (tokens, heads * vdim))
        self._dense(norm_weight, "norm_weight", torch.float32, (vdim,))
        self._dense(out, "out", conv.dtype, (tokens, heads * vdim))
        self._dense(state, "state", torch.float32)
        if state.dim() != 2 or state.shape[1] < heads * dim * vdim:
            self._refuse(f"the state must be [slots, at least {heads * dim * vdim}], got {tuple(state.shape)}")
        if max(ctx.host_seq_slots) >= state.shape[0]:
            self._refuse("a request's slot lies outside the state")
        self.check_delta_rule_sizes(heads, groups, dim, vdim)
        self._step_arrays(ctx, tokens)
        lib = self._parts()
        workspace = self._delta_workspace(int(lib.akv_delta_rule_workspace(tokens, heads, groups, dim, vdim)))
        self._check(lib.akv_delta_rule(
            _ptr(conv), _long(width), self._code_of(conv), _ptr_at(beta_logits, beta_at), _long(beta_logits.shape[1]),
            _ptr(decay_logits), _ptr(decay_bias), _ptr(rate), _ptr(gates), _ptr(norm_weight), ctypes.c_float(unit_eps),
            ctypes.c_float(norm_eps), ctypes.c_float(q_scale), _ptr(state), _long(state.shape[1]), _ptr(ctx.q_start),
            _ptr(ctx.seq_slots), _ptr(workspace), _ptr(out), tokens, ctx.num_seqs, heads, groups, dim, vdim,
            int(ctx.max_new_tokens) or tokens, self._stream()),
            "delta_rule")

    def _delta_workspace(self, need: int) -> torch.Tensor:
        """Where the tokens' unit vectors, decays and raw outputs lie during a step."""
        held = self.__dict__.get("_delta_buffer")
        if held is None or held.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                self._refuse("a recorded step needs more room for the delta rule's tokens than the steps before it")
            self.__dict__.setdefault("_delta_outgrown", []).append(held)
            held = self.__dict__["_delta_buffer"] = torch.empty(max(need, 1 << 22), dtype=torch.float32, device=self.device)
        return held

    def selective_scan(self, x, dt, bc, xz, a, d, state, taps, ctx, out) -> None:
        """Per request and channel, token after token: S <- exp(softplus(dt) A) S + softplus(dt) x B, y = S C + D x,
        out = y * silu(z), with z the second half of `xz`'s columns and S [channels, n_state] at the start of the
        request's state (read at the portion's start, written back at its end).  `dt` is left as softplus(dt)."""
        tokens, channels = x.shape
        n_state = a.shape[1]
        self._dense(x, "x", None, (tokens, channels))
        self._dense(dt, "dt", torch.float32, (tokens, channels))
        self._dense(bc, "bc", torch.float32, (tokens, 2 * n_state))
        self._dense(xz, "xz", x.dtype, (tokens, 2 * channels))
        self._dense(a, "a", torch.float32, (channels, n_state))
        self._dense(d, "d", torch.float32, (channels,))
        self._dense(out, "out", x.dtype, (tokens, channels))
        self._scan_state(state, ctx, channels, n_state, taps)
        self._step_arrays(ctx, tokens)
        z = xz[:, channels:]
        self._check(self._parts().akv_selective_scan(
            _ptr(x), self._code_of(x), _ptr(dt), _ptr(bc), ctypes.c_void_p(z.data_ptr()), _long(2 * channels), _ptr(a),
            _ptr(d), _ptr(state), _long(state.shape[1]), _ptr(ctx.q_start), _ptr(ctx.seq_slots), _ptr(out), tokens,
            ctx.num_seqs, channels, n_state, self._stream()), "selective_scan")

    # ---- routed feed-forward -------------------------------------------------------------------------------------------
    def route(self, logits, gates, top: int, groups: int, keep: int) -> None:
        """gates[t, e] = softmax(logits_t)[e] for the `top` best experts among those of the `keep` best of `groups`
        groups of neighbouring experts (a group's score is its best expert's), 0 for every other expert."""
        tokens, experts = logits.shape
        self._dense(logits, "logits", torch.float32)
        self._dense(gates, "gates", torch.float32, (tokens, experts))
        self._check(self._parts().akv_route(_ptr(logits), _ptr(gates), tokens, experts, top, groups, keep, self._stream()),
                    "route")

    def gate_relu_squared(self, up, gates, act) -> None:
        """act[t, e * ff + j] = gates[t, e] * relu(up[t, e * ff + j])^2 (may be in place)."""
        tokens, experts = gates.shape
        self._dense(up, "up")
        if up.shape[0] != tokens or up.shape[1] % experts:
            self._refuse(f"up must be [tokens, experts * ff], got {tuple(up.shape)} for {experts} experts")
        self._dense(act, "act", up.dtype, tuple(up.shape))
        self._dense(gates, "gates", torch.float32)
        self._check(self._parts().akv_gate_relu_squared(_ptr(up), _ptr(gates), _ptr(act), self._code_of(up), _long(tokens),
                                                        experts, up.shape[1] // experts, self._stream()),
                    "gate_relu_squared")

    def route_chosen(self, logits, gates, experts: int, top: int, law: str = "softmax") -> None:
        """gates[t, e] = the softmax over the `top` largest of the first `experts` logits for those experts (equal logits
        go to the lower index), 0 for the others; every further column of a row becomes its sigmoid.  `law="sigmoid"`:
        logits [tokens, experts]; a chosen expert's gate is the sigmoid of its own logit, and every further column of
        `gates` becomes 1."""
        tokens = logits.shape[0]
        self._dense(logits, "logits", torch.float32)
        if law == "sigmoid":
            self._dense(logits, "logits", torch.float32, (tokens, experts))
            self._dense(gates, "gates", torch.float32)
            if gates.dim() != 2 or gates.shape[0] != tokens or gates.shape[1] < experts:
                self._refuse(f"gates must be [tokens, at least {experts}], got {tuple(gates.shape)}")
        elif law == "softmax":
            self._dense(gates, "gates", torch.float32, (tokens, logits.shape[1]))
        else:
            self._refuse(f"chosen experts are weighted by 'softmax' or 'sigmoid', not {law!r}")
        self._check(self._parts().akv_route_chosen(_ptr(logits), _ptr(gates), tokens, experts, gates.shape[1], top,
                                                   1 if law == "sigmoid" else 0, self._stream()), "route_chosen")

    EXPERT_ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu_squared": 3}

    def gate_activation(self, up, gates, act, experts: int, ff: int, activation: str, inside: bool) -> None:
        """act[t, c] = f(gates[t, e(c)] * up[t, c]) (`inside`) or gates[t, e(c)] * f(up[t, c]); column c belongs to expert
        c // ff below experts * ff and to the expert every token uses beyond (gate number `experts`); exact zeros where the
        gate is zero.  (May be in place.)"""
        tokens, columns = act.shape
        self._dense(act, "act")
        self._dense(up, "up", act.dtype, (tokens, columns))
        self._dense(gates, "gates", torch.float32)
        if gates.dim() != 2 or gates.shape[0] != tokens or gates.shape[1] < experts + (1 if columns > experts * ff else 0):
            self._refuse(f"gates must be [tokens, at least the experts (and the shared one)], got {tuple(gates.shape)}")
        if activation not in self.EXPERT_ACTIVATIONS:
            self._refuse(f"an expert's activation is one of {sorted(self.EXPERT_ACTIVATIONS)}, not {activation!r}")
        self._check(self._parts().akv_gate_activation(_ptr(up), _ptr(gates), _ptr(act), self._code_of(act), _long(tokens),
                                                      experts, ff, columns, gates.shape[1], self.EXPERT_ACTIVATIONS[activation],
                                                      1 if inside else 0, self._stream()), "gate_activation")

    def gate_silu_mul(self, gate_up, gates, act, experts: int, ff: int) -> None:
        """act[t, c] = gates[t, e(c)] * silu(gate_up[t, c]) * gate_up[t, columns + c]; column c belongs to expert c // ff
        below experts * ff and to the expert every token uses beyond (gate number `experts`)."""
        tokens, columns = act.shape
        self._dense(act, "act")
        self._dense(gate_up, "gate_up", act.dtype, (tokens, 2 * columns))
        self._dense(gates, "gates", torch.float32)
        if gates.dim() != 2 or gates.shape[0] != tokens or gates.shape[1] < experts + (1 if columns > experts * ff else 0):
            self._refuse(f"gates must be [tokens, at least the experts (and the shared one)], got {tuple(gates.shape)}")
        self._check(self._parts().akv_gate_silu_mul(_ptr(gate_up), _ptr(gates), _ptr(act), self._code_of(act), _long(tokens),
                                                    experts, ff, columns, gates.shape[1], self._stream()), "gate_silu_mul")

    # ---- attention with unit-normed queries and keys, a softcap, chunks, a sink and a gate per head ----------------------
    MAX_VALUE_DIM = 256
    MATRIX_CORE_HEAD_DIMS = (32, 64, 128, 256)      # widths of keys and of values that the portions' kernel is built for

    def check_gated_attention_sizes(self, q_heads: int, kv_heads: int, dim: int, vdim: int, page_size: int) -> None:
        if q_heads % kv_heads:
            self._refuse(f"q_heads {q_heads} is not a multiple of kv_heads {kv_heads}")
        if not 0 < vdim <= self.MAX_VALUE_DIM or not 0 < dim <= 2048:
            self._refuse(f"the attention takes values up to {self.MAX_VALUE_DIM} wide and keys up to 2048, not {vdim} and {dim}")

    def _gated_pages(self, k_pages, v_pages, kv_heads, dim, vdim, dtype):
        self._dense(k_pages, "k_pages", dtype)
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != dim:
            self._refuse(f"key pages must be [pages, {kv_heads}, page_size, {dim}], got {tuple(k_pages.shape)}")
        self._dense(v_pages, "v_pages", dtype, (k_pages.shape[0], kv_heads, vdim, k_pages.shape[2]))
        return k_pages.shape[0], k_pages.shape[2]

    def unit_norm_write(self, projected, q_heads, kv_heads, dim, vdim, eps, slot_map, k_pages, v_pages, q_out, at: int = 0,
                        maps: int = 1, table=None, rot_dims: int = 0, positions=None, q_weight=None, k_weight=None,
                        whole: bool = False, interleaved: bool = False) -> None:
        """projected [tokens, ... | q | k | v | ...] with q at column `at`: the query heads divided by their root mean square (eps inside the root;
        `eps` None: as they are) -> q_out; with `slot_map` the key heads, the same way, and the value heads into the
        tokens' slots of the pages.  `maps` > 1: a head's queries and keys are `maps` vectors of `dim` side by side, each
        normed and rotated for itself; a key head's record in the pages is `maps * dim` wide.  `table` [positions,
        rot_dims / 2, 2] (cos, sin): every vector's first `rot_dims` dimensions are rotated by the token's position
        (`positions`), dimension i with i + rot_dims / 2 (`interleaved`: 2 i with 2 i + 1), after the norm.  `whole`: the
        root mean square is taken over all of a token's query vectors at once, and over all its key vectors.  `q_weight`,
        `k_weight` (float32, one value per column of the queries and of the keys): multiplied in after the norm."""
        tokens = projected.shape[0]
        if q_weight is not None:
            self._dense(q_weight, "q_weight", torch.float32, (q_heads * maps * dim,))
        if k_weight is not None:
            self._dense(k_weight, "k_weight", torch.float32, (kv_heads * maps * dim,))
        self._dense(projected, "projected")
        if projected.dim() != 2 or at < 0 or projected.shape[1] < at + (q_heads + kv_heads) * maps * dim + kv_heads * vdim:
            self._refuse(f"projected rows must hold queries, keys and values, got {tuple(projected.shape)}")
        self._dense(q_out, "q_out", projected.dtype, (tokens, q_heads * maps * dim))
        num_pages, page_size = self._gated_pages(k_pages, v_pages, kv_heads, maps * dim, vdim, projected.dtype)
        if slot_map is not None:
            self._dense(slot_map, "slot_map", torch.int32, (tokens,))
        table_positions = 0
        if table is not None:
            self._dense(table, "table", torch.float32)
            if rot_dims <= 0 or rot_dims % 2 or rot_dims > dim or table.dim() != 3 or table.shape[1] != rot_dims // 2 or table.shape[2] != 2:
                self._refuse(f"the rotation table must be [positions, {rot_dims // 2}, 2] for an even rot_dims of at most {dim}, "
                             f"got {tuple(table.shape)} for {rot_dims}")
            self._dense(positions, "positions", torch.int32, (tokens,))
            table_positions = table.shape[0]
        self._check(self._parts().akv_unit_norm_write(
            _ptr_at(projected, at), _long(projected.shape[1]), self._code_of(projected), _long(tokens), q_heads, kv_heads, dim,
            vdim, ctypes.c_float(eps if eps is not None else 0.0), 0 if eps is None else 1, _ptr(slot_map), _ptr(k_pages),
            _ptr(v_pages), page_size, _long(num_pages), _ptr(q_out), maps, _ptr(table), table_positions,
            rot_dims if table is not None else 0, _ptr(positions) if table is not None else ctypes.c_void_p(0),
            _ptr(q_weight), _ptr(k_weight), 1 if whole else 0, 1 if interleaved else 0, self._stream()), "unit_norm_write")

    def gated_attention(self, q, k_pages, v_pages, gates, gate_at, ctx, meta, q_heads, kv_heads, dim, vdim, scale, softcap,
                        chunk, window, sink, out, out_at: int = 0, out_scale: float = 1.0, sink_logits=None,
                        maps: int = 1, keep_first: int = 0) -> None:
        """Every query head attends the keys of its request that it sees (see `parts/gated_attention.py`) -> columns
        out_at .. out_at + q_heads * vdim of `out`, times `out_scale`; `gates` [tokens, width]: head h's output times
        sigmoid(gates[t, gate_at + h]).  `sink_logits` [q_heads] float32 (with `sink`): the denominator's extra term is
        exp(sink_logits[h]) instead of exp(0).  `maps` > 1: a head has `maps` query vectors, each an attention of its own
        over the vector of the same number in its key head's record ([pages, kv_heads, page, maps * dim]) and over the
        head's values; out then holds q_heads * maps outputs a token, a head's maps side by side.  `keep_first`: a request's
        first so many keys stay visible behind the window."""
        tokens = q.shape[0]
        heads = q_heads
        q_heads = heads * maps          # (from here on: query vectors)
        self._dense(q, "q", None, (tokens, q_heads * dim))
        self._dense(out, "out", q.dtype)
        if out.dim() != 2 or out.shape[0] != tokens or out_at < 0 or out_at + q_heads * vdim > out.shape[1]:
            self._refuse(f"out must be [tokens, at least {out_at + q_heads * vdim}], got {tuple(out.shape)}")
        num_pages, page_size = self._gated_pages(k_pages, v_pages, kv_heads, maps * dim, vdim, q.dtype)
        if maps > 1 and gates is not None:
            self._refuse("a gate per head and several maps per head do not go together")
        if sink_logits is not None:
            self._dense(sink_logits, "sink_logits", torch.float32, (q_heads,))
            if not sink:
                self._refuse("sink logits without a sink")
        gate_stride = 0
        if gates is not None:
            self._dense(gates, "gates", q.dtype)
            if gates.dim() != 2 or gates.shape[0] != tokens or gate_at + q_heads > gates.shape[1]:
                self._refuse(f"gates must be [tokens, at least {gate_at + q_heads}], got {tuple(gates.shape)}")
            gate_stride = gates.shape[1]
        self._dense(meta.block_table, "block_table", torch.int32)
        if meta.block_table.dim() != 2 or meta.block_table.shape[1] != meta.width:
            self._refuse("the block table does not have the width the step names")
        self._step_arrays(ctx, tokens)
        if meta.rows is not None:
            self._dense(meta.rows, "table rows", torch.int32, (ctx.num_seqs,))
            if max(ctx.host_seq_slots) >= meta.block_table.shape[0]:
                self._refuse("a request's slot lies outside the block table")
        elif ctx.num_seqs > meta.block_table.shape[0]:
            self._refuse("the block table has fewer rows than the step has requests")
        if ctx.max_seq_len > meta.width * page_size:
            self._refuse("a request is longer than its row of the block table")
        tail = (ctypes.c_float(scale), ctypes.c_float(softcap if softcap is not None else 0.0),
                int(chunk) if chunk is not None else 0, int(window) if window is not None else 0, 1 if sink else 0,
                _long(out.shape[1]), ctypes.c_float(out_scale), _ptr(sink_logits), maps, int(keep_first), self._stream())
        singles = tokens
        if (q.dtype == torch.bfloat16 and dim in self.MATRIX_CORE_HEAD_DIMS and vdim in self.MATRIX_CORE_HEAD_DIMS
                and page_size % 16 == 0 and out.shape[1] % 4 == 0 and out_at % 4 == 0):
            # single tokens: a wave per token and head; the portions' rows, which follow them, go to the matrix cores
            singles = ctx.num_decode_seqs
            self._check(self._parts().akv_gated_attention_tiles(
                _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(gates), _long(gate_stride), gate_at, _ptr(ctx.seq_of_token),
                _ptr(ctx.q_start), _ptr(ctx.positions), _ptr(meta.block_table), _ptr(meta.rows), meta.width,
                _ptr_at(out, out_at), singles, tokens, q_heads, kv_heads, dim, vdim, page_size, _long(num_pages), *tail),
                "gated_attention on the matrix cores")
        if singles:
            # waves that share a token's head: by the most keys a row can see (a bound that a recorded step keeps), fewer
            # where the rows alone fill the device
            span = min(x for x in (chunk, window, ctx.max_seq_len) if x is not None)
            row_waves = max(1, min(16 if singles * q_heads <= 4096 else 4, span // 128))
            self._check(self._parts().akv_gated_attention_rows(
                _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(gates), _long(gate_stride), gate_at, _ptr(ctx.seq_of_token),
                _ptr(ctx.positions), _ptr(meta.block_table), _ptr(meta.rows), meta.width, _ptr_at(out, out_at),
                self._code_of(q), _long(singles), q_heads, kv_heads, dim, vdim, page_size, _long(num_pages), *tail[:-4], row_waves,
                *tail[-4:]), "gated_attention")

    # ---- mixers with a state of fixed size -----------------------------------------------------------------------------
    def check_retention_sizes(self, heads: int, dim: int, vdim: int) -> None:
        if not 0 < vdim <= 1024 or dim <= 0 or vdim * ((dim + 63) // 64) > 1024:
            self._refuse(f"retention keeps a head's state [{dim}, {vdim}] in one block's registers: up to 65,536 values")

    def retention(self, projected, heads, dim, vdim, rot_dims, table, key_scale, decay, eps, state, ctx, out, at: int = 0,
                  out_at: int = 0, out_scale: float = 1.0, input_activation: str | None = None, raw=None) -> None:
        """projected [tokens, ... | q | k | v | g | ...] with q at column `at` -> columns out_at .. out_at + heads * vdim of
        `out` = (S^T q) / rms * silu(g) * out_scale with S <- decay S + k v^T per request and head (see
        `parts/retention.py`); S lies in the request's slot of `state`, float32.  `input_activation="silu"`: q, k and v
        pass silu as they are read.  `raw` [tokens, heads * vdim] float32: the outputs S^T q are left there as they are,
        `out` (then None) is not written, and the rows need hold no gates."""
        tokens = projected.shape[0]
        self._dense(projected, "projected")
        if projected.dim() != 2 or at < 0 or projected.shape[1] < at + heads * (2 * dim + vdim) + (heads * vdim if raw is None else 0):
            self._refuse(f"projected rows must hold queries, keys, values and gates from column {at}, got {tuple(projected.shape)}")
        if input_activation not in (None, "silu"):
            self._refuse(f"retention's inputs pass 'silu' or nothing, not {input_activation!r}")
        if raw is not None:
            self._dense(raw, "raw", torch.float32, (tokens, heads * vdim))
            if out is not None:
                self._refuse("raw outputs are left instead of normed and gated ones")
            out, out_at = raw, 0      # (stands in where an address is formed; the kernels do not write it)
        else:
            self._dense(out, "out", projected.dtype)
            if out.dim() != 2 or out.shape[0] != tokens or out_at < 0 or out_at + heads * vdim > out.shape[1]:
                self._refuse(f"out must be [tokens, at least {out_at + heads * vdim}], got {tuple(out.shape)}")
        self._dense(decay, "decay", torch.float32, (heads,))
        self._dense(state, "state", torch.float32)
        if state.dim() != 2 or state.shape[1] != heads * dim * vdim:
            self._refuse(f"retention's state must be [slots, {heads * dim * vdim}], got {tuple(state.shape)}")
        if max(ctx.host_seq_slots) >= state.shape[0]:
            self._refuse("a request's slot lies outside the state")
        positions = 0
        if rot_dims:
            self._dense(table, "table", torch.float32)
            if table.dim() != 3 or table.shape[1] != rot_dims // 2 or table.shape[2] != 2:
                self._refuse(f"the rotation table must be [positions, {rot_dims // 2}, 2], got {tuple(table.shape)}")
            positions = table.shape[0]       # (the engine admits no request beyond the positions its tables were built for)
        self._step_arrays(ctx, tokens)
        head = (_ptr_at(projected, at), _long(projected.shape[1]), self._code_of(projected), ctx.num_seqs, heads, dim, vdim,
                rot_dims, _ptr(table) if rot_dims else ctypes.c_void_p(0), positions, ctypes.c_float(key_scale), _ptr(decay),
                ctypes.c_float(eps), _ptr(state), _long(state.shape[1]), _ptr(ctx.q_start), _ptr(ctx.seq_slots),
                _ptr(ctx.positions), _ptr_at(out, out_at), _long(out.shape[1]), ctypes.c_float(out_scale))
        extras = (1 if input_activation == "silu" else 0, _ptr(raw))
        length = self._retention_chunk(dim, vdim)
        if ctx.max_new_tokens >= self.RETENTION_CHUNKED_FROM and length:
            # portions: chunks side by side (the step's shape alone decides, so a recorded step replays the same launches)
            chunks = (ctx.max_new_tokens + length - 1) // length
            sums = self._retention_sums(2 * ctx.num_seqs * heads * chunks * dim * vdim)
            self._check(self._parts().akv_retention_chunked(*head, _ptr(sums), length, chunks, *extras, self._stream()),
                        "retention over chunks")
            return
        self._check(self._parts().akv_retention(*head, *extras, self._stream()), "retention")

    RETENTION_CHUNKED_FROM = 24       # steps whose longest portion has fewer tokens take them one after the other

    @staticmethod
    def _retention_chunk(dim: int, vdim: int) -> int:
        """Tokens per chunk: the most of 32, 16, 8 whose operands fit into 128 KB of LDS (0: none does)."""
        for length in (32, 16, 8):
            if (2 * length * (dim + 1) + 2 * length * vdim + length * (length + 1) + length + 1) * 4 <= 128 * 1024:
                return length
        return 0

    def _retention_sums(self, need: int) -> torch.Tensor:
        """Where the chunks' sums and the states before them lie during a step."""
        held = self.__dict__.get("_retention_buffer")
        if held is None or held.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                self._refuse("a recorded step needs more room for retention's chunks than the steps before it")
            self.__dict__.setdefault("_retention_outgrown", []).append(held)
            held = self.__dict__["_retention_buffer"] = torch.empty(max(need, 1 << 22), dtype=torch.float32, device=self.device)
        return held

    @staticmethod
    def _scan_runs(longest_portion: int) -> int:
        """Runs that the longest portion of a step is cut into: 16 tokens a run and more, 64 runs at most (the step's shape
        alone decides, so a recorded step is cut as the same step run eagerly)."""
        return max(1, min(64, longest_portion // 16))

    def gated_linear_scan(self, u, gates, gate_bias, rate, xy, blocks, state, taps, ctx, out) -> None:
        """Per request and channel, token after token: a = exp(rate * sigmoid(gates_r + bias)), S <- a S + sqrt(1 - a^2)
        sigmoid(gates_i + bias) u, out = S * gelu_tanh(y), with y the second half of `xy`'s columns and S at the start of
        the request's state."""
        tokens, channels = u.shape
        self._dense(u, "u")
        self._dense(gates, "gates", torch.float32, (tokens, blocks, 2 * (channels // blocks)))
        self._dense(gate_bias, "gate_bias", torch.float32, (blocks, 2 * (channels // blocks)))
        self._dense(rate, "rate", torch.float32, (channels,))
        self._dense(xy, "xy", u.dtype, (tokens, 2 * channels))
        self._dense(out, "out", u.dtype, (tokens, channels))
        self._scan_state(state, ctx, channels, 1, taps)
        self._step_arrays(ctx, tokens)
        y = xy[:, channels:]
        self._check(self._parts().akv_gated_linear_scan(
            _ptr(u), self._code_of(u), _ptr(gates), _ptr(gate_bias), _ptr(rate), ctypes.c_void_p(y.data_ptr()),
            _long(2 * channels), ctx.num_seqs, channels, blocks, self._scan_runs(ctx.max_new_tokens), _ptr(state),
            _long(state.shape[1]), _ptr(ctx.q_start),
            _ptr(ctx.seq_slots), _ptr(out), self._stream()), "gated_linear_scan")
