"""Token embedding (a row gather without scaling, ampere_kv/runner.py:282) and the output head
(ampere_kv/runner.py:293-297: final norm, then logits = n W^T for the wanted rows only)."""

from __future__ import annotations

import torch

from ..weights.spec import EMBEDDING, MATRIX, TensorSpec
from .base import Part, register_part
from .linear import Linear


class Embedding(Part):
    def __init__(self, spec, runtime):
        self.rt = runtime
        self.vocab, self.hidden = int(spec["vocab_size"]), int(spec["hidden_size"])
        self.name = spec["name"]
        self.weight = None

    def tensors(self, prefix=""):
        return [TensorSpec(self.name, (self.vocab, self.hidden), EMBEDDING)]

    def load(self, fetch, prefix=""):
        self.weight = fetch(self.tensors()[0]).contiguous()

    def weight_bytes(self):
        return 0  # a step reads one row per token, not the table

    def forward(self, token_ids: torch.Tensor, stream: torch.Tensor, ctx=None) -> torch.Tensor:
        """token_ids int32 [tokens] -> stream float32 [tokens, hidden] (the start of the residual sum).  With the
        step's context an id of -1 is the token chosen last for the row's request."""
        self.rt.kernels.embed(token_ids, self.weight, stream, ctx)
        return stream

    def add(self, token_ids: torch.Tensor, stream: torch.Tensor, ctx=None) -> None:
        """stream += the tokens' rows once more: what a pass over repeated layers adds before its first layer where the
        run order says so (`RunEntry.adds_embedding`).  The rows are gathered again rather than kept."""
        if type(self) is not Embedding:
            raise NotImplementedError("only the plain embedding's output is added to the residual sum a second time")
        self.rt.kernels.embed_add(token_ids, self.weight, stream, ctx)


class NormedEmbedding(Embedding):
    """The token's row, normed before the first layer: x = norm(table[id]), in float32 (one kernel).  `norm` is the
    specification of an RMS norm whose weight is kept float32; its tensor is named `norm_name`."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        from .base import build_part
        self.norm = build_part("norm", spec["norm"], runtime)
        self.norm_name = spec["norm_name"]

    def tensors(self, prefix=""):
        return super().tensors() + self.norm.tensors(self.norm_name)

    def load(self, fetch, prefix=""):
        super().load(fetch)
        self.norm.load(fetch, self.norm_name)

    def forward(self, token_ids, stream, ctx=None):
        self.rt.kernels.embed_normed(token_ids, self.weight, self.norm.weight, self.norm.eps, stream, ctx)
        return stream


class RowTable(Part):
    """A table [rows, hidden] of vectors, float32, of which the model's pass adds one to every token's residual sum
    where the run order says so (`RunEntry.adds_row`)."""
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.rows, self.hidden = int(spec["rows"]), int(spec["hidden_size"])
        self.name = spec["name"]
        self.table = None

    def tensors(self, prefix=""):
        return [TensorSpec(self.name, (self.rows, self.hidden), EMBEDDING)]

    def load(self, fetch, prefix=""):
        self.table = fetch(self.tensors()[0]).to(torch.float32).contiguous()

    def row(self, index: int) -> torch.Tensor:
        return self.table[index]


class PairHashEmbedding(Embedding):
    """The token's row plus a row of a second table that is chosen by the token AND the one before it:
    row = (previous id * mul_prev + id * mul_cur) mod buckets; a request's first token takes the table's last row
    (number `buckets`).  The token a request was fed last is part of what it keeps between steps: a word of its slot
    on the device, so a portion's first token finds its predecessor whatever step brought it."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.pair_name = spec["pair_name"]
        self.buckets, self.mul_prev, self.mul_cur = int(spec["buckets"]), int(spec["mul_prev"]), int(spec["mul_cur"])
        if self.buckets <= 0:
            raise ValueError(f"a table of token pairs needs at least one bucket, got {self.buckets}")
        self.pairs = None

    def tensors(self, prefix=""):
        return super().tensors() + [TensorSpec(self.pair_name, (self.buckets + 1, self.hidden), EMBEDDING)]

    def load(self, fetch, prefix=""):
        super().load(fetch)
        self.pairs = fetch(self.tensors()[1]).contiguous()

    def forward(self, token_ids, stream, ctx=None):
        self.rt.kernels.embed_pairs(token_ids, self.weight, self.pairs, self.buckets, self.mul_prev, self.mul_cur, stream, ctx)
        return stream


class LinearHead(Part):
    """logits = x W^T in float32.  When `tied_to` names the embedding, the head uses that matrix and the
    file may leave the head's own tensor out."""

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.vocab, self.hidden = int(spec["vocab_size"]), int(spec["hidden_size"])
        self.name = spec["name"]
        self.tied_to = spec.get("tied_to")
        self.linear = Linear(runtime, self.hidden, [self.vocab], [self.name])

    def tensors(self, prefix=""):
        if self.tied_to is not None:
            return []
        return self.linear.tensors("")

    def load(self, fetch, prefix="", tied_weight=None):
        if self.tied_to is not None:
            self.linear.adopt(tied_weight)
        else:
            self.linear.load(fetch, "")

    def weight_bytes(self):
        return self.linear.weight_bytes()

    def forward(self, x: torch.Tensor, logits: torch.Tensor) -> torch.Tensor:
        """x [rows, hidden] -> logits float32 [rows, vocab]."""
        return self.linear.forward(x, logits)


register_part("embedding", "embedding", Embedding)
register_part("embedding", "pair_hash_embedding", PairHashEmbedding)
register_part("embedding", "normed_embedding", NormedEmbedding)
register_part("embedding", "row_table", RowTable)
register_part("head", "linear_head", LinearHead)
