"""Architecture-neutral description of a model: which parts every layer is made of and in which order layers run.

A typed architecture configuration (for instance `Qwen3Config`) turns itself into a `ModelSpec`.  The model
is then assembled from the spec alone through the part registries, so no part ever learns which
architecture it belongs to.  All sizes and constants travel inside the specs; none lives in part code.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from types import MappingProxyType
from typing import Any, Mapping


def _freeze(params: Mapping[str, Any]) -> Mapping[str, Any]:
    return MappingProxyType(dict(params))


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: its registered kind and the parameters that its constructor takes."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self):
        object.__setattr__(self, "params", _freeze(self.params))

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


def part(kind: str, **params: Any) -> PartSpec:
    return PartSpec(kind, params)


@dataclass(frozen=True)
class LayerSpec:
    """A block and the parts it arranges.  `prefix` is the tensor-name prefix of the layer's weights."""
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    prefix: str


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.  `layer` indexes `ModelSpec.layers` (a layer may be named twice);
    `cache_layer` names the layer whose cache the mixer uses (its own by default); `writes_cache` is False
    for an entry that only reads what another entry wrote.  A layer that runs several times with the same weights
    and a cache or state of its own each time names the time in `cache_copy` (0, 1, ...): every (cache_layer,
    cache_copy) is a cache of its own.  `adds_row`: before this entry runs, row `adds_row` of the model's table of
    vectors (`ModelSpec.pass_vectors`) is added to every token's residual sum.  `adds_embedding`: before this entry runs,
    the embedding's output - the residual sum as it was before the first layer - is added to it."""
    layer: int
    cache_layer: int
    writes_cache: bool = True
    cache_copy: int = 0
    adds_row: int | None = None
    adds_embedding: bool = False


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    run_order: tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: tuple[int, ...] = ()
    max_position: int | None = None
    pass_vectors: PartSpec | None = None        # a table [rows, hidden] of vectors that run-order entries add (`adds_row`)

    def __post_init__(self):
        for entry in self.run_order:
            if not (0 <= entry.layer < len(self.layers) and 0 <= entry.cache_layer < len(self.layers)):
                raise ValueError(f"run order entry {entry} names a layer outside 0..{len(self.layers) - 1}")
            if entry.cache_copy < 0:
                raise ValueError(f"run order entry {entry} names a negative copy of its cache")
            if entry.adds_row is not None and (self.pass_vectors is None or not 0 <= entry.adds_row < self.pass_vectors["rows"]):
                raise ValueError(f"run order entry {entry} adds a row that the model's table of vectors does not have")

    def cache_key(self, entry: RunEntry) -> int:
        """The number under which the cache manager keeps the cache that `entry` uses."""
        return entry.cache_layer + entry.cache_copy * len(self.layers)


def default_run_order(num_layers: int) -> tuple[RunEntry, ...]:
    return tuple(RunEntry(i, i) for i in range(num_layers))
