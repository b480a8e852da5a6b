"""Position encodings.  `rope_half` is the rotary encoding with pairs (j, j + d/2) over the whole head
(ampere_kv/runner.py:80-98): angle = position * theta^(-2j/d) in float32; x' = x cos + rot(x) sin with
rot(x) = cat(-x[d/2:], x[:d/2]).  `none` leaves q and k as they are.

`rope_scaled` is a table for mixers that rotate the first `dims` dimensions of a head themselves, with frequencies
f_i = base^(-2i / dims) that a rule stretches for contexts longer than the `original` one:
  * "yarn": with dim(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(dim(fast)), 0), hi =
    min(ceil(dim(slow)), dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):
    f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i); cos and sin are multiplied by 0.1 ln(factor) + 1;
  * "llama3": with the wavelength l_i = 2 pi / f_i: f_i stays where l_i < original / high, becomes f_i / factor where
    l_i > original / low, and between the two, with s = (original / l_i - low) / (high - low), (1 - s) f_i / factor + s f_i;
  * none: the frequencies as they are.
`layout` says which dimensions pair i turns: "halves" (i with i + dims / 2, the default) or "interleaved" (2 i with 2 i + 1);
the table is the same, the mixer's kernels are told.
Frequencies are formed in double precision and rounded once; angles are float32 products of position and frequency."""

from __future__ import annotations

import torch

from .base import Part, register_part


class RotaryHalf(Part):
    def __init__(self, spec, runtime):
        self.head_dim = int(spec["head_dim"])
        self.theta = float(spec["theta"])
        if self.head_dim % 2:
            raise ValueError(f"rotary head_dim must be even, got {self.head_dim}")
        self.rt = runtime
        # inverse frequencies exactly as the reference forms them (runner.py:42-43): float32 on the host
        exponent = torch.arange(0, self.head_dim, 2, dtype=torch.int64).float() / self.head_dim
        self.inv_freq = (1.0 / (self.theta ** exponent)).to(runtime.device)
        # cos/sin of every position the engine can reach, float32 [max_seq_len, d/2, 2]: built once per model - every
        # layer with the same head size and theta is handed the same table (runner.py:41-44 builds inv_freq once)
        self.table = runtime.shared_buffer(
            ("rope_half", self.head_dim, self.theta, runtime.max_seq_len),
            (runtime.max_seq_len, self.head_dim // 2, 2), torch.float32,
            lambda table: runtime.kernels.rope_table(self.inv_freq, table))

    def apply(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Rotate x [tokens, heads, head_dim] in place by each token's absolute position."""
        self.rt.kernels.rope(x, positions, self.table)
        return x


def stretched_frequencies(dims: int, base: float, scaling) -> tuple[list[float], float]:
    """(the dims / 2 frequencies, the factor on cos and sin) under `scaling`: None, or a mapping with `kind` ("yarn":
    factor, original, fast, slow; "llama3": factor, original, low, high)."""
    import math
    freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling is None:
        return freqs, 1.0
    kind, factor, original = scaling["kind"], float(scaling["factor"]), float(scaling["original"])
    if kind == "yarn":
        turned = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(turned(float(scaling["fast"]))), 0)
        hi = min(math.ceil(turned(float(scaling["slow"]))), dims - 1)
        out = []
        for i, f in enumerate(freqs):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f / factor * ramp + f * (1.0 - ramp))
        return out, 0.1 * math.log(factor) + 1.0
    if kind == "llama3":
        low, high = float(scaling["low"]), float(scaling["high"])
        out = []
        for f in freqs:
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                out.append(f)
            elif wavelength > original / low:
                out.append(f / factor)
            else:
                share = (original / wavelength - low) / (high - low)
                out.append((1.0 - share) * f / factor + share * f)
        return out, 1.0
    raise ValueError(f"frequencies are stretched by 'yarn' or 'llama3', not {kind!r}")


class ScaledRotary(Part):
    """The cos/sin table of a rotation over a head's first `dims` dimensions with stretched frequencies; the mixer that
    owns it rotates inside its own kernels (`table`, `dims`).  One table for all layers with the same constants."""

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.dims, self.base = int(spec["dims"]), float(spec["base"])
        self.layout = spec.get("layout", "halves")
        if self.layout not in ("halves", "interleaved"):
            raise ValueError(f"a rotation pairs dimensions in 'halves' or 'interleaved', not {self.layout!r}")
        self.interleaved = self.layout == "interleaved"
        scaling = spec.get("scaling")
        if self.dims <= 0 or self.dims % 2:
            raise ValueError(f"a rotation turns an even number of dimensions, got {self.dims}")
        freqs, magnitude = stretched_frequencies(self.dims, self.base, scaling)
        self.magnitude = magnitude
        half = self.dims // 2
        reach = (runtime.max_seq_len + runtime.page_size - 1) // runtime.page_size * runtime.page_size     # whole pages
        key = ("rope_scaled", self.dims, self.base, tuple(sorted(scaling.items())) if scaling is not None else None, reach)
        freq = torch.tensor(freqs, dtype=torch.float64).to(torch.float32)

        def fill(table):
            runtime.kernels.rope_table(freq.to(runtime.device), table)
            if magnitude != 1.0:
                table.mul_(magnitude)
        self.table = runtime.shared_buffer(key, (reach, half, 2), torch.float32, fill)

    def apply(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError("a stretched rotation is applied by the mixer that owns it, inside its kernels")


class NoPosition(Part):
    def __init__(self, spec, runtime):
        self.table = None

    def apply(self, x, positions):
        return x


register_part("position", "rope_half", RotaryHalf)
register_part("position", "none", NoPosition)
register_part("position", "rope_scaled", ScaledRotary)
