"""A plain, slow float32 implementation of the Lirulix decoder, one function per mechanism, written from the design's
equations and sharing no code with the engine.  Everything works on one whole sequence at a time: there is no cache,
no state and no batch here, so whatever the engine does with pages, slots and portions has to come out as if it had
not happened.  Recurrences are loops over the tokens; attentions are full score matrices with a mask.

Notation: n tokens, d model width.  Linear weights are [out, in] and applied as W x.  `dtype` is float32 everywhere
unless the caller asks for float64 (a reference for the float32 arithmetic itself).
"""

from __future__ import annotations

import math

import torch


# ---- small pieces ----------------------------------------------------------------------------------------------------

def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """The model's norm: its weight is stored around zero and applied as 1 + w."""
    return unit_rms(x, eps) * (1.0 + weight)


def unit_length(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """x / sqrt(sum(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


# ---- rotary positions and the two ways of stretching their frequencies -----------------------------------------------

def base_frequencies(dims: int, base: float) -> torch.Tensor:
    """f_i = base^(-2i / dims), i = 0 .. dims/2 - 1 (float64)."""
    return torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)


def yarn_frequencies(dims: int, base: float, scaling: dict) -> tuple[torch.Tensor, float]:
    """The frequencies after the ramp between stretched and unstretched ones, and the factor on cos and sin."""
    factor, original = float(scaling["factor"]), float(scaling["original"])
    f = base_frequencies(dims, base)

    def turned_dim(turns: float) -> float:            # the dimension whose wave makes `turns` turns over `original`
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turned_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turned_dim(float(scaling["slow"]))), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def llama3_frequencies(dims: int, base: float, scaling: dict) -> tuple[torch.Tensor, float]:
    factor, original = float(scaling["factor"]), float(scaling["original"])
    low, high = float(scaling["low"]), float(scaling["high"])
    out = []
    for f in base_frequencies(dims, base).tolist():
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=torch.float64), 1.0


def frequencies(rot: dict, kind: str) -> tuple[torch.Tensor, float]:
    """kind: "yarn" (the mixer `attention`) or "llama3" (`attention_2`); without `scaling` the plain frequencies."""
    scaling = rot.get("scaling")
    if scaling is None:
        return base_frequencies(rot["dims"], float(rot["base"])), 1.0
    return (yarn_frequencies if kind == "yarn" else llama3_frequencies)(rot["dims"], float(rot["base"]), scaling)


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict, kind: str) -> torch.Tensor:
    """x [n, heads, width]: dimension i of the first `dims` is turned with dimension i + dims/2 by position * f_i; the
    rest pass.  Angles are formed in float32 from float32 frequencies."""
    dims = rot["dims"]
    half = dims // 2
    freq, magnitude = frequencies(rot, kind)
    angle = positions.to(torch.float32)[:, None] * freq.to(torch.float32)[None, :]
    cos = (angle.cos() * magnitude).to(x.dtype)[:, None, :]
    sin = (angle.sin() * magnitude).to(x.dtype)[:, None, :]
    first, second = x[..., :half], x[..., half:dims]
    return torch.cat((first * cos - second * sin, second * cos + first * sin, x[..., dims:]), dim=-1)


# ---- attention with a learned sink -----------------------------------------------------------------------------------

def seen(n: int, window: int | None) -> torch.Tensor:
    """[n, n] True where query i sees key j: j <= i, and i - j < window where there is one."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    mask = j <= i
    if window is not None:
        mask = mask & (i - j < window)
    return mask


def softmax_with_sink(scores: torch.Tensor, mask: torch.Tensor, sink: torch.Tensor | None) -> torch.Tensor:
    """Softmax over the seen keys; with `sink` the denominator also holds exp(sink), which has no key and no value."""
    scores = scores.masked_fill(~mask, -math.inf)
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.expand_as(top))
    weights = torch.exp(scores - top)
    total = weights.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink - top)
    return weights / total


def sink_attention(h: torch.Tensor, w: dict, m: dict) -> torch.Tensor:
    n = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(n)
    q = rotate((h @ w["q"].T).view(n, heads, dim), positions, m["rot"], "yarn")
    k = rotate((h @ w["k"].T).view(n, groups, dim), positions, m["rot"], "yarn")
    v = (h @ w["v"].T).view(n, groups, vdim)
    mask = seen(n, m["mask"]["size"] if m.get("mask") else None)
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for head in range(heads):
        source = head // (heads // groups)
        scores = (q[:, head] @ k[:, source].T) * m["scale"]
        out[:, head] = softmax_with_sink(scores, mask, w["sink"][head]) @ v[:, source]
    return out.reshape(n, heads * vdim) @ w["o"].T


# ---- differential attention over a sliding window --------------------------------------------------------------------

def difference_weight(w: dict, diff: float) -> torch.Tensor:
    """lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer."""
    return torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + diff


def differential_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, groups, dim, vdim, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["diff"])
    positions = torch.arange(n)
    # rows lie head by head as [map 1, map 2]: 2 * heads (2 * groups) vectors of `dim`, each rotated by itself
    q = rotate((h @ w["q"].T).view(n, heads * 2, dim), positions, m["rot"], "llama3").view(n, heads, 2, dim)
    k = rotate((h @ w["k"].T).view(n, groups * 2, dim), positions, m["rot"], "llama3").view(n, groups, 2, dim)
    v = (h @ w["v"].T).view(n, groups, vdim)
    mask = seen(n, m["mask"]["size"] if m.get("mask") else None)
    lam = difference_weight(w, diff)
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for head in range(heads):
        source = head // (heads // groups)
        maps = [softmax_with_sink((q[:, head, i] @ k[:, source, i].T) * m["scale"], mask, None) @ v[:, source] for i in (0, 1)]
        out[:, head] = unit_rms(maps[0] - lam * maps[1], eps) * (1.0 - diff)
    out = out.reshape(n, heads * vdim) * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


# ---- the gated delta rule with a decay per key channel -----------------------------------------------------------------

def causal_conv(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x [n, channels]; weight [channels, taps], whose last column meets the current token; zeros before the start."""
    n, taps = x.shape[0], weight.shape[1]
    out = torch.zeros_like(x)
    for t in range(n):
        for tap in range(taps):
            source = t - (taps - 1 - tap)
            if source >= 0:
                out[t] += weight[:, tap] * x[source]
    return out


def delta_rule(q, k, v, beta, decay):
    """Per head, token after token: S <- decay * S (rows are key channels); u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q.  q, k, decay [n, heads, dim]; v [n, heads, vdim]; beta [n, heads]; returns o [n, heads, vdim]."""
    n, heads, dim = q.shape
    vdim = v.shape[-1]
    S = torch.zeros(heads, dim, vdim, dtype=q.dtype)
    out = torch.zeros(n, heads, vdim, dtype=q.dtype)
    for t in range(n):
        S = decay[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def channel_delta(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w["q"].T, w["q.conv"])).view(n, groups, dim)
    k = silu(causal_conv(h @ w["k"].T, w["k.conv"])).view(n, groups, dim)
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).view(n, heads, vdim)
    q = unit_length(q) * dim ** -0.5
    k = unit_length(k)
    share = heads // groups
    q, k = q.repeat_interleave(share, dim=1), k.repeat_interleave(share, dim=1)       # head h reads q/k head h // share
    beta = torch.sigmoid(h @ w["b"].T)
    rate = torch.exp(w["A_log"])[None, :, None]
    decay = torch.exp(-rate * softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(n, heads, dim))
    o = delta_rule(q, k, v, beta, decay)
    o = unit_rms(o, eps) * w["norm"]
    o = o * torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(n, heads, vdim)
    return o.reshape(n, heads * vdim) @ w["o"].T


# ---- feed-forward ----------------------------------------------------------------------------------------------------

def gated_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


# ---- the whole model -------------------------------------------------------------------------------------------------

def under(tensors: dict, prefix: str, dtype=torch.float32) -> dict:
    return {name[len(prefix):]: t.to(dtype) for name, t in tensors.items() if name.startswith(prefix)}


def layer_runs(raw: dict) -> list[tuple[int, int | None]]:
    """(layer, pass that begins with it or None) in the order the layers run: those from `start` to `stop` - 1 run
    `times` times in a row, then the rest."""
    count = len(raw["layers"])
    loop = raw.get("loop")
    if not loop:
        return [(i, None) for i in range(count)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None) for i in range(start)]
    for t in range(times):
        runs += [(i, t if i == start else None) for i in range(start, stop)]
    return runs + [(i, None) for i in range(stop, count)]


def forward(raw: dict, tensors: dict, ids: list[int], layer_outputs: list | None = None, dtype=torch.float32) -> torch.Tensor:
    """Logits [n, vocab] of one sequence.  `layer_outputs`: a list to which the residual sum after every layer run is
    added."""
    eps = float(raw["norm"]["eps"])
    get = lambda name: tensors[name].to(dtype)
    x = offset_norm(get("embed")[torch.tensor(ids)], get("embed.norm"), eps)
    for index, begins_pass in layer_runs(raw):
        layer = raw["layers"][index]
        if begins_pass is not None:
            x = x + get("loop.step")[begins_pass]
        w = under(tensors, f"l{index}.", dtype)
        h = offset_norm(x, w["norm1"], eps)
        mix = under(tensors, f"l{index}.mix.", dtype)
        if layer["type"] == "attention":
            mixed = sink_attention(h, mix, layer["mixer"])
        elif layer["type"] == "attention_2":
            mixed = differential_attention(h, mix, layer["mixer"], eps)
        elif layer["type"] == "channel_delta":
            mixed = channel_delta(h, mix, layer["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + mixed
        if layer.get("mlp") is not None:
            x = x + gated_ff(offset_norm(x, w["norm2"], eps), under(tensors, f"l{index}.mlp.", dtype))
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return offset_norm(x, get("final.norm"), eps) @ get("head").T
