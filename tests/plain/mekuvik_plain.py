"""A plain, slow implementation of the Mekuvik decoder, one function per mechanism, written from the design's equations
and sharing no code with the engine.  Everything works on one whole sequence at a time: there is no cache, no state and
no batch here, so whatever the engine does with pages, slots and portions has to come out as if it had not happened.
Recurrences are loops over the tokens; attentions are full score matrices with a mask.

Notation: n tokens, d model width.  Linear weights are [out, in] and applied as W x.  Arithmetic is float32 unless the
caller asks for float64.
"""

from __future__ import annotations

import math

import torch


# ---- small pieces ----------------------------------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


# ---- rotary positions ------------------------------------------------------------------------------------------------

def rotary_frequencies(dims: int, base: float, scaling: dict | None = None) -> tuple[torch.Tensor, float]:
    """(f_i for i = 0 .. dims/2 - 1 in float64, the factor on cos and sin).  f_i = base^(-2i / dims); with `scaling`
    (factor, original, fast, slow) a ramp over the pair index moves f_i to f_i / factor."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    if scaling is None:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, dims: int, freqs: torch.Tensor, magnitude: float = 1.0):
    """x [n, heads, width]: the first `dims` dimensions of every head are turned, dimension 2i with 2i + 1, by the angle
    position * f_i; cos and sin times `magnitude`.  The other dimensions pass."""
    angle = positions.to(x.dtype)[:, None] * freqs.to(x.dtype)[None, :]                 # [n, dims / 2]
    cos, sin = (torch.cos(angle) * magnitude)[:, None, :], (torch.sin(angle) * magnitude)[:, None, :]
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = even * cos - odd * sin
    out[..., 1:dims:2] = odd * cos + even * sin
    return out


# ---- masks -----------------------------------------------------------------------------------------------------------

def window_mask(n: int, size: int | None, keep_first: int = 0) -> torch.Tensor:
    """[n, n] bool: query i sees key j if j <= i and (i - j < size or j < keep_first); size None: every j <= i."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & ((i - j < size) | (j < keep_first))
    return seen


def masked_softmax(scores: torch.Tensor, seen: torch.Tensor) -> torch.Tensor:
    scores = scores.masked_fill(~seen, float("-inf"))
    return torch.softmax(scores, dim=-1)


# ---- mixers ----------------------------------------------------------------------------------------------------------

def lightning(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Linear attention with a decay per head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token."""
    n = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).view(n, heads, dim)
    k = silu(h @ w["k"].T).view(n, heads, dim)
    v = silu(h @ w["v"].T).view(n, heads, vdim)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    state = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    out = torch.empty(n, heads, vdim, dtype=h.dtype)
    for t in range(n):
        state = decay[:, None, None] * state + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", state, q[t])
    normed = rms_norm(out.reshape(n, heads * vdim), w["norm"], eps)
    return (normed * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Grouped-query attention; q and k normed over their whole projection; the first rot.dims dimensions of every head
    turned; a sliding window that also keeps a request's first tokens."""
    n = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w["q"].T, w["q.norm"], eps).view(n, heads, dim)
    k = rms_norm(h @ w["k"].T, w["k.norm"], eps).view(n, groups, dim)
    v = (h @ w["v"].T).view(n, groups, vdim)
    rot = m.get("rot")
    positions = torch.arange(n)
    if rot is not None:
        freqs, magnitude = rotary_frequencies(rot["dims"], float(rot["base"]), rot.get("scaling"))
        q = rotate_interleaved(q, positions, rot["dims"], freqs, magnitude)
        k = rotate_interleaved(k, positions, rot["dims"], freqs, magnitude)
    mask = m.get("mask")
    seen = window_mask(n, mask["size"] if mask else None, mask.get("keep_first", 0) if mask else 0)
    per = heads // groups
    out = torch.empty(n, heads, vdim, dtype=h.dtype)
    for head in range(heads):
        g = head // per
        scores = (q[:, head] @ k[:, g].T) * m["scale"]
        out[:, head] = masked_softmax(scores, seen) @ v[:, g]
    return out.reshape(n, heads * vdim) @ w["o"].T


def latent_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Attention whose keys and values are expanded from a latent per token; one turned key part for all heads; a
    sigmoid gate on the heads' outputs."""
    n = h.shape[0]
    heads, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(n, heads, dim + rot_dim)
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    shared_key = down[:, rank:].view(n, 1, rot_dim)
    rot = m["rot"]
    freqs, magnitude = rotary_frequencies(rot["dims"], float(rot["base"]), rot.get("scaling"))
    positions = torch.arange(n)
    q_turned = rotate_interleaved(q[..., dim:], positions, rot["dims"], freqs, magnitude)
    k_turned = rotate_interleaved(shared_key, positions, rot["dims"], freqs, magnitude)[:, 0]
    keys = (c @ w["uk"].T).view(n, heads, dim)
    values = (c @ w["uv"].T).view(n, heads, vdim)
    mask = m.get("mask")
    seen = window_mask(n, mask["size"] if mask else None, mask.get("keep_first", 0) if mask else 0)
    out = torch.empty(n, heads, vdim, dtype=h.dtype)
    for head in range(heads):
        scores = (q[:, head, :dim] @ keys[:, head].T + q_turned[:, head] @ k_turned.T) * m["scale"]
        out[:, head] = masked_softmax(scores, seen) @ values[:, head]
    gated = out.reshape(n, heads * vdim) * torch.sigmoid(h @ w["g"].T)
    return gated @ w["o"].T


MIXERS = {"lightning": lightning, "attention": attention, "latent_attention": latent_attention}


# ---- feed-forwards ---------------------------------------------------------------------------------------------------

def dense_feed_forward(h: torch.Tensor, w: dict) -> torch.Tensor:
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def small_expert(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return gelu_erf(h @ up.T) @ down.T


def routed_choice(h: torch.Tensor, router: torch.Tensor, top: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(chosen experts [n, top], their weights [n, top]): the largest sigmoid scores, weights as they are."""
    scores = torch.sigmoid(h @ router.T)
    order = torch.sort(h @ router.T, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(scores, 1, order)


def routed_feed_forward(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    """sum over the chosen experts of expert(weight * h), plus the shared expert of every token."""
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    chosen, weights = routed_choice(h, w["router"], top)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for slot in range(top):
            e = int(chosen[t, slot])
            out[t] += small_expert(weights[t, slot] * h[t], w[f"e{e}.up"], w[f"e{e}.down"])
    if mlp.get("shared") is not None:
        out = out + small_expert(h, w["shared.up"], w["shared.down"])
    return out


def feed_forward(h: torch.Tensor, w: dict, mlp: dict | None):
    if mlp is None:
        return None
    return dense_feed_forward(h, w) if mlp["kind"] == "dense" else routed_feed_forward(h, w, mlp)


# ---- the model -------------------------------------------------------------------------------------------------------

def sub_weights(weights: dict, prefix: str) -> dict:
    return {name[len(prefix):]: tensor for name, tensor in weights.items() if name.startswith(prefix)}


def layer(x: torch.Tensor, weights: dict, index: int, spec: dict, eps: float) -> torch.Tensor:
    """One norm, both sublayers read it: x + (mixer(h) + ff(h))."""
    h = rms_norm(x, weights[f"l{index}.norm1"], eps)
    branch = MIXERS[spec["type"]](h, sub_weights(weights, f"l{index}.mix."), spec["mixer"], eps)
    other = feed_forward(h, sub_weights(weights, f"l{index}.mlp."), spec.get("mlp"))
    if other is not None:
        branch = branch + other
    return x + branch


def run_order(config: dict) -> list[tuple[int, bool]]:
    """(layer, whether the embedding's output is added before it) in the order the layers run."""
    count, loop = len(config["layers"]), config.get("loop")
    if loop is None:
        return [(i, False) for i in range(count)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(start)]
    for turn in range(times):
        order += [(i, turn > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, count)]


def forward(config: dict, weights: dict, tokens, dtype=torch.float32, streams: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one whole sequence.  `streams`, if given, collects the residual sum after every layer run."""
    weights = {name: t.to(dtype) if t.is_floating_point() else t for name, t in weights.items()}
    eps = float(config["norm"]["eps"])
    start = weights["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = start
    for index, adds_start in run_order(config):
        if adds_start:
            x = x + start
        x = layer(x, weights, index, config["layers"][index], eps)
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, weights["final.norm"], eps) @ weights["embed"].T * float(config.get("logit_scale", 1.0))
