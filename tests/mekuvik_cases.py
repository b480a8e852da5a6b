"""Shared by the Mekuvik tests on the GPU and, with the torch double of the kernel set, on the host: small
configurations whose sizes differ from each other in every respect, model folders with random weights made sharp
enough that a fault shows, the expectation from the plain implementation, and the check of a schedule."""

import json
import os

import torch
from safetensors.torch import load_file, save_file

import keranex_cases as K
import schedules
import tukevik_cases as T
from conftest import random_ids
from plain import mekuvik_plain as plain

YARN = lambda factor, original, fast, slow: dict(factor=factor, original=original, fast=fast, slow=slow)
ROT = lambda dims, base, scaling=None: dict(dims=dims, base=base, **({"scaling": scaling} if scaling else {}))
LIGHT = lambda heads, dim, vdim, decay: dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))
ATTN = lambda heads, kv, dim, vdim, scale, rot, window=None, keep=None: dict(
    heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, rot=rot,
    **({"mask": dict(size=window, **({"keep_first": keep} if keep is not None else {}))} if window else {}))
LATENT = lambda heads, dim, rot_dim, vdim, kv, q, scale, base, scaling=None: dict(
    heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv, q_rank=q, scale=scale, rot=ROT(rot_dim, base, scaling))
DENSE = lambda ff: dict(kind="dense", ff=ff)
MOE = lambda experts, top, ff, shared=None: dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top),
                                                 **({"shared": dict(ff=shared)} if shared else {}))

# The loop begins with the model's first layer and takes three passes (the embedding is added twice more, before a linear
# attention); a layer without a feed-forward; grouped attention whose keys, values and rotated dimensions all differ, a
# window that is no multiple of a page with three kept tokens (less than a page); two experts a token and a shared one;
# a latent attention behind the loop with stretched frequencies; widths that are no multiple of 16; logits times one half.
MEKUVIK_A = dict(
    architecture="Mekuvik", vocab=211, width=96, norm=dict(eps=1e-6), logit_scale=0.5,
    layers=[
        dict(type="lightning", mixer=LIGHT(3, 24, 20, (0.7, 0.95, 0.999)), mlp=None),
        dict(type="attention", mixer=ATTN(6, 2, 24, 16, 0.3, ROT(16, 100.0), 13, 3), mlp=MOE(6, 2, 20, 24)),
        dict(type="latent_attention", mixer=LATENT(3, 16, 8, 24, 40, 24, 0.2, 100.0, YARN(4.0, 32, 8.0, 2.0)), mlp=DENSE(72)),
    ],
    loop=dict(start=0, stop=2, times=3))
# One pass ("times" 1) over the model's end; no logit scale; a latent attention first, every expert chosen and none
# shared; a rotation over the whole head with stretched frequencies, a window of exactly two pages that keeps nothing; a
# window of a single position that keeps twenty tokens (more than two pages); one key head for all; linear attention of
# one head and of six.
MEKUVIK_B = dict(
    architecture="Mekuvik", vocab=130, width=64, norm=dict(eps=1e-5),
    layers=[
        dict(type="latent_attention", mixer=LATENT(5, 32, 16, 8, 72, 40, 0.15, 1e4), mlp=MOE(2, 2, 32)),
        dict(type="attention", mixer=ATTN(4, 4, 8, 24, 0.5, ROT(8, 1e6, YARN(2.0, 64, 16.0, 1.0)), 16, 0), mlp=None),
        dict(type="lightning", mixer=LIGHT(1, 40, 8, (0.9,)), mlp=DENSE(48)),
        dict(type="attention", mixer=ATTN(2, 1, 16, 16, 0.4, ROT(4, 50.0), 1, 20), mlp=MOE(8, 1, 8, 40)),
        dict(type="lightning", mixer=LIGHT(6, 8, 16, (0.5, 0.8, 0.9, 0.97, 0.99, 1.0)), mlp=MOE(3, 1, 40, 16)),
    ],
    loop=dict(start=3, stop=5, times=1))
# Sizes in multiples of 32 and 64 and pages of 16 - where the prompts' attention runs on the matrix cores in bfloat16 -, a
# loop in the middle that holds all three mixers' neighbours, an attention without any window, sixteen latent heads.
MEKUVIK_C = dict(
    architecture="Mekuvik", vocab=300, width=128, norm=dict(eps=1e-5), logit_scale=2.0,
    layers=[
        dict(type="attention", mixer=ATTN(8, 2, 64, 32, 0.125, ROT(32, 1e5), 50, 5), mlp=DENSE(192)),
        dict(type="lightning", mixer=LIGHT(4, 64, 64, (0.6, 0.9, 0.97, 0.999)), mlp=MOE(4, 2, 32, 64)),
        dict(type="latent_attention", mixer=LATENT(16, 32, 32, 32, 128, 64, 0.12, 1e4, YARN(8.0, 64, 32.0, 1.0)), mlp=MOE(4, 1, 64)),
        dict(type="attention", mixer=ATTN(2, 1, 128, 64, 0.1, ROT(64, 1e4)), mlp=None),
    ],
    loop=dict(start=1, stop=3, times=2))
MEKUVIK = {"A": (MEKUVIK_A, 51, 4), "B": (MEKUVIK_B, 52, 8), "C": (MEKUVIK_C, 53, 16)}        # config, weight seed, page size

LENGTHS, PROMPTS, POOL_TOKENS = K.LENGTHS, K.PROMPTS, K.POOL_TOKENS
# float32: a few hundred float32 operations and recurrences over a hundred tokens.  bfloat16: as served, against the plain
# float32 logits; a tenth of a request's positions may lie beyond where a rounded activation turns a router's close call.
LIMITS = {"float32": dict(max=2e-4, rms=2e-4), "bfloat16": dict(max=0.08, rms=0.1)}
BEYOND = {"float32": 0.0, "bfloat16": 0.1}


def sharpen(folder: str, raw: dict, seed: int = 0) -> None:
    """Random tensors of N(0, 0.02) hide faults: softmaxes are flat and one key more or less hardly shows, a linear
    attention's k v^T vanishes beside anything else, sigmoid gates and routers' scores all sit at one half, and the
    embedding that a pass adds again is lost beside the residual sum.  Normed queries are scaled through their norm's
    weight, the latent attention's up-projections and shared key rows through their matrices, the linear attention's
    projections, the gates, the routers and the embedding through theirs."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    scaled = lambda name, factor: (tensors[name].float() * factor).to(torch.bfloat16)
    tensors["embed"] = scaled("embed", 25.0)
    for index, layer in enumerate(raw["layers"]):
        p, m = f"l{index}.mix.", layer["mixer"]
        if layer["type"] == "lightning":
            for name, factor in (("q", 20.0), ("k", 20.0), ("v", 20.0), ("g", 30.0)):
                tensors[p + name] = scaled(p + name, factor)
        elif layer["type"] == "attention":
            tensors[p + "q.norm"] = scaled(p + "q.norm", 3.0)
            tensors[p + "v"] = scaled(p + "v", 4.0)
        else:
            for name, factor in (("uq", 30.0), ("uk", 30.0), ("uv", 5.0), ("g", 30.0)):
                tensors[p + name] = scaled(p + name, factor)
            down = tensors[p + "dkv"].float()
            down[m["kv_rank"]:] *= 8.0
            tensors[p + "dkv"] = down.to(torch.bfloat16)
        mlp = layer.get("mlp")
        if mlp is not None and mlp["kind"] == "moe":
            q = f"l{index}.mlp."
            tensors[q + "router"] = scaled(q + "router", 40.0)
            for name in [n for n in tensors if n.startswith(q) and n.endswith((".up", ".down"))]:
                tensors[name] = scaled(name, 4.0)
    save_file(tensors, path, metadata={"format": "pt"})


def make_folder(folder: str, raw: dict, seed: int) -> str:
    from ampere_kv_engine_amd.config import MekuvikConfig
    from ampere_kv_engine_amd.weights import write_random_model
    write_random_model(folder, MekuvikConfig.from_dict(raw), seed)
    sharpen(folder, raw, seed)
    return folder


def plain_logits(folder: str, ids: list[int]) -> torch.Tensor:
    with open(os.path.join(folder, "config.json")) as handle:
        raw = json.load(handle)
    return plain.forward(raw, load_file(os.path.join(folder, "model.safetensors")), ids)


def plain_greedy(folder: str, prompt: list[int], new_tokens: int) -> list[int]:
    ids, out = list(prompt), []
    for _ in range(new_tokens):
        out.append(int(plain_logits(folder, ids)[-1].argmax()))
        ids.append(out[-1])
    return out


def make_case(name: str, folder: str, config=None) -> dict:
    raw, seed, page_size = config if config is not None else MEKUVIK[name]
    make_folder(folder, raw, seed)
    requests = {r: random_ids(raw["vocab"], n, seed=500 + i) for i, (r, n) in enumerate(LENGTHS.items())}
    expected = {r: plain_logits(folder, ids) for r, ids in requests.items()}
    return dict(name=name, folder=folder, page_size=page_size, requests=requests, expected=expected, raw=raw)


make_engine = K.make_engine


def errors(got, want, dtype):
    saved = K.LIMITS, K.BEYOND
    K.LIMITS, K.BEYOND = LIMITS, BEYOND
    try:
        return K.errors(got, want, dtype)
    finally:
        K.LIMITS, K.BEYOND = saved


def assert_close(got, want, dtype: str, what: str = ""):
    position, by_max, by_rms = errors(got, want, dtype)
    if position is not None:
        raise AssertionError(f"{what}: first wrong position {position} of {want.reshape(-1, want.shape[-1]).shape[0]}; "
                             f"worst max error {by_max:.2f} x its limit, worst rms error {by_rms:.2f} x its limit ({dtype})")
    return max(by_max, by_rms)


def check(engine, case, schedule):
    got, pages = schedules.run(engine, case["requests"], schedule)
    dtype = engine.config.dtype
    worst = 0.0
    for name, want in case["expected"].items():
        worst = max(worst, assert_close(got[name], want, dtype, f"{case['name']}/{dtype} request {name}"))
    assert engine.cache.num_free_pages == [engine.config.num_pages] * len(engine.cache.groups), "pages were lost"
    assert engine.cache.slots.num_free == engine.config.max_seqs, "slots were lost"
    print(f"[mekuvik {case['name']} {dtype}] worst error {worst:.2f} of its limit")
    return pages


# ---- the cuttings (those of the other designs' cases, held to this design's limits) -----------------------------------

def _with_this_check(cutting):
    def run(engine, case, **more):
        saved = T.check, T.plain_logits, T.plain_greedy
        T.check, T.plain_logits, T.plain_greedy = check, plain_logits, plain_greedy
        try:
            return cutting(engine, case, **more)
        finally:
            T.check, T.plain_logits, T.plain_greedy = saved
    run.__name__ = cutting.__name__
    return run


case_whole = _with_this_check(T.case_whole)
case_prefill_then_token_by_token = _with_this_check(T.case_prefill_then_token_by_token)
case_token_by_token_from_the_first = _with_this_check(T.case_token_by_token_from_the_first)
case_portions_down_to_two_tokens = _with_this_check(T.case_portions_down_to_two_tokens)
case_mixed_with_pages_and_slots_used_again = _with_this_check(T.case_mixed_with_pages_and_slots_used_again)
case_first_tokens = _with_this_check(T.case_first_tokens)
case_long_decoding = _with_this_check(T.case_long_decoding)
case_greedy_generation = _with_this_check(T.case_greedy_generation)

CUTTINGS = [case_whole, case_prefill_then_token_by_token, case_token_by_token_from_the_first,
            case_portions_down_to_two_tokens, case_mixed_with_pages_and_slots_used_again, case_first_tokens,
            case_long_decoding, case_greedy_generation]


# ---- one mechanism alone: a small model in which nothing else contributes ----------------------------------------------

def alone(mechanism: str) -> tuple:
    """(config, weight seed, page size) of a small model in which one mechanism alone shapes the logits."""
    light = dict(type="lightning", mixer=LIGHT(2, 12, 20, (0.8, 0.995)), mlp=None)
    tiny = dict(type="lightning", mixer=LIGHT(1, 8, 8, (0.5,)), mlp=None)
    layers = {
        "linear attention": [light],
        "windowed attention": [dict(type="attention", mlp=None, mixer=ATTN(4, 2, 16, 24, 0.35, ROT(12, 1000.0), 11, 2))],
        "latent attention": [dict(type="latent_attention", mlp=None,
                                  mixer=LATENT(3, 12, 8, 20, 24, 16, 0.3, 200.0, YARN(3.0, 24, 6.0, 1.5)))],
        "dense feed-forward": [dict(tiny, mlp=DENSE(56))],
        "routed feed-forward": [dict(tiny, mlp=MOE(7, 3, 12, 20))],
        "passes": [light, dict(tiny, mlp=DENSE(24))],
    }
    raw = dict(architecture="Mekuvik", vocab=150, width=48, norm=dict(eps=1e-6), logit_scale=0.7, layers=layers[mechanism])
    if mechanism == "passes":
        raw["loop"] = dict(start=0, stop=2, times=4)
    return raw, 61 + sorted(layers).index(mechanism), 4


MECHANISMS = ("linear attention", "windowed attention", "latent attention", "dense feed-forward", "routed feed-forward",
              "passes")
