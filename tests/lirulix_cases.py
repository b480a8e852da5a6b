"""Shared by the Lirulix tests on the GPU and, with the torch double of the kernel set, on the host: small
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
from plain import lirulix_plain as plain

YARN = lambda factor, original, fast, slow: dict(factor=factor, original=original, fast=fast, slow=slow)
LLAMA3 = lambda factor, original, low, high: dict(factor=factor, original=original, low=low, high=high)
ROT = lambda dims, base, scaling=None: dict(dims=dims, base=base, **({"scaling": scaling} if scaling else {}))
SINK = lambda heads, kv, dim, vdim, scale, rot, window=None: dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, rot=rot,
                                                                  **({"mask": dict(size=window)} if window else {}))
DIFF = lambda heads, kv, dim, vdim, scale, rot, window, diff: dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, rot=rot,
                                                                   diff=diff, **({"mask": dict(size=window)} if window else {}))
DELTA = lambda heads, kv, dim, vdim, conv, decay_rank, gate_rank: dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, conv=conv,
                                                                       ranks=dict(decay=decay_rank, gate=gate_rank))
DENSE = lambda ff: dict(kind="dense", ff=ff)

# The loop begins with the model's first layer (its first vector meets the embedding's norm) and takes three passes; a
# delta rule first and without a feed-forward, two heads a key head, four taps; grouped attention whose keys, values and
# rotated dimensions all differ; a window that is no multiple of a page; widths that are no multiple of 16.
LIRULIX_A = dict(
    architecture="Lirulix", vocab=211, width=96, norm=dict(eps=1e-6),
    layers=[
        dict(type="channel_delta", mixer=DELTA(4, 2, 24, 20, 4, 8, 12), mlp=None),
        dict(type="attention", mixer=SINK(6, 2, 24, 16, 0.3, ROT(16, 100.0, YARN(4.0, 32, 8.0, 2.0))), mlp=DENSE(72)),
        dict(type="attention_2", mixer=DIFF(3, 3, 16, 40, 0.4, ROT(8, 50.0, LLAMA3(4.0, 16, 1.0, 4.0)), 13, 0.2), mlp=DENSE(40)),
    ],
    loop=dict(start=0, stop=2, times=3))
# One pass ("times" 1) over the model's end; one key head for all; a window of exactly two pages and a window of a single
# position (a query sees itself alone - and the sink); a sink attention with a window; no stretching of the frequencies;
# a rotation over the whole head; a convolution of one tap (no inputs kept) and of two; a delta rule of one head.
LIRULIX_B = dict(
    architecture="Lirulix", vocab=130, width=64, norm=dict(eps=1e-5),
    layers=[
        dict(type="attention_2", mixer=DIFF(4, 1, 32, 32, 0.25, ROT(32, 1e4), 16, 0.5), mlp=None),
        dict(type="channel_delta", mixer=DELTA(1, 1, 40, 8, 1, 4, 4), mlp=DENSE(48)),
        dict(type="attention", mixer=SINK(4, 4, 8, 24, 0.5, ROT(4, 1e6, YARN(2.0, 64, 16.0, 1.0)), window=1), mlp=DENSE(32)),
        dict(type="channel_delta", mixer=DELTA(6, 3, 8, 16, 2, 16, 8), mlp=None),
        dict(type="attention_2", mixer=DIFF(2, 2, 8, 8, 0.6, ROT(8, 100.0, LLAMA3(8.0, 64, 1.0, 2.0)), 1, 0.1), mlp=DENSE(56)),
    ],
    loop=dict(start=3, stop=5, times=1))
# Sizes in multiples of 32 and 64 and pages of 16 - where the prompts' attention runs on the matrix cores in bfloat16 -,
# no loop at all, a window longer than most requests.
LIRULIX_C = dict(
    architecture="Lirulix", vocab=300, width=128, norm=dict(eps=1e-5),
    layers=[
        dict(type="attention", mixer=SINK(8, 2, 64, 32, 0.125, ROT(32, 1e5, YARN(2.0, 64, 32.0, 1.0))), mlp=DENSE(192)),
        dict(type="channel_delta", mixer=DELTA(4, 4, 64, 64, 3, 16, 16), mlp=DENSE(64)),
        dict(type="attention_2", mixer=DIFF(4, 2, 32, 64, 0.2, ROT(32, 1e4, LLAMA3(8.0, 128, 1.0, 4.0)), 50, 0.3), mlp=None),
        dict(type="attention_2", mixer=DIFF(2, 1, 64, 128, 0.15, ROT(16, 1e4), 200, 0.25), mlp=DENSE(128)),
    ])
LIRULIX = {"A": (LIRULIX_A, 31, 4), "B": (LIRULIX_B, 32, 8), "C": (LIRULIX_C, 33, 16)}        # config, weight seed, page size

LENGTHS, PROMPTS, POOL_TOKENS = K.LENGTHS, K.PROMPTS, K.POOL_TOKENS
# float32: a few hundred float32 operations and recurrences over a hundred tokens.  bfloat16: as served, against the plain
# float32 logits.
LIMITS = {"float32": dict(max=2e-4, rms=2e-4), "bfloat16": dict(max=0.08, rms=0.1)}
BEYOND = {"float32": 0.0, "bfloat16": 0.0}


def sharpen(folder: str, raw: dict, seed: int = 0) -> None:
    """Random tensors of N(0, 0.02) hide faults: softmaxes are flat and one key more or less hardly shows, sinks of 0.02
    all weigh the same, a delta rule whose decay is exp(-softplus(0)) forgets its state within two tokens, convolutions
    with weights of 0.02 pass almost nothing of the earlier inputs, lambda is its constant and the vectors of the passes
    vanish beside the residual sum.  Queries and keys are scaled up, sinks spread over several units, decays drawn
    between 0.7 and 0.999 with a visible share from the token, convolutions, gates and pass vectors scaled up."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    generator = torch.Generator().manual_seed(2000 + seed)
    scaled = lambda name, factor: (tensors[name].float() * factor).to(torch.bfloat16)
    for index, layer in enumerate(raw["layers"]):
        p = f"l{index}.mix."
        if layer["type"] == "channel_delta":
            heads = layer["mixer"]["heads"]
            tensors[p + "A_log"] = (-4.5 + 3.5 * torch.rand(heads, generator=generator)).to(torch.bfloat16)
            for name, factor in (("q.conv", 20.0), ("k.conv", 20.0), ("v.conv", 20.0), ("q", 5.0), ("k", 5.0), ("v", 5.0),
                                 ("a1", 10.0), ("a2", 10.0), ("g1", 10.0), ("g2", 10.0), ("b", 40.0), ("dt_bias", 20.0)):
                tensors[p + name] = scaled(p + name, factor)
        else:
            for name in ("q", "k"):
                tensors[p + name] = scaled(p + name, 12.0)
            tensors[p + "v"] = scaled(p + "v", 4.0)
            if layer["type"] == "attention":
                tensors[p + "sink"] = scaled(p + "sink", 100.0)
            else:
                tensors[p + "g"] = scaled(p + "g", 10.0)
                for name in ("lq1", "lk1", "lq2", "lk2"):
                    tensors[p + name] = scaled(p + name, 12.0)
    if "loop.step" in tensors:
        tensors["loop.step"] = scaled("loop.step", 25.0)
    save_file(tensors, path, metadata={"format": "pt"})


def make_folder(folder: str, raw: dict, seed: int) -> str:
    from ampere_kv_engine_amd.config import LirulixConfig
    from ampere_kv_engine_amd.weights import write_random_model
    write_random_model(folder, LirulixConfig.from_dict(raw), seed)
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
    raw, seed, page_size = config if config is not None else LIRULIX[name]
    make_folder(folder, raw, seed)
    requests = {r: random_ids(raw["vocab"], n, seed=400 + i) for i, (r, n) in enumerate(LENGTHS.items())}
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
    print(f"[lirulix {case['name']} {dtype}] worst error {worst:.2f} of its limit")
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


# ---- one mechanism alone: a model of one layer in which nothing else contributes --------------------------------------

def alone(mechanism: str) -> tuple:
    """(config, weight seed, page size) of a small model in which one mechanism alone shapes the logits."""
    delta = dict(type="channel_delta", mixer=DELTA(2, 1, 12, 20, 3, 6, 10), mlp=None)
    tiny = dict(type="channel_delta", mixer=DELTA(1, 1, 8, 8, 1, 2, 2), mlp=None)
    layers = {
        "attention with a sink": [dict(type="attention", mlp=None,
                                       mixer=SINK(4, 2, 16, 24, 0.35, ROT(12, 1000.0, YARN(3.0, 24, 6.0, 1.5))))],
        "differential attention": [dict(type="attention_2", mlp=None,
                                        mixer=DIFF(4, 2, 16, 12, 0.35, ROT(16, 200.0, LLAMA3(4.0, 32, 1.0, 4.0)), 11, 0.35))],
        "delta rule": [delta],
        "feed-forward": [dict(tiny, mlp=DENSE(56))],
        "passes": [delta, dict(tiny, mlp=DENSE(24))],
    }
    raw = dict(architecture="Lirulix", vocab=150, width=48, norm=dict(eps=1e-6), layers=layers[mechanism])
    if mechanism == "passes":
        raw["loop"] = dict(start=0, stop=2, times=4)
    return raw, 41 + sorted(layers).index(mechanism), 4


MECHANISMS = ("attention with a sink", "differential attention", "delta rule", "feed-forward", "passes")
