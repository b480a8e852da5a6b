"""Lirulix on the GPU: every kernel of its own against the plain implementation's function of the same mechanism, and
the engine with the HIP kernels through the cuttings of `lirulix_cases` - float32 against tight limits, bfloat16 as
it is served."""

import json
import math
import os
import random
import subprocess
import sys
from types import SimpleNamespace

import pytest
import torch

import lirulix_cases as L
import schedules
from conftest import ROOT
from plain import lirulix_plain as plain
from test_tukevik_gpu import _ctx

pytestmark = pytest.mark.gpu
DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def hip():
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return HipKernels(DEVICE)


@pytest.fixture(scope="module", params=list(L.LIRULIX))
def case(request, tmp_path_factory):
    return L.make_case(request.param, str(tmp_path_factory.mktemp(f"lirulix_{request.param}")))


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, case):
    return L.make_engine(case, request.param, DEVICE)


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("cutting", L.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is L.case_greedy_generation and engine.config.dtype != "float32":
        pytest.skip("greedy tokens are compared with the plain float32 implementation's")
    cutting(engine, case)
    assert engine.kernels.parts_library_path.endswith("libakv_parts.so")


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mechanism", L.MECHANISMS)
def test_one_mechanism_alone(mechanism, dtype, tmp_path):
    case = L.make_case(mechanism, str(tmp_path), L.alone(mechanism))
    engine = L.make_engine(case, dtype, DEVICE)
    L.case_whole(engine, case)
    L.case_prefill_then_token_by_token(engine, case)
    L.case_portions_down_to_two_tokens(engine, case)
    L.case_mixed_with_pages_and_slots_used_again(engine, case)


def test_steps_are_recorded_and_replayed(case):
    """Decode steps come again and again: the second is recorded, the later ones are replays; all agree with the plain
    implementation, and with an engine that records nothing to a few units in the last place (a recording cuts a row's keys
    over waves by a bound on the request's length, an eager step by the length itself: the order of the sums differs where
    no window bounds the keys)."""
    ids = case["requests"]["d"]
    want = case["expected"]["d"]
    outs = {}
    for graphs in (True, False):
        engine = L.make_engine(case, "float32", DEVICE, decode_graphs=graphs)
        got, _ = schedules.run(engine, {"d": ids}, schedules.last_one_by_one({"d": ids}, 60))
        L.assert_close(got["d"], want, "float32", f"graphs {graphs}")
        outs[graphs] = got["d"]
        if graphs:
            assert any(g is not None for g in engine._graphs.values()), "nothing was recorded"
    torch.testing.assert_close(outs[True], outs[False], rtol=0, atol=2e-5 * float(want.abs().max()))


def test_trace_replay_of_a_random_model(case, tmp_path):
    """bin/trace_run on a configuration file and a seed: the mixed cutting, every position against the plain model."""
    from ampere_kv_engine_amd.config import LirulixConfig
    from ampere_kv_engine_amd.weights import write_random_model
    import numpy as np
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), LirulixConfig.from_dict(case["raw"]), 9)
    requests = {name: case["requests"][name] for name in ("a", "b", "e")}
    schedule = schedules.mixed(requests, L.PROMPTS, 16, 64, seed=3)
    out = tmp_path / "out"
    lines = "\n".join(json.dumps(r) for r in schedules.to_trace(requests, schedule)) + "\n"
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--random-config", str(config_path),
                           "--weights-seed", "9", "--dtype", "float32", "--out", str(out), "--max-tokens", "1024"],
                          input=lines, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [l for l in done.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(schedule))]
    fed = {name: 0 for name in requests}
    for number, (entries, _) in enumerate(schedule):
        got = torch.from_numpy(np.fromfile(out / f"{number}.f32", dtype="<f4").reshape(-1, case["raw"]["vocab"]).copy())
        row = 0
        for name, count in entries:
            want = L.plain_logits(folder, requests[name][:fed[name] + count])[fed[name]:]
            L.assert_close(got[row:row + count], want, "float32", f"step {number} request {name}")
            fed[name] += count
            row += count


def test_the_command_line_generates_with_a_lirulix_model(case, tmp_path):
    """`python -m ampere_kv_engine_amd.runner` on a configuration file and a seed: one request, and several through the
    scheduler, greedy; the tokens of the plain implementation."""
    import re
    from ampere_kv_engine_amd.config import LirulixConfig
    from ampere_kv_engine_amd.weights import write_random_model
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), LirulixConfig.from_dict(case["raw"]), 5)
    prompts = [case["requests"]["a"][:19], case["requests"]["b"][:6], case["requests"]["c"][:31]]
    want = [L.plain_greedy(folder, ids, 6) for ids in prompts]
    base = [sys.executable, "-m", "ampere_kv_engine_amd.runner", "--random-config", str(config_path), "--weights-seed", "5",
            "--max-new-tokens", "6", "--ignore-eos"]
    run = lambda more: subprocess.run(base + more, capture_output=True, text=True, timeout=600, cwd=ROOT)
    one = run(["--mode", "generate", "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompts[0])), "--prefill-chunk", "8"])
    assert one.returncode == 0, one.stderr[-2000:]
    assert json.loads(re.search(r"generated_token_ids = (\[.*\])", one.stdout).group(1)) == want[0]
    prompts_file = tmp_path / "prompts.txt"
    prompts_file.write_text("\n".join(" ".join(map(str, ids)) for ids in prompts) + "\n")
    many = run(["--mode", "generate", "--dtype", "float32", "--prompts-file", str(prompts_file), "--max-seqs", "2",
                "--prefill-chunk", "5"])
    assert many.returncode == 0, many.stderr[-2000:]
    got = [json.loads(line)["generated_token_ids"] for line in many.stdout.splitlines() if line.startswith("{")]
    assert got == want, many.stdout
    check = run(["--mode", "check", "--prompt-len", "40"])
    assert check.returncode == 0, check.stdout[-1500:] + check.stderr[-1500:]


def random_configuration(seed: int) -> tuple:
    """Sizes, constants, the order of layers and the passes drawn from a seed: any head counts and groupings, keys, values
    and rotated dimensions of different widths (some no multiple of 8), windows from one position to longer than a
    request, any number of taps, layers without a feed-forward, stretched and unstretched frequencies."""
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.choice((2, 3, 4, 5))):
        mlp = rng.choice((None, L.DENSE(rng.choice((40, 64, 100, 132)))))
        kind = rng.choice(("attention", "attention_2", "channel_delta"))
        kv, group = rng.choice((1, 2, 3)), rng.choice((1, 2, 4, 5))
        dim = rng.choice((8, 12, 32, 64, 80))
        vdim = rng.choice((4, 8, 24, 64, 72))
        if kind == "channel_delta":
            layers.append(dict(type=kind, mlp=mlp, mixer=L.DELTA(kv * group, kv, dim, vdim, rng.choice((1, 2, 3, 4, 5)),
                                                                 rng.choice((2, 8, 24)), rng.choice((4, 8, 16)))))
            continue
        dims = rng.choice([d for d in (2, 4, 8, 12, 32, 64) if d <= dim])
        window = rng.choice((None, 1, 2, 5, 16, 31, 64, 100, 500))
        original = rng.choice((16, 64, 256))
        if kind == "attention":
            scaling = rng.choice((None, L.YARN(rng.choice((2.0, 4.0, 16.0)), original, rng.choice((8.0, 32.0)), rng.choice((0.5, 1.0, 2.0)))))
            mixer = L.SINK(kv * group, kv, dim, vdim, rng.uniform(0.1, 0.5), L.ROT(dims, rng.choice((100.0, 1e4, 1e6)), scaling), window)
        else:
            scaling = rng.choice((None, L.LLAMA3(rng.choice((2.0, 8.0)), original, 1.0, rng.choice((2.0, 4.0, 8.0)))))
            mixer = L.DIFF(kv * group, kv, dim, vdim, rng.uniform(0.1, 0.5), L.ROT(dims, rng.choice((100.0, 1e4, 1e6)), scaling),
                           window, rng.choice((0.1, 0.3, 0.8)))
        layers.append(dict(type=kind, mlp=mlp, mixer=mixer))
    raw = dict(architecture="Lirulix", vocab=rng.choice((97, 260, 1000)), width=rng.choice((40, 72, 96, 120, 192)),
               norm=dict(eps=rng.choice((1e-5, 1e-6))), layers=layers)
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        raw["loop"] = dict(start=start, stop=rng.randint(start + 1, len(layers)), times=rng.choice((1, 2, 3)))
    return raw, seed, rng.choice((4, 8, 16, 32))


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("seed", range(600, 608))
def test_a_random_configuration_through_the_cuttings(seed, tmp_path):
    config = random_configuration(seed)
    print(f"seed {seed}: {config[0]}, pages of {config[2]}", flush=True)
    case = L.make_case(f"random {seed}", str(tmp_path), config)
    for dtype in ("float32", "bfloat16"):
        engine = L.make_engine(case, dtype, DEVICE)
        L.case_whole(engine, case)
        L.case_portions_down_to_two_tokens(engine, case)
        L.case_prefill_then_token_by_token(engine, case)
        L.case_mixed_with_pages_and_slots_used_again(engine, case)


# ---- the kernels one by one, against the plain functions ----------------------------------------------------------------

def _pages_for(lengths, page, kv_heads, key_width, vdim, dtype):
    """Pages in a shuffled order for requests of `lengths` tokens: (k_pages, v_pages, block table)."""
    needed = sum((n + page - 1) // page for n in lengths)
    k_pages = torch.zeros(needed + 2, kv_heads, page, key_width, dtype=dtype, device=DEVICE)
    v_pages = torch.zeros(needed + 2, kv_heads, vdim, page, dtype=dtype, device=DEVICE)
    order = torch.randperm(needed + 2).tolist()
    table = torch.full((len(lengths), max((n + page - 1) // page for n in lengths)), -1, dtype=torch.int32)
    for r, n in enumerate(lengths):
        for i in range((n + page - 1) // page):
            table[r, i] = order.pop()
    return k_pages, v_pages, table


def _through_the_attention(hip, rows, lengths, steps, page, heads, kv_heads, dim, vdim, maps, rot, kind, scale, window, sinks, dtype):
    """The projected rows of two requests through the rotation with its cache write and the attention, step by step."""
    freqs, magnitude = plain.frequencies(rot, kind)
    table = torch.empty(max(lengths) + page, rot["dims"] // 2, 2, dtype=torch.float32, device=DEVICE)
    hip.rope_table(freqs.float().to(DEVICE), table)
    table.mul_(magnitude)
    k_pages, v_pages, block_table = _pages_for(lengths, page, kv_heads, maps * dim, vdim, dtype)
    got = [torch.zeros(n, heads * maps * vdim) for n in lengths]
    for befores, counts in steps:
        ctx = _ctx(befores, counts)
        projected = torch.cat([rows[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        slot_map = torch.tensor([int(block_table[r, p // page]) * page + p % page for r, (b, c) in enumerate(zip(befores, counts))
                                 for p in range(b, b + c)], dtype=torch.int32, device=DEVICE)
        meta = SimpleNamespace(block_table=block_table.to(DEVICE), rows=None, width=block_table.shape[1], slot_map=slot_map)
        q = torch.empty(ctx.num_tokens, heads * maps * dim, dtype=dtype, device=DEVICE)
        out = torch.empty(ctx.num_tokens, heads * maps * vdim, dtype=dtype, device=DEVICE)
        hip.unit_norm_write(projected, heads, kv_heads, dim, vdim, None, slot_map, k_pages, v_pages, q, maps=maps, table=table,
                            rot_dims=rot["dims"], positions=ctx.positions)
        hip.gated_attention(q, k_pages, v_pages, None, 0, ctx, meta, heads, kv_heads, dim, vdim, scale, None, None, window,
                            sinks is not None, out, sink_logits=sinks, maps=maps)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    return got


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,dims,page,window", [
    (4, 2, 16, 24, 12, 4, None), (3, 1, 40, 8, 40, 16, None), (8, 2, 64, 64, 32, 16, None), (2, 1, 128, 256, 64, 16, None),
    (8, 8, 64, 32, 64, 8, 20), (2, 2, 32, 128, 2, 32, 33), (1, 1, 256, 32, 128, 16, None)])
def test_attention_with_a_sink_alone(hip, dtype, heads, kv_heads, dim, vdim, dims, page, window):
    """Two requests in two portions each and a last token alone, against the plain attention of the whole sequences.  Scores
    are made sharp; the first key of each request is made to stand out for every later query, however far (hundreds of
    positions in the long request) - while no window hides it; the sinks differ from head to head by several units."""
    torch.manual_seed(heads * 100 + dim)
    lengths, scale = (75, 700 if dim <= 64 else 330), 1.2 / math.sqrt(dim)
    rot = dict(dims=dims, base=1000.0, scaling=L.YARN(4.0, 64, 16.0, 1.0))
    width = heads * dim + kv_heads * (dim + vdim)
    rows = [torch.randn(n, width) for n in lengths]
    for projected in rows:
        projected[0, heads * dim + dims:heads * dim + dim] = projected[1:, dims:dim].mean(0) * 30 if dims < dim else 0.0
    rows = [r.to(dtype).float() for r in rows]
    sinks = (torch.randn(heads) * 3).to(DEVICE)
    steps = [((0, 0), (41, 5)), ((41, 5), (lengths[0] - 42, lengths[1] - 6)), ((lengths[0] - 1, lengths[1] - 1), (1, 1))]
    got = _through_the_attention(hip, rows, lengths, steps, page, heads, kv_heads, dim, vdim, 1, rot, "yarn", scale, window,
                                 sinks, dtype)
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot, **({"mask": dict(size=window)} if window else {}))
    qk = heads * dim + kv_heads * dim
    pick = lambda lo, hi: torch.eye(width)[lo:hi]
    w = {"q": pick(0, heads * dim), "k": pick(heads * dim, qk), "v": pick(qk, width), "o": torch.eye(heads * vdim), "sink": sinks.cpu()}
    for r, n in enumerate(lengths):
        want = plain.sink_attention(rows[r], w, m)
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (3e-5 if dtype == torch.float32 else 0.03), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,dims,page,window", [
    (4, 2, 16, 12, 16, 4, 11), (3, 3, 24, 40, 8, 16, 16), (4, 2, 32, 64, 32, 16, 50), (2, 1, 64, 128, 16, 16, 130),
    (2, 2, 8, 8, 8, 8, 1), (1, 1, 128, 32, 64, 32, None)])
def test_differential_attention_alone(hip, dtype, heads, kv_heads, dim, vdim, dims, page, window):
    """The two maps of every head through rotation, cache and attention, then the difference, its norm and the gates,
    against the plain mixer with identity projections.  A key at position 9 stands out in map 1 of every head: queries see
    it exactly while it lies in their window, in prompts and in the tokens that follow alone."""
    torch.manual_seed(heads * 10 + dim)
    lengths, scale, diff, eps = (90, 9 + (window or 40) + 6), 1.5 / math.sqrt(dim), 0.3, 1e-6
    rot = dict(dims=dims, base=500.0, scaling=L.LLAMA3(8.0, 32, 1.0, 4.0))
    q_size, k_size, v_size, o_size = heads * 2 * dim, kv_heads * 2 * dim, kv_heads * vdim, heads * vdim
    width = q_size + k_size + v_size + o_size
    rows = [torch.randn(n, width) for n in lengths]
    for projected in rows:           # (the part of map 1's key that the rotation leaves alone, along the queries' mean)
        if dims < dim:
            for g in range(kv_heads):
                projected[9, q_size + g * 2 * dim + dims:q_size + g * 2 * dim + dim] = projected[10:, dims:dim].mean(0) * 25
    rows = [r.to(dtype).float() for r in rows]
    tail = 4
    steps = [((0, 0), (30, 7)), ((30, 7), (lengths[0] - 30 - tail, lengths[1] - 7 - tail))]
    steps += [((lengths[0] - tail + i, lengths[1] - tail + i), (1, 1)) for i in range(tail)]
    maps = _through_the_attention(hip, rows, lengths, steps, page, heads, kv_heads, dim, vdim, 2, rot, "llama3", scale, window,
                                  None, dtype)
    lam_vectors = {name: torch.randn(dim) * 0.3 for name in ("lq1", "lk1", "lq2", "lk2")}
    lam = plain.difference_weight(lam_vectors, diff).reshape(1).to(DEVICE)
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot, diff=diff,
             **({"mask": dict(size=window)} if window else {}))
    pick = lambda lo, hi: torch.eye(width)[lo:hi]
    w = dict(lam_vectors, q=pick(0, q_size), k=pick(q_size, q_size + k_size), v=pick(q_size + k_size, q_size + k_size + v_size),
             g=pick(q_size + k_size + v_size, width), o=torch.eye(o_size))
    for r, n in enumerate(lengths):
        out = torch.empty(n, o_size, dtype=dtype, device=DEVICE)
        hip.difference_norm_gate(maps[r].to(dtype).to(DEVICE), lam, eps, 1.0 - diff, rows[r].to(dtype).to(DEVICE),
                                 q_size + k_size + v_size, heads, vdim, out)
        want = plain.differential_attention(rows[r], w, m, eps)
        error = (out.float().cpu() - want).abs().max() / want.abs().max()
        assert error < (5e-5 if dtype == torch.float32 else 0.05), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,groups,dim,vdim,taps", [(4, 2, 24, 20, 4), (1, 1, 40, 8, 1), (6, 3, 8, 16, 2), (4, 4, 64, 64, 3),
                                                        (2, 1, 128, 128, 4), (2, 2, 300, 72, 2), (16, 16, 128, 128, 4)])
def test_delta_rule_kernels_alone(hip, dtype, heads, groups, dim, vdim, taps):
    """Convolutions with the inputs they keep, the unit vectors, decays, betas, the recurrence over steps of several
    requests and the gated norm, against the plain functions; a slot that is used again starts from zero."""
    torch.manual_seed(dim + vdim)
    lengths, unit_eps, eps = (70, 9), 1e-6, 1e-5
    qk, vs = groups * dim, heads * vdim
    channels = 2 * qk + vs
    width = channels + heads
    rows = [(torch.randn(n, width) * 2).to(dtype).float() for n in lengths]
    decay_logits = [torch.randn(n, heads * dim) for n in lengths]
    gate_logits = [torch.randn(n, vs) * 2 for n in lengths]
    conv = (torch.randn(channels, taps) * 0.5).to(dtype)
    a_log, dt_bias = -4.0 + 3.5 * torch.rand(heads), torch.randn(heads * dim) * 0.5
    norm_weight = 1 + 0.2 * torch.randn(vdim)
    state = torch.full((3, heads * dim * vdim + (taps - 1) * channels), 7.0, dtype=torch.float32, device=DEVICE)
    state[:2] = 0.0
    got = [torch.zeros(n, vs) for n in lengths]
    for befores, counts in (((0, 0), (33, 2)), ((33, 2), (1, 1)), ((34, 3), (36, 6))):
        ctx = _ctx(befores, counts)
        cut = lambda parts: torch.cat([parts[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))])
        projected = cut(rows).to(dtype).to(DEVICE)
        tokens = projected.shape[0]
        conved = torch.empty(tokens, channels, dtype=dtype, device=DEVICE)
        hip.conv_silu(projected, channels, conv.to(DEVICE), None, state, 0, ctx, conved, conv_at=heads * dim * vdim)
        out = torch.empty(tokens, vs, dtype=dtype, device=DEVICE)
        hip.delta_rule(conved, projected, channels, cut(decay_logits).to(DEVICE), dt_bias.to(DEVICE), torch.exp(a_log).to(DEVICE),
                       cut(gate_logits).to(DEVICE), norm_weight.to(DEVICE), unit_eps, eps, dim ** -0.5, heads, groups, dim, vdim,
                       state, ctx, out)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    assert (state[2] == 7.0).all()
    share = heads // groups
    for r, n in enumerate(lengths):
        x = rows[r]
        split = lambda lo, hi, kernel: plain.silu(plain.causal_conv(x[:, lo:hi], kernel.float()))
        q = plain.unit_length(split(0, qk, conv[:qk]).view(n, groups, dim), unit_eps) * dim ** -0.5
        k = plain.unit_length(split(qk, 2 * qk, conv[qk:2 * qk]).view(n, groups, dim), unit_eps)
        v = split(2 * qk, channels, conv[2 * qk:]).view(n, heads, vdim)
        if dtype == torch.bfloat16:      # (the kernels read the convolutions' rounded outputs)
            q = plain.unit_length(split(0, qk, conv[:qk]).to(dtype).float().view(n, groups, dim), unit_eps) * dim ** -0.5
            k = plain.unit_length(split(qk, 2 * qk, conv[qk:2 * qk]).to(dtype).float().view(n, groups, dim), unit_eps)
            v = v.to(dtype).float()
        beta = torch.sigmoid(x[:, channels:])
        decay = torch.exp(-torch.exp(a_log)[None, :, None] * plain.softplus(decay_logits[r] + dt_bias).view(n, heads, dim))
        o = plain.delta_rule(q.repeat_interleave(share, dim=1), k.repeat_interleave(share, dim=1), v, beta, decay)
        want = (plain.unit_rms(o, eps) * norm_weight * torch.sigmoid(gate_logits[r]).view(n, heads, vdim)).reshape(n, vs)
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (3e-5 if dtype == torch.float32 else 0.02), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,extra,taps", [(64, 0, 4), (264, 8, 2), (40, 16, 3), (512, 24, 5), (48, 4, 4), (36, 4, 3), (16, 0, 6)])
def test_convolution_over_long_and_short_steps(hip, dtype, channels, extra, taps):
    """The convolution's kernel of eight channels a thread (rows of whole eights, 2 to 5 taps, steps of 32 tokens and
    more; four tokens a thread from 256 tokens on) and the plain one, through steps whose portions begin in the middle
    of a thread's tokens: a request's first taps come from its slot, never from the neighbouring request's rows."""
    torch.manual_seed(channels + taps)
    lengths = (700, 340)
    rows = [(torch.randn(n, channels + extra) * 2).to(dtype).float() for n in lengths]
    conv = (torch.randn(channels, taps) * 0.5).to(dtype)
    state = torch.zeros(3, 5 + (taps - 1) * channels, dtype=torch.float32, device=DEVICE)
    got = [torch.zeros(n, channels) for n in lengths]
    for befores, counts in (((0, 0), (301, 2)), ((301, 2), (1, 1)), ((302, 3), (3, 326)), ((305, 329), (60, 2)), ((365, 331), (335, 9))):
        ctx = _ctx(befores, counts)
        projected = torch.cat([rows[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        conved = torch.empty(projected.shape[0], channels, dtype=dtype, device=DEVICE)
        hip.conv_silu(projected, channels, conv.to(DEVICE), None, state, 0, ctx, conved, conv_at=5)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = conved[at:at + c].float().cpu()
            at += c
    assert (state[2] == 0.0).all() and (state[:2, :5] == 0.0).all()
    for r, n in enumerate(lengths):
        want = plain.silu(plain.causal_conv(rows[r][:, :channels], conv.float()))
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (2e-6 if dtype == torch.float32 else 0.01), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_wise_kernels(hip, dtype):
    """The normed embedding, the norm that takes a branch and a vector along, the gated activation."""
    torch.manual_seed(5)
    for hidden in (96, 100, 4096):
        table = torch.randn(50, hidden).to(dtype)
        weight = 1 + 0.1 * torch.randn(hidden)
        ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
        out = torch.empty(4, hidden, device=DEVICE)
        hip.embed_normed(ids.to(DEVICE), table.to(DEVICE), weight.to(DEVICE), 1e-6, out)
        torch.testing.assert_close(out.cpu(), plain.unit_rms(table.float()[ids.long()], 1e-6) * weight, rtol=2e-6, atol=2e-6)
        stream = torch.randn(9, hidden, device=DEVICE)
        delta = torch.randn(9, hidden, device=DEVICE).to(dtype)
        vector = torch.randn(hidden, device=DEVICE)
        for with_delta in (True, False):
            mine = stream.clone()
            want_stream = (stream + delta.float() if with_delta else stream) + vector
            normed = torch.empty(9, hidden, dtype=dtype, device=DEVICE)
            hip.norm_add_norm(mine, delta if with_delta else None, None, 0.0, weight.to(DEVICE), 1e-6, normed, offset=vector)
            torch.testing.assert_close(mine, want_stream, rtol=1e-6, atol=1e-6)
            want = plain.unit_rms(want_stream, 1e-6) * weight.to(DEVICE)
            torch.testing.assert_close(normed.float(), want.to(dtype).float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)
            mine = stream.clone()
            hip.norm_add_norm(mine, delta if with_delta else None, None, 0.0, None, 0.0, None, offset=vector)
            torch.testing.assert_close(mine, want_stream, rtol=1e-6, atol=1e-6)
    gate_up = (torch.randn(7, 2 * 88) * 3).to(dtype)
    act = torch.empty(7, 88, dtype=dtype, device=DEVICE)
    hip.gated_activation(gate_up.to(DEVICE), act, "gelu_tanh")
    want = plain.gelu_tanh(gate_up[:, :88].float()) * gate_up[:, 88:].float()
    torch.testing.assert_close(act.float().cpu(), want.to(dtype).float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)
    hip.gated_activation(gate_up.to(DEVICE), act, "silu")
    want = plain.silu(gate_up[:, :88].float()) * gate_up[:, 88:].float()
    torch.testing.assert_close(act.float().cpu(), want.to(dtype).float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)
