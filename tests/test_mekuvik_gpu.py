"""Mekuvik on the GPU: every kernel of its own against the plain implementation's function of the same mechanism, and
the engine with the HIP kernels through the cuttings of `mekuvik_cases` - float32 against tight limits, bfloat16 as
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

import mekuvik_cases as M
import schedules
from conftest import ROOT
from plain import mekuvik_plain as plain
from test_tukevik_gpu import _ctx

pytestmark = pytest.mark.gpu
DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def hip():
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return HipKernels(DEVICE)


@pytest.fixture(scope="module", params=list(M.MEKUVIK))
def case(request, tmp_path_factory):
    return M.make_case(request.param, str(tmp_path_factory.mktemp(f"mekuvik_{request.param}")))


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, case):
    return M.make_engine(case, request.param, DEVICE)


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("cutting", M.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is M.case_greedy_generation and engine.config.dtype != "float32":
        pytest.skip("greedy tokens are compared with the plain float32 implementation's")
    cutting(engine, case)
    assert engine.kernels.parts_library_path.endswith("libakv_parts.so")


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mechanism", M.MECHANISMS)
def test_one_mechanism_alone(mechanism, dtype, tmp_path):
    case = M.make_case(mechanism, str(tmp_path), M.alone(mechanism))
    engine = M.make_engine(case, dtype, DEVICE)
    M.case_whole(engine, case)
    M.case_prefill_then_token_by_token(engine, case)
    M.case_portions_down_to_two_tokens(engine, case)
    M.case_mixed_with_pages_and_slots_used_again(engine, case)


def test_steps_are_recorded_and_replayed(case):
    """Decode steps come again and again: the second is recorded, the later ones are replays; all agree with the plain
    implementation, and with an engine that records nothing to a few units in the last place."""
    ids = case["requests"]["d"]
    want = case["expected"]["d"]
    outs = {}
    for graphs in (True, False):
        engine = M.make_engine(case, "float32", DEVICE, decode_graphs=graphs)
        got, _ = schedules.run(engine, {"d": ids}, schedules.last_one_by_one({"d": ids}, 60))
        M.assert_close(got["d"], want, "float32", f"graphs {graphs}")
        outs[graphs] = got["d"]
        if graphs:
            assert any(g is not None for g in engine._graphs.values()), "nothing was recorded"
    torch.testing.assert_close(outs[True], outs[False], rtol=0, atol=2e-5 * float(want.abs().max()))


def test_trace_replay_of_a_random_model(case, tmp_path):
    """bin/trace_run on a configuration file and a seed: the mixed cutting, every position against the plain model."""
    from ampere_kv_engine_amd.config import MekuvikConfig
    from ampere_kv_engine_amd.weights import write_random_model
    import numpy as np
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), MekuvikConfig.from_dict(case["raw"]), 9)
    requests = {name: case["requests"][name] for name in ("a", "b", "e")}
    schedule = schedules.mixed(requests, M.PROMPTS, 16, 64, seed=3)
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
            want = M.plain_logits(folder, requests[name][:fed[name] + count])[fed[name]:]
            M.assert_close(got[row:row + count], want, "float32", f"step {number} request {name}")
            fed[name] += count
            row += count


def test_the_command_line_generates_with_a_mekuvik_model(case, tmp_path):
    """`python -m ampere_kv_engine_amd.runner` on a configuration file and a seed: one request, and several through the
    scheduler, greedy; the tokens of the plain implementation."""
    import re
    from ampere_kv_engine_amd.config import MekuvikConfig
    from ampere_kv_engine_amd.weights import write_random_model
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), MekuvikConfig.from_dict(case["raw"]), 5)
    prompts = [case["requests"]["a"][:19], case["requests"]["b"][:6], case["requests"]["c"][:31]]
    want = [M.plain_greedy(folder, ids, 6) for ids in prompts]
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
    and rotated dimensions of different widths (some no multiple of 8), windows from one position to longer than a request
    or none, kept first tokens from none to several pages, one to all experts a token, layers without a feed-forward,
    stretched and unstretched frequencies."""
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.choice((2, 3, 4, 5))):
        experts = rng.choice((1, 2, 5, 8, 17))
        mlp = rng.choice((None, M.DENSE(rng.choice((40, 64, 100, 132))),
                          M.MOE(experts, rng.randint(1, min(experts, 4)), rng.choice((8, 20, 33, 64)), rng.choice((None, 8, 48)))))
        kind = rng.choice(("attention", "lightning", "latent_attention"))
        kv, group = rng.choice((1, 2, 3)), rng.choice((1, 2, 4, 5))
        dim = rng.choice((8, 12, 32, 64, 80))
        vdim = rng.choice((4, 8, 24, 64, 72))
        scaling = rng.choice((None, M.YARN(rng.choice((2.0, 4.0, 16.0)), rng.choice((16, 64, 256)), rng.choice((8.0, 32.0)),
                                           rng.choice((0.5, 1.0, 2.0)))))
        base = rng.choice((100.0, 1e4, 1e6))
        if kind == "lightning":
            heads = kv * group
            layers.append(dict(type=kind, mlp=mlp, mixer=M.LIGHT(heads, dim, vdim, [rng.choice((0.5, 0.9, 0.99, 0.999, 1.0)) for _ in range(heads)])))
        elif kind == "attention":
            dims = rng.choice([d for d in (2, 4, 8, 12, 32, 64) if d <= dim])
            window = rng.choice((None, 1, 2, 5, 16, 31, 64, 100, 500))
            keep = rng.choice((None, 0, 1, 4, 7, 16, 40))
            layers.append(dict(type=kind, mlp=mlp, mixer=M.ATTN(kv * group, kv, dim, vdim, rng.uniform(0.1, 0.5), M.ROT(dims, base, scaling), window, keep)))
        else:
            rot_dim = rng.choice((2, 4, 8, 16, 32))
            layers.append(dict(type=kind, mlp=mlp, mixer=M.LATENT(rng.choice((1, 2, 5, 8, 16)), dim, rot_dim, vdim, rng.choice((16, 40, 128)),
                                                                  rng.choice((8, 24, 64)), rng.uniform(0.1, 0.4), base, scaling)))
    raw = dict(architecture="Mekuvik", vocab=rng.choice((97, 260, 1000)), width=rng.choice((40, 72, 96, 120, 192)),
               norm=dict(eps=rng.choice((1e-5, 1e-6))), layers=layers)
    if rng.random() < 0.7:
        raw["logit_scale"] = rng.choice((0.1, 0.25, 3.0))
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        raw["loop"] = dict(start=start, stop=rng.randint(start + 1, len(layers)), times=rng.choice((1, 2, 3)))
    return raw, seed, rng.choice((4, 8, 16, 32))


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("seed", range(700, 710))
def test_a_random_configuration_through_the_cuttings(seed, tmp_path):
    config = random_configuration(seed)
    print(f"seed {seed}: {config[0]}, pages of {config[2]}", flush=True)
    case = M.make_case(f"random {seed}", str(tmp_path), config)
    for dtype in ("float32", "bfloat16"):
        engine = M.make_engine(case, dtype, DEVICE)
        M.case_whole(engine, case)
        M.case_portions_down_to_two_tokens(engine, case)
        M.case_prefill_then_token_by_token(engine, case)
        M.case_mixed_with_pages_and_slots_used_again(engine, case)


LONG = {
    "attention without a window": dict(type="attention", mlp=None, mixer=M.ATTN(4, 2, 32, 16, 0.5, M.ROT(16, 1e4))),
    "attention over a long window": dict(type="attention", mlp=None, mixer=M.ATTN(6, 3, 16, 24, 0.6, M.ROT(16, 1e5, M.YARN(4.0, 128, 16.0, 1.0)), 200, 7)),
    "latent attention": dict(type="latent_attention", mlp=None, mixer=M.LATENT(5, 24, 8, 16, 48, 32, 0.3, 1e4, M.YARN(8.0, 64, 32.0, 1.0))),
    "linear attention": dict(type="lightning", mlp=None, mixer=M.LIGHT(3, 16, 24, (0.97, 0.995, 0.9995))),
}


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mechanism", list(LONG))
def test_long_requests_whose_far_keys_count(mechanism, dtype, tmp_path):
    """One mixer alone, made sharp, over requests of several hundred tokens in pages of 16: a query's few heavy keys lie
    anywhere in its history (a state carries hundreds of tokens), so a page, a tile of keys or a chunk of the recurrence
    that went missing far back moves the logits.  Whole, in portions of 2 to 128 tokens, and with the last 40 tokens one by
    one - where a window of 200 passes over decoded tokens while its seven kept keys stay."""
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine
    from conftest import random_ids
    raw = dict(architecture="Mekuvik", vocab=150, width=64, norm=dict(eps=1e-6), logit_scale=0.3, layers=[LONG[mechanism]])
    folder = M.make_folder(str(tmp_path), raw, 71 + list(LONG).index(mechanism))
    requests = {"a": random_ids(150, 530, seed=1), "b": random_ids(150, 263, seed=2)}
    expected = {name: M.plain_logits(folder, ids) for name, ids in requests.items()}
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=56, max_seqs=4, max_batched_tokens=640,
                                                     max_seq_len=640, device=DEVICE))
    for what, schedule in (("whole", schedules.whole(requests)),
                           ("portions", schedules.portions(requests, sizes=(2, 3, 37, 64, 5, 128, 2, 16, 90, 2))),
                           ("last tokens one by one", schedules.last_one_by_one(requests, 40))):
        got, _ = schedules.run(engine, requests, schedule)
        for name, want in expected.items():
            M.assert_close(got[name], want, dtype, f"{mechanism}, {what}, request {name}")
    assert engine.cache.num_free_pages == [56] * len(engine.cache.groups)


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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,dims,page,window,keep", [
    (4, 2, 16, 24, 12, 4, 11, 2), (3, 1, 40, 8, 40, 16, 64, 0), (8, 2, 64, 64, 32, 16, 72, 5), (2, 1, 128, 256, 64, 16, 200, 17),
    (8, 8, 64, 32, 64, 8, 20, 70), (2, 2, 32, 128, 2, 32, 33, 1), (1, 1, 256, 32, 128, 16, None, 0), (6, 3, 64, 64, 16, 16, 1, 3)])
def test_windowed_attention_with_kept_first_tokens_alone(hip, dtype, heads, kv_heads, dim, vdim, dims, page, window, keep):
    """Two requests in two portions each and a last token alone, through the norm over the whole projection with its
    weights, the interleaved rotation, the cache write and the attention, against the plain attention of the whole
    sequences.  Scores are sharp; keys are made to stand out at position 0 (kept, or not), at the last kept position and
    the first that is not, and in the middle of the long request: each must count exactly for the queries that see it -
    just inside and just outside the window, in prompts and for the token that comes alone."""
    torch.manual_seed(heads * 100 + dim)
    lengths, eps = (75, 700 if dim <= 64 else 330), 1e-5
    scale = 4.0 / math.sqrt(dim)
    rot = dict(dims=dims, base=1000.0, scaling=M.YARN(4.0, 64, 16.0, 1.0))
    q_size, k_size = heads * dim, kv_heads * dim
    width = q_size + k_size + kv_heads * vdim
    rows = [torch.randn(n, width) for n in lengths]
    # every query leans along one direction (beyond the rotated dimensions, where there are any); the marked keys lie along it
    lo = dims if dims < dim else 0
    along = torch.zeros(dim)
    along[lo:] = torch.randint(0, 2, (dim - lo,)).float() * 2 - 1
    for projected, n in zip(rows, lengths):
        projected[:, :q_size].view(n, heads, dim).add_(0.7 * along)
        for needle in {0, max(keep - 1, 0), keep, n // 2}:
            projected[needle, q_size:q_size + k_size].view(kv_heads, dim)[:, lo:] = along[lo:] * 40
    rows = [r.to(dtype).float() for r in rows]
    q_weight, k_weight = (1 + 0.3 * torch.randn(q_size)).to(DEVICE), (1 + 0.3 * torch.randn(k_size)).to(DEVICE)
    freqs, magnitude = plain.rotary_frequencies(dims, rot["base"], rot["scaling"])
    table = torch.empty(max(lengths) + page, dims // 2, 2, dtype=torch.float32, device=DEVICE)
    hip.rope_table(freqs.float().to(DEVICE), table)
    table.mul_(magnitude)
    k_pages, v_pages, block_table = _pages_for(lengths, page, kv_heads, dim, vdim, dtype)
    got = [torch.zeros(n, heads * vdim) for n in lengths]
    steps = [((0, 0), (41, 5)), ((41, 5), (lengths[0] - 42, lengths[1] - 6)), ((lengths[0] - 1, lengths[1] - 1), (1, 1))]
    for befores, counts in steps:
        ctx = _ctx(befores, counts)
        projected = torch.cat([rows[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        slot_map = torch.tensor([int(block_table[r, p // page]) * page + p % page for r, (b, c) in enumerate(zip(befores, counts))
                                 for p in range(b, b + c)], dtype=torch.int32, device=DEVICE)
        meta = SimpleNamespace(block_table=block_table.to(DEVICE), rows=None, width=block_table.shape[1], slot_map=slot_map)
        q = torch.empty(ctx.num_tokens, q_size, dtype=dtype, device=DEVICE)
        out = torch.empty(ctx.num_tokens, heads * vdim, dtype=dtype, device=DEVICE)
        hip.unit_norm_write(projected, heads, kv_heads, dim, vdim, eps, slot_map, k_pages, v_pages, q, table=table, rot_dims=dims,
                            positions=ctx.positions, q_weight=q_weight, k_weight=k_weight, whole=True, interleaved=True)
        hip.gated_attention(q, k_pages, v_pages, None, 0, ctx, meta, heads, kv_heads, dim, vdim, scale, None, None, window, False,
                            out, keep_first=keep)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot,
             **({"mask": dict(size=window, keep_first=keep)} if window else {}))
    pick = lambda lo, hi: torch.eye(width)[lo:hi]
    w = {"q": pick(0, q_size), "k": pick(q_size, q_size + k_size), "v": pick(q_size + k_size, width), "o": torch.eye(heads * vdim),
         "q.norm": q_weight.cpu(), "k.norm": k_weight.cpu()}
    for r, n in enumerate(lengths):
        want = plain.attention(rows[r], w, m, eps)
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (3e-5 if dtype == torch.float32 else 0.05), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim", [(2, 16, 12), (1, 64, 32), (3, 24, 40), (2, 128, 128), (4, 64, 64), (1, 256, 256)])
def test_linear_attention_kernels_alone(hip, dtype, heads, dim, vdim):
    """Two requests through three steps (a portion that is walked over chunks, single tokens, a portion again) in slots
    that are not their rows: the recurrence with silu on its inputs and raw outputs, then the norm over all heads with
    its weight and the sigmoid gate, against the plain mixer."""
    torch.manual_seed(dim + vdim)
    lengths, eps = (70, 9), 1e-6
    m = dict(heads=heads, dim=dim, vdim=vdim, decay=[0.9, 0.999, 1.0, 0.6][:heads])
    qk, vs = heads * dim, heads * vdim
    width = 2 * qk + 2 * vs
    rows = [(torch.randn(n, width) * 1.5).to(dtype).float() for n in lengths]
    state = torch.zeros(4, heads * dim * vdim, dtype=torch.float32, device=DEVICE)
    decay = torch.tensor(m["decay"], dtype=torch.float32, device=DEVICE)
    weight = (1 + 0.3 * torch.randn(vs)).to(DEVICE)
    got = [torch.zeros(n, vs) for n in lengths]
    for befores, counts in (((0, 0), (33, 2)), ((33, 2), (1, 1)), ((34, 3), (36, 6))):
        ctx = _ctx(befores, counts)
        ctx.seq_slots = torch.tensor([3, 1], dtype=torch.int32, device=DEVICE)
        ctx.host_seq_slots = [3, 1]
        projected = torch.cat([rows[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        raw = torch.empty(ctx.num_tokens, vs, dtype=torch.float32, device=DEVICE)
        out = torch.empty(ctx.num_tokens, vs, dtype=dtype, device=DEVICE)
        hip.retention(projected, heads, dim, vdim, 0, None, 1.0, decay, eps, state, ctx, None, input_activation="silu", raw=raw)
        hip.norm_gate_rows(raw, weight, eps, projected, 2 * qk + vs, "sigmoid", out)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    assert not state[0].any() and not state[2].any() and state[3].any() and state[1].any()
    pick = lambda lo, hi: torch.eye(width)[lo:hi]
    w = {"q": pick(0, qk), "k": pick(qk, 2 * qk), "v": pick(2 * qk, 2 * qk + vs), "g": pick(2 * qk + vs, width), "o": torch.eye(vs),
         "norm": weight.cpu()}
    for r, n in enumerate(lengths):
        want = plain.lightning(rows[r], w, m, eps)
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (3e-5 if dtype == torch.float32 else 0.03), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens,experts,top,ff,shared", [(5, 7, 3, 12, 20), (40, 16, 1, 64, 128), (3, 2, 2, 33, 0), (130, 8, 8, 8, 8), (1, 5, 2, 7, 3)])
def test_routing_by_sigmoid_scores_and_the_weight_inside_the_activation(hip, dtype, tokens, experts, top, ff, shared):
    torch.manual_seed(tokens + experts)
    logits = (torch.randn(tokens, experts) * 3).to(DEVICE)
    logits[0, :] = 0.5                                   # equal logits: the lower indices are chosen
    if tokens > 2:
        logits[2, -1] = -120.0                           # a score of exactly zero
    columns = experts * ff + shared
    gates = torch.full((tokens, experts + (1 if shared else 0)), 7.0, device=DEVICE)
    hip.route_chosen(logits, gates, experts, top, law="sigmoid")
    chosen = torch.sort(logits.cpu(), dim=-1, descending=True, stable=True).indices[:, :top]      # (equal logits: the lower index)
    want = torch.zeros(tokens, experts).scatter_(1, chosen, torch.sigmoid(torch.gather(logits.cpu(), 1, chosen)))
    torch.testing.assert_close(gates[:, :experts].cpu(), want, rtol=1e-6, atol=1e-7)
    assert gates[0, :top].ne(0).all() and gates[0, top:experts].eq(0).all()
    if shared:
        assert gates[:, experts].eq(1).all()
    up = (torch.randn(tokens, columns) * 2).to(dtype).to(DEVICE)
    for inside in (True, False):
        act = torch.empty(tokens, columns, dtype=dtype, device=DEVICE)
        hip.gate_activation(up, gates, act, experts, ff, "gelu", inside)
        per_column = torch.cat((gates[:, :experts].repeat_interleave(ff, dim=1), gates[:, experts:].expand(-1, shared)), dim=1).cpu()
        z = up.float().cpu()
        expected = plain.gelu_erf(per_column * z) if inside else per_column * plain.gelu_erf(z)
        torch.testing.assert_close(act.float().cpu(), expected.to(dtype).float(), rtol=1e-5 if dtype == torch.float32 else 8e-3, atol=1e-6)
        assert act[:, :experts * ff][per_column[:, :experts * ff].to(DEVICE) == 0].eq(0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_wise_kernels(hip, dtype):
    """Two branches into the residual sum in one kernel; the embedding added a second time (also for a token that the
    sampler left in the request's slot); rows normed, weighted and gated; the interleaved rotation of a latent
    attention's key part and queries."""
    torch.manual_seed(3)
    for tokens, hidden in ((5, 96), (3, 40), (2, 4100), (1, 10)):
        stream = torch.randn(tokens, hidden, device=DEVICE)
        a, b = (torch.randn(tokens, hidden, device=DEVICE).to(dtype) for _ in range(2))
        weight = 1 + 0.2 * torch.randn(hidden, device=DEVICE)
        out = torch.empty(tokens, hidden, dtype=dtype, device=DEVICE)
        want_stream = stream + 0.5 * (a.float() + b.float())
        hip.norm_add_norm(stream, a, None, 0.0, weight, 1e-5, out, delta_scale=0.5, delta2=b)
        torch.testing.assert_close(stream, want_stream, rtol=1e-6, atol=1e-6)
        want = plain.rms_norm(want_stream, weight, 1e-5)
        torch.testing.assert_close(out.float(), want.to(dtype).float(), rtol=1e-5 if dtype == torch.float32 else 8e-3, atol=1e-6)
    table = torch.randn(50, 72, device=DEVICE).to(dtype)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEVICE)
    stream = torch.randn(4, 72, device=DEVICE)
    want = stream + table[ids.long()].float()
    hip.embed_add(ids, table, stream)
    torch.testing.assert_close(stream, want, rtol=0, atol=0)
    ctx = _ctx((4, 9), (1, 1))
    ctx.slot_words = torch.zeros(2, 8, dtype=torch.int32, device=DEVICE)
    ctx.slot_words[0, 1], ctx.slot_words[1, 1] = 17, 5
    stream = torch.zeros(2, 72, device=DEVICE)
    hip.embed_add(torch.tensor([-1, 6], dtype=torch.int32, device=DEVICE), table, stream, ctx)
    torch.testing.assert_close(stream, table[[17, 6]].float(), rtol=0, atol=0)
    for width, gate, eps, has_weight in ((60, "sigmoid", 1e-6, True), (33, "silu", 1e-5, False), (256, None, 1e-6, True), (7, "sigmoid", None, False)):
        x = torch.randn(6, width + 5, device=DEVICE)
        gates = torch.randn(6, width + 9, device=DEVICE).to(dtype)
        weight = (1 + 0.2 * torch.randn(width, device=DEVICE)) if has_weight else None
        out = torch.zeros(6, width + 3, dtype=dtype, device=DEVICE)
        hip.norm_gate_rows(x, weight, eps, gates, 9, gate, out, out_at=3, out_scale=0.5, x_at=5, width=width)
        v = x[:, 5:]
        if eps is not None:
            v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)
        if weight is not None:
            v = v * weight
        g = gates[:, 9:].float()
        v = v * (torch.sigmoid(g) if gate == "sigmoid" else plain.silu(g) if gate == "silu" else 1.0) * 0.5
        torch.testing.assert_close(out[:, 3:].float(), v.to(dtype).float(), rtol=1e-5 if dtype == torch.float32 else 8e-3, atol=1e-6)
        assert out[:, :3].eq(0).all()
    # the latent attention's rotations, pairs (2 i, 2 i + 1), stretched frequencies
    tokens, heads, dim, rot, q_rank, kv_rank, page = 7, 3, 12, 8, 16, 24, 4
    freqs, magnitude = plain.rotary_frequencies(rot, 200.0, M.YARN(3.0, 24, 6.0, 1.5))
    angles = torch.empty(64, rot // 2, 2, dtype=torch.float32, device=DEVICE)
    hip.rope_table(freqs.float().to(DEVICE), angles)
    angles.mul_(magnitude)
    positions = torch.tensor([0, 1, 5, 30, 31, 2, 63], dtype=torch.int32, device=DEVICE)
    down = torch.randn(tokens, q_rank + kv_rank + rot + 10, device=DEVICE).to(dtype)
    records = torch.zeros(4, 1, page, kv_rank + rot, dtype=dtype, device=DEVICE)
    slot_map = torch.tensor([9, 2, 0, 15, 7, 4, 11], dtype=torch.int32, device=DEVICE)
    cq = torch.empty(tokens, q_rank, dtype=dtype, device=DEVICE)
    ones = torch.ones(max(q_rank, kv_rank), device=DEVICE)
    hip.latent_encode(down, q_rank, kv_rank, rot, rot, ones[:q_rank], ones[:kv_rank], 1e-6, angles, positions, slot_map, cq, records,
                      interleaved=True)
    key = down[:, q_rank + kv_rank:q_rank + kv_rank + rot].float().cpu().view(tokens, 1, rot)
    want = plain.rotate_interleaved(key, positions.cpu(), rot, freqs, magnitude)[:, 0]
    got = records.view(-1, kv_rank + rot)[slot_map.long()][:, kv_rank:].float().cpu()
    torch.testing.assert_close(got, want.to(dtype).float(), rtol=1e-5 if dtype == torch.float32 else 8e-3, atol=1e-5)
    q = torch.randn(tokens, heads * (dim + rot), device=DEVICE).to(dtype)
    q_abs = torch.zeros(tokens, heads, kv_rank + rot, dtype=torch.float32, device=DEVICE)
    hip.rotate_queries(q, heads, dim, rot, rot, angles, positions, q_abs, kv_rank, interleaved=True)
    want = plain.rotate_interleaved(q.float().cpu().view(tokens, heads, dim + rot)[..., dim:], positions.cpu(), rot, freqs, magnitude)
    torch.testing.assert_close(q_abs[..., kv_rank:].cpu(), want, rtol=1e-5, atol=1e-5)
