"""Lirulix on the host: its configuration, and the engine's side of it - registry, loading, caches and states of layers
that run several times, windows whose pages are given back, batching, the scheduler - with the torch double standing in
for the HIP kernels, against the plain implementation.  The HIP kernels meet the same cases in `test_lirulix_gpu.py`."""

import copy
import json
import math
import os

import pytest
import torch

import lirulix_cases as L
from ampere_kv_engine_amd.config import ConfigError, LirulixConfig, RunEntry, load_config
from ampere_kv_engine_amd.engine.model import expected_tensors
from ampere_kv_engine_amd.parts.position import stretched_frequencies
from plain import lirulix_plain as plain
from torch_kernels import TorchKernels


@pytest.fixture(scope="module", params=["A", "B"])       # (the third configuration, of served sizes, meets the GPU alone)
def case(request, tmp_path_factory):
    return L.make_case(request.param, str(tmp_path_factory.mktemp(f"lirulix_{request.param}")))


@pytest.fixture(scope="module")
def engine(case):
    return L.make_engine(case, "float32", "cpu", kernels=TorchKernels())


@pytest.mark.parametrize("cutting", L.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is L.case_long_decoding:
        cutting(engine, case, tokens=90)         # (the double steps through recurrences token by token on the host)
    else:
        cutting(engine, case)


@pytest.mark.parametrize("mechanism", L.MECHANISMS)
def test_one_mechanism_alone(mechanism, tmp_path):
    case = L.make_case(mechanism, str(tmp_path), L.alone(mechanism))
    engine = L.make_engine(case, "float32", "cpu", kernels=TorchKernels())
    L.case_whole(engine, case)
    L.case_portions_down_to_two_tokens(engine, case)
    L.case_mixed_with_pages_and_slots_used_again(engine, case)


def test_the_configuration_names_every_part_and_tensor(tmp_path):
    raw = copy.deepcopy(L.LIRULIX_A)
    folder = str(tmp_path)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    config = load_config(folder)                     # found through the key "architecture"
    assert isinstance(config, LirulixConfig) and config.to_dict() == raw
    spec = config.to_model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["gated_delta_rule", "gated_attention", "differential_attention"]
    assert [layer.feed_forward.kind for layer in spec.layers] == ["none", "swiglu", "swiglu"]
    assert all(layer.block.kind == "scaled_prenorm" and layer.block["norm"]["unit_offset"] for layer in spec.layers)
    assert spec.layers[1].feed_forward["activation"] == "gelu_tanh" and spec.layers[1].mixer["sink"] == "learned"
    assert spec.layers[1].mixer["position"]["scaling"]["kind"] == "yarn" and spec.layers[2].mixer["position"]["scaling"]["kind"] == "llama3"
    # three passes over layers 0 and 1, each with caches of its own and a vector before its first layer; then layer 2
    assert spec.run_order == tuple([RunEntry(0, 0, True, t, t) if i == 0 else RunEntry(1, 1, True, t, None)
                                    for t in range(3) for i in range(2)] + [RunEntry(2, 2)])
    assert len({spec.cache_key(entry) for entry in spec.run_order}) == 7
    names = {t.name: tuple(t.shape) for t in expected_tensors(spec) if not t.optional}
    assert names["embed"] == (211, 96) and names["embed.norm"] == (96,) and names["head"] == (211, 96)
    assert names["loop.step"] == (3, 96) and names["final.norm"] == (96,) and "l0.norm2" not in names
    assert names["l0.mix.q"] == (48, 96) and names["l0.mix.v"] == (80, 96) and names["l0.mix.q.conv"] == (48, 4)
    assert names["l0.mix.v.conv"] == (80, 4) and names["l0.mix.b"] == (4, 96) and names["l0.mix.A_log"] == (4,)
    assert names["l0.mix.a1"] == (8, 96) and names["l0.mix.a2"] == (96, 8) and names["l0.mix.dt_bias"] == (96,)
    assert names["l0.mix.g1"] == (12, 96) and names["l0.mix.g2"] == (80, 12) and names["l0.mix.norm"] == (20,)
    assert names["l0.mix.o"] == (96, 80) and names["l1.mix.q"] == (144, 96) and names["l1.mix.k"] == (48, 96)
    assert names["l1.mix.v"] == (32, 96) and names["l1.mix.sink"] == (6,) and names["l1.mix.o"] == (96, 96)
    assert names["l2.mix.q"] == (96, 96) and names["l2.mix.k"] == (96, 96) and names["l2.mix.v"] == (120, 96)
    assert names["l2.mix.g"] == (120, 96) and names["l2.mix.lq2"] == (16,) and names["l2.mlp.down"] == (96, 40)


def test_low_ranks_come_from_the_checkpoint_where_the_configuration_does_not_name_them(tmp_path):
    folder = L.make_folder(str(tmp_path), L.LIRULIX_A, 3)
    with open(os.path.join(folder, "config.json")) as handle:
        raw = json.load(handle)
    del raw["layers"][0]["mixer"]["ranks"]
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    config = load_config(folder)
    assert config.layers[0]["mixer"]["ranks"] == dict(decay=8, gate=12)
    with pytest.raises(ConfigError, match="ranks"):
        LirulixConfig.from_dict(raw)                 # neither named nor to be found
    raw["layers"][0]["mixer"]["ranks"] = dict(decay=9, gate=12)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    with pytest.raises(ConfigError, match="a1"):
        load_config(folder)


@pytest.mark.parametrize("change,message", [
    (lambda raw: raw["layers"][1].update(type="rglru"), "type"),
    (lambda raw: raw["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda raw: raw["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda raw: raw["layers"][1]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
    (lambda raw: raw["layers"][2]["mixer"]["rot"]["scaling"].pop("high"), "high"),
    (lambda raw: raw["layers"][2]["mixer"].pop("diff"), "diff"),
    (lambda raw: raw["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda raw: raw["layers"][2]["mlp"].update(kind="moe"), "kind"),
    (lambda raw: raw["loop"].update(stop=4), "loop"),
    (lambda raw: raw["loop"].update(times=0), "times"),
    (lambda raw: raw.pop("width"), "width"),
])
def test_configurations_the_design_does_not_allow_are_refused(change, message):
    raw = copy.deepcopy(L.LIRULIX_A)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        LirulixConfig.from_dict(raw)


def test_every_pass_has_caches_and_states_of_its_own_and_slots_start_fresh(case, engine):
    from ampere_kv_engine_amd.engine import StepEntry
    spec, layers, page = engine.spec, case["raw"]["layers"], case["page_size"]
    keys = [spec.cache_key(entry) for entry in spec.run_order]
    assert len(set(keys)) == len(keys) == len(engine.cache.layer_cache)
    for entry in spec.run_order:
        view, m = engine.cache.layer_cache[spec.cache_key(entry)], layers[entry.layer]["mixer"]
        if layers[entry.layer]["type"] == "channel_delta":
            channels = 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"]
            assert view.k is None and view.state.shape == (4, m["heads"] * m["dim"] * m["vdim"] + (m["conv"] - 1) * channels)
        else:
            maps = 2 if layers[entry.layer]["type"] == "attention_2" else 1
            assert view.k.shape[1:] == (m["kv_heads"], page, maps * m["dim"]) and view.v.shape[1:] == (m["kv_heads"], m["vdim"], page)
            assert view.state is None
    tensors = [view.k if view.k is not None else view.state for view in engine.cache.layer_cache.values()]
    assert len({t.data_ptr() for t in tensors}) == len(tensors)
    seq = engine.open("w")
    engine.step([StepEntry(seq, case["requests"]["d"], [])])
    engine.step([StepEntry(seq, case["requests"]["a"][:1], [])])    # (what a window has passed is given back when tokens register)
    for table, group in zip(seq.tables, engine.cache.groups):
        if group.need.window is not None:
            assert table.num_held <= (group.need.window + page - 1) // page + 1
    states = [view.state for view in engine.cache.layer_cache.values() if view.state is not None]
    assert all(state[seq.slot].any() for state in states)
    slot = seq.slot
    engine.close(seq)
    seq = engine.open("again")           # the slot comes round again: nothing of its predecessor is left
    assert seq.slot == slot and not any(state[slot].any() for state in states)
    engine.close(seq)


# ---- the plain implementation's own mechanisms, where a sentence of the design can be checked by hand -----------------

def test_plain_mechanisms_by_hand():
    assert plain.seen(4, 2).int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 0, 1, 1]]
    assert plain.seen(3, None).int().tolist() == [[1, 0, 0], [1, 1, 0], [1, 1, 1]]
    p = plain.softmax_with_sink(torch.tensor([[0.0, math.log(2.0), 5.0]]), torch.tensor([[True, True, False]]), torch.tensor(math.log(5.0)))
    torch.testing.assert_close(p, torch.tensor([[0.125, 0.25, 0.0]]))           # 1 / (1 + 2 + 5), 2 / 8: the sink counts once
    p = plain.softmax_with_sink(torch.tensor([[0.0, math.log(3.0)]]), torch.tensor([[True, True]]), None)
    torch.testing.assert_close(p, torch.tensor([[0.25, 0.75]]))
    out = plain.causal_conv(torch.tensor([[1.0], [2.0], [4.0]]), torch.tensor([[100.0, 10.0, 1.0]]))
    assert out[:, 0].tolist() == [1.0, 12.0, 124.0]
    torch.testing.assert_close(plain.unit_length(torch.tensor([3.0, 4.0]), 0.0), torch.tensor([0.6, 0.8]))
    torch.testing.assert_close(plain.offset_norm(torch.tensor([[3.0, -3.0]]), torch.tensor([0.5, -0.5]), 0.0), torch.tensor([[1.5, -0.5]]))
    w = {"lq1": torch.tensor([1.0, 0.0]), "lk1": torch.tensor([math.log(3.0), 9.0]), "lq2": torch.tensor([0.0, 0.0]), "lk2": torch.ones(2)}
    torch.testing.assert_close(plain.difference_weight(w, 0.25), torch.tensor(3.0 - 1.0 + 0.25))
    assert plain.layer_runs(dict(layers=[0] * 4, loop=dict(start=1, stop=3, times=2))) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert plain.layer_runs(dict(layers=[0] * 2)) == [(0, None), (1, None)]
    turned = plain.rotate(torch.arange(6.0).view(1, 1, 6), torch.tensor([2]), dict(dims=4, base=100.0), "yarn")
    assert torch.equal(turned[..., 4:], torch.tensor([[[4.0, 5.0]]]))
    torch.testing.assert_close(turned[0, 0, 0], torch.tensor(0 * math.cos(2.0) - 2 * math.sin(2.0)))
    torch.testing.assert_close(turned[0, 0, 3], torch.tensor(3 * math.cos(0.2) + 1 * math.sin(0.2)))


def test_the_delta_rule_by_hand():
    """One head, two key channels, one value: the first token writes beta v k^T; the second reads it through its own k
    after the decay, corrects it, and the read-out sees the correction."""
    q = torch.tensor([[[1.0, 0.0]], [[1.0, 1.0]]])
    k = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]]])
    v = torch.tensor([[[2.0]], [[5.0]]])
    beta = torch.tensor([[0.5], [1.0]])
    decay = torch.tensor([[[1.0, 1.0]], [[0.5, 0.25]]])
    out = plain.delta_rule(q, k, v, beta, decay)
    # t = 0: S = [[1], [0]] (0.5 * 2 on the first key channel); o = 1.  t = 1: S <- [[0.5], [0]]; u = 5 - 0.5 = 4.5;
    # S = [[5], [0]]; o = q . S = 5.
    assert out[:, 0, 0].tolist() == [1.0, 5.0]


def test_stretched_frequencies_by_hand():
    base = [100.0 ** (-2.0 * i / 8) for i in range(4)]
    got, magnitude = stretched_frequencies(8, 100.0, None)
    assert got == base and magnitude == 1.0
    # llama3: wavelengths 6.3, 19.9, 62.8, 198.7 against original / high = 16 and original / low = 64
    got, magnitude = stretched_frequencies(8, 100.0, dict(kind="llama3", factor=4.0, original=64.0, low=1.0, high=4.0))
    share = lambda f: (64.0 / (2 * math.pi / f) - 1.0) / 3.0
    want = [base[0], (1 - share(base[1])) * base[1] / 4 + share(base[1]) * base[1],
            (1 - share(base[2])) * base[2] / 4 + share(base[2]) * base[2], base[3] / 4]
    assert magnitude == 1.0 and got == pytest.approx(want, rel=1e-12)
    # yarn: the ramp runs from dimension lo = 0 to hi = 2 here, and cos and sin grow by 0.1 ln(factor) + 1
    got, magnitude = stretched_frequencies(8, 100.0, dict(kind="yarn", factor=2.0, original=40.0, fast=4.0, slow=0.5))
    turned = lambda turns: 8 * math.log(40.0 / (2 * math.pi * turns)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(turned(4.0)), 0), min(math.ceil(turned(0.5)), 7)
    assert (lo, hi) == (0, 3)
    want = [f / 2 * r + f * (1 - r) for f, r in zip(base, (0.0, 1 / 3, 2 / 3, 1.0))]
    assert got == pytest.approx(want, rel=1e-12) and magnitude == pytest.approx(0.1 * math.log(2.0) + 1.0)
    for kind, scaling in (("yarn", L.YARN(4.0, 32, 8.0, 2.0)), ("llama3", L.LLAMA3(4.0, 16, 1.0, 4.0))):
        mine, factor = stretched_frequencies(16, 100.0, dict(kind=kind, **scaling))
        theirs, other = plain.frequencies(dict(dims=16, base=100.0, scaling=scaling), kind)
        assert mine == pytest.approx(theirs.tolist(), rel=1e-12) and factor == pytest.approx(other)


def test_a_key_at_the_windows_edge_and_a_far_key_decide_the_output():
    """The plain attentions with inputs made so that one key stands out: under a window it is seen from exactly `size`
    positions; without one, from every later position however far, unless the sink outweighs it."""
    n, size = 30, 7
    h = torch.zeros(n, 3)
    h[:, 0] = 1.0                      # every token: the same query direction
    h[5, 1] = 1.0                      # position 5: a key along the queries, a value of its own
    rot = dict(dims=2, base=10000.0)
    wide = lambda rows, cols, entries: torch.tensor([[entries.get((r, c), 0.0) for c in range(cols)] for r in range(rows)])
    # differential attention of one head: map 1 looks for the key, map 2 sees nothing special; dims beyond the rotated pair
    m = dict(heads=1, kv_heads=1, dim=4, vdim=2, mask=dict(size=size), scale=8.0, diff=0.0, rot=rot)
    w = {"q": wide(8, 3, {(2, 0): 1.0}), "k": wide(8, 3, {(2, 1): 1.0}), "v": wide(2, 3, {(0, 1): 1.0, (1, 0): 0.01}),
         "g": torch.zeros(2, 3), "o": torch.eye(2), "lq1": torch.zeros(4), "lk1": torch.zeros(4), "lq2": torch.zeros(4), "lk2": torch.zeros(4)}
    # lambda = 1 - 1 + 0 = 0: the output is map 1, normed: its first value dominates exactly while position 5 is seen
    out = plain.differential_attention(h, w, m, 1e-6)
    strong = (out[:, 0] > 0.5).nonzero().flatten().tolist()
    assert strong == list(range(5, 5 + size))
    # attention with a sink, no window: seen from everywhere behind; a huge sink takes the weight away
    m = dict(heads=1, kv_heads=1, dim=4, vdim=2, scale=8.0, rot=rot)
    w = {"q": wide(4, 3, {(2, 0): 1.0}), "k": wide(4, 3, {(2, 1): 1.0}), "v": wide(2, 3, {(0, 1): 1.0}), "o": torch.eye(2),
         "sink": torch.tensor([-20.0])}
    out = plain.sink_attention(h, w, m)
    assert (out[5:, 0] > 0.98).all() and (out[:5, 0].abs() < 1e-6).all()
    w["sink"] = torch.tensor([20.0])
    assert (plain.sink_attention(h, w, m)[:, 0] < 1e-4).all()
