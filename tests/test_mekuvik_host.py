"""Mekuvik on the host: its configuration, and the engine's side of it - registry, loading, caches and states of layers
that run several times, a window whose first pages are kept while those behind it are given back, batching, the
scheduler - with the torch double standing in for the HIP kernels, against the plain implementation.  The HIP kernels
meet the same cases in `test_mekuvik_gpu.py`."""

import copy
import json
import math
import os

import pytest
import torch

import mekuvik_cases as M
from ampere_kv_engine_amd.cache.pages import RELEASED, BlockTable, PageAllocator
from ampere_kv_engine_amd.config import ConfigError, MekuvikConfig, RunEntry, load_config
from ampere_kv_engine_amd.engine.model import expected_tensors
from plain import mekuvik_plain as plain
from torch_kernels import TorchKernels


@pytest.fixture(scope="module", params=["A", "B"])       # (the third configuration, of served sizes, meets the GPU alone)
def case(request, tmp_path_factory):
    return M.make_case(request.param, str(tmp_path_factory.mktemp(f"mekuvik_{request.param}")))


@pytest.fixture(scope="module")
def engine(case):
    return M.make_engine(case, "float32", "cpu", kernels=TorchKernels())


@pytest.mark.parametrize("cutting", M.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is M.case_long_decoding:
        cutting(engine, case, tokens=90)         # (the double steps through recurrences token by token on the host)
    else:
        cutting(engine, case)


@pytest.mark.parametrize("mechanism", M.MECHANISMS)
def test_one_mechanism_alone(mechanism, tmp_path):
    case = M.make_case(mechanism, str(tmp_path), M.alone(mechanism))
    engine = M.make_engine(case, "float32", "cpu", kernels=TorchKernels())
    M.case_whole(engine, case)
    M.case_portions_down_to_two_tokens(engine, case)
    M.case_mixed_with_pages_and_slots_used_again(engine, case)


def test_the_configuration_names_every_part_and_tensor(tmp_path):
    raw = copy.deepcopy(M.MEKUVIK_A)
    folder = str(tmp_path)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    config = load_config(folder)                     # found through the key "architecture"
    assert isinstance(config, MekuvikConfig) and config.to_dict() == raw
    spec = config.to_model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["retention", "gated_attention", "latent_attention"]
    assert [layer.feed_forward.kind for layer in spec.layers] == ["none", "routed_experts", "swiglu"]
    assert all(layer.block.kind == "shared_norm" and layer.block["norm"]["single_rounding"] for layer in spec.layers)
    light, attention, latent = (layer.mixer for layer in spec.layers)
    assert light["input_activation"] == "silu" and light["norm"] == "all_heads" and light["gate"] == "sigmoid"
    assert light["key_scale"] == 1.0 and light["rotary_dims"] == 0 and light["decay"] == (0.7, 0.95, 0.999)
    assert attention["window"] == 13 and attention["keep_first"] == 3 and attention["projection_norm_eps"] == 1e-6
    assert attention["position"]["layout"] == "interleaved" and attention["position"]["scaling"] is None and not attention["sink"]
    assert latent["position"]["scaling"]["kind"] == "yarn" and latent["gate"] and latent["window"] is None
    routed = spec.layers[1].feed_forward
    assert routed["weights"] == "sigmoid_chosen" and routed["activation"] == "gelu" and routed["weight_on_input"]
    assert routed["shared_size"] == 24 and not routed["shared_gate"] and routed["top"] == 2
    assert spec.final_norm["output_scale"] == 0.5 and spec.head["tied_to"] == "embed"
    # three passes over layers 0 and 1, each with caches of its own; the second and third begin with the embedding; then layer 2
    assert spec.run_order == tuple([RunEntry(i, i, True, t, None, t > 0 and i == 0) for t in range(3) for i in range(2)]
                                   + [RunEntry(2, 2)])
    assert len({spec.cache_key(entry) for entry in spec.run_order}) == 7
    names = {t.name: tuple(t.shape) for t in expected_tensors(spec) if not t.optional}
    assert names["embed"] == (211, 96) and names["final.norm"] == (96,) and "head" not in names and "l0.norm2" not in names
    assert names["l0.norm1"] == (96,) and names["l0.mix.q"] == (72, 96) and names["l0.mix.v"] == (60, 96)
    assert names["l0.mix.g"] == (60, 96) and names["l0.mix.norm"] == (60,) and names["l0.mix.o"] == (96, 60)
    assert names["l1.mix.q"] == (144, 96) and names["l1.mix.k"] == (48, 96) and names["l1.mix.v"] == (32, 96)
    assert names["l1.mix.q.norm"] == (144,) and names["l1.mix.k.norm"] == (48,) and names["l1.mix.o"] == (96, 96)
    assert names["l1.mlp.router"] == (6, 96) and names["l1.mlp.e5.up"] == (20, 96) and names["l1.mlp.e0.down"] == (96, 20)
    assert names["l1.mlp.shared.up"] == (24, 96) and names["l1.mlp.shared.down"] == (96, 24) and "l1.mlp.shared.sg" not in names
    assert names["l2.mix.dq"] == (24, 96) and names["l2.mix.dq.norm"] == (24,) and names["l2.mix.uq"] == (72, 24)
    assert names["l2.mix.dkv"] == (48, 96) and names["l2.mix.dkv.norm"] == (40,) and names["l2.mix.uk"] == (48, 40)
    assert names["l2.mix.uv"] == (72, 40) and names["l2.mix.g"] == (72, 96) and names["l2.mix.o"] == (96, 72)
    assert names["l2.mlp.gate"] == (72, 96) and names["l2.mlp.down"] == (96, 72)


def test_a_latent_querys_rank_comes_from_the_checkpoint_where_the_configuration_does_not_name_it(tmp_path):
    folder = M.make_folder(str(tmp_path), M.MEKUVIK_A, 3)
    with open(os.path.join(folder, "config.json")) as handle:
        raw = json.load(handle)
    del raw["layers"][2]["mixer"]["q_rank"]
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    assert load_config(folder).layers[2]["mixer"]["q_rank"] == 24
    with pytest.raises(ConfigError, match="q_rank"):
        MekuvikConfig.from_dict(raw)                 # neither named nor to be found


@pytest.mark.parametrize("change,message", [
    (lambda raw: raw["layers"][1].update(type="rglru"), "type"),
    (lambda raw: raw["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda raw: raw["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda raw: raw["layers"][2]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
    (lambda raw: raw["layers"][0]["mixer"].update(decay=[0.5, 0.5]), "decay"),
    (lambda raw: raw["layers"][1]["mixer"]["mask"].update(keep_first=-1), "keep_first"),
    (lambda raw: raw["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda raw: raw["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda raw: raw["layers"][1]["mlp"]["router"].update(top=7), "router"),
    (lambda raw: raw["layers"][2]["mlp"].update(kind="glu"), "kind"),
    (lambda raw: raw["loop"].update(stop=4), "loop"),
    (lambda raw: raw["loop"].update(times=0), "times"),
    (lambda raw: raw.pop("width"), "width"),
])
def test_configurations_the_design_does_not_allow_are_refused(change, message):
    raw = copy.deepcopy(M.MEKUVIK_A)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        MekuvikConfig.from_dict(raw)


def test_every_pass_has_caches_and_states_of_its_own_and_kept_pages_stay(case, engine):
    from ampere_kv_engine_amd.engine import StepEntry
    spec, layers, page = engine.spec, case["raw"]["layers"], case["page_size"]
    keys = [spec.cache_key(entry) for entry in spec.run_order]
    assert len(set(keys)) == len(keys) == len(engine.cache.layer_cache)
    for entry in spec.run_order:
        view, m = engine.cache.layer_cache[spec.cache_key(entry)], layers[entry.layer]["mixer"]
        kind = layers[entry.layer]["type"]
        if kind == "lightning":
            assert view.k is None and view.state.shape == (4, m["heads"] * m["dim"] * m["vdim"])
        elif kind == "attention":
            assert view.k.shape[1:] == (m["kv_heads"], page, m["dim"]) and view.v.shape[1:] == (m["kv_heads"], m["vdim"], page)
            assert view.state is None
        else:
            assert view.k.shape[1:] == (1, page, m["kv_rank"] + m["rot_dim"]) and view.state is None
    tensors = [view.k if view.k is not None else view.state for view in engine.cache.layer_cache.values()]
    assert len({t.data_ptr() for t in tensors}) == len(tensors)
    seq = engine.open("w")
    engine.step([StepEntry(seq, case["requests"]["d"], [])])
    engine.step([StepEntry(seq, case["requests"]["a"][:1], [])])    # (what a window has passed is given back when tokens register)
    windowed = 0
    for table, group in zip(seq.tables, engine.cache.groups):
        if group.need.window is None:
            continue
        windowed += 1
        kept = (group.need.keep_first + page - 1) // page
        assert table.num_held <= (group.need.window + page - 1) // page + 1 + kept
        assert all(p != RELEASED for p in table.pages[:kept]), "a page of the kept first tokens was given back"
        assert RELEASED in table.pages, "nothing behind the window was given back"
    assert windowed == sum(layer["type"] == "attention" and "mask" in layer["mixer"] for layer in layers)
    states = [view.state for view in engine.cache.layer_cache.values() if view.state is not None]
    assert all(state[seq.slot].any() for state in states)
    slot = seq.slot
    engine.close(seq)
    seq = engine.open("again")           # the slot comes round again: nothing of its predecessor is left
    assert seq.slot == slot and not any(state[slot].any() for state in states)
    engine.close(seq)
    assert engine.cache.num_free_pages == [engine.config.num_pages] * len(engine.cache.groups)


def test_a_table_keeps_the_pages_of_the_first_tokens():
    pool = PageAllocator(12)
    table = BlockTable(pool, 4, window=6, keep_first=5)          # two kept pages
    table.append_tokens(3)
    assert table.num_held == 1
    table.append_tokens(30)
    assert table.num_held == 9                                   # (pages are given back when tokens register, not before)
    table.append_tokens(1)                                       # position 33 reads keys from 28 on: pages 2 .. 6 go
    assert table.pages[:2] == (0, 1) and table.pages[2:7] == (RELEASED,) * 5 and RELEASED not in table.pages[7:]
    assert table.num_held == 4 and pool.num_free == 8
    for position in (0, 4, 7, 28, 33):
        table.locate(position)
    with pytest.raises(ValueError, match="passed"):
        table.locate(9)
    table.release()
    table.release()
    assert pool.num_free == 12
    plain_table = BlockTable(pool, 4, window=6)
    plain_table.append_tokens(33)
    plain_table.append_tokens(1)
    assert plain_table.pages[0] == RELEASED and plain_table.num_held == 2
    plain_table.release()


# ---- the plain implementation's own mechanisms, where a sentence of the design can be checked by hand -----------------

def test_plain_mechanisms_by_hand():
    assert plain.window_mask(5, 2, 1).int().tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [1, 1, 1, 0, 0], [1, 0, 1, 1, 0], [1, 0, 0, 1, 1]]
    assert plain.window_mask(4, 2).int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 0, 1, 1]]
    assert plain.window_mask(3, None, 7).int().tolist() == [[1, 0, 0], [1, 1, 0], [1, 1, 1]]
    torch.testing.assert_close(plain.rms_norm(torch.tensor([[3.0, -3.0]]), torch.tensor([0.5, 2.0]), 0.0), torch.tensor([[0.5, -2.0]]))
    assert plain.run_order(dict(layers=[0] * 4, loop=dict(start=1, stop=3, times=2))) == [
        (0, False), (1, False), (2, False), (1, True), (2, False), (3, False)]
    assert plain.run_order(dict(layers=[0] * 2)) == [(0, False), (1, False)]
    # pairs (0, 1) and (2, 3) are turned, each by its own frequency; the last two dimensions pass
    freqs, magnitude = plain.rotary_frequencies(4, 100.0)
    assert freqs.tolist() == [1.0, 0.1] and magnitude == 1.0
    turned = plain.rotate_interleaved(torch.arange(6.0).view(1, 1, 6), torch.tensor([2]), 4, freqs)
    assert torch.equal(turned[..., 4:], torch.tensor([[[4.0, 5.0]]]))
    torch.testing.assert_close(turned[0, 0, :4], torch.tensor([0 * math.cos(2.0) - 1 * math.sin(2.0), 1 * math.cos(2.0) + 0 * math.sin(2.0),
                                                                2 * math.cos(0.2) - 3 * math.sin(0.2), 3 * math.cos(0.2) + 2 * math.sin(0.2)]))
    # the ramp runs from pair lo = 0 to hi = 3 here, and cos and sin grow by 0.1 ln(factor) + 1
    base = [100.0 ** (-2.0 * i / 8) for i in range(4)]
    got, magnitude = plain.rotary_frequencies(8, 100.0, dict(factor=2.0, original=40.0, fast=4.0, slow=0.5))
    assert got.tolist() == pytest.approx([f / 2 * r + f * (1 - r) for f, r in zip(base, (0.0, 1 / 3, 2 / 3, 1.0))], rel=1e-12)
    assert magnitude == pytest.approx(0.1 * math.log(2.0) + 1.0)
    # the two largest scores are chosen and weigh as they are: sigmoids, not renormalised
    chosen, weights = plain.routed_choice(torch.tensor([[1.0, 0.0]]), torch.tensor([[0.0, 5.0], [2.0, 0.0], [-1.0, 0.0], [1.0, 0.0]]), 2)
    assert chosen.tolist() == [[1, 3]]
    torch.testing.assert_close(weights, torch.sigmoid(torch.tensor([[2.0, 1.0]])))


def test_linear_attention_by_hand():
    """One head, two key channels, one value, an identity behind silu's inverse: the state decays by one half a token."""
    inverse = lambda y: torch.tensor(y, dtype=torch.float64).apply_(
        lambda v: next(x / 1e4 for x in range(0, 100000) if x / 1e4 / (1 + math.exp(-x / 1e4)) >= v))
    h = torch.stack((inverse([1.0, 0.0, 2.0, 1.0, 0.0]), inverse([0.0, 1.0, 3.0, 1.0, 1.0]))).float()   # k | v | q per token
    pick = lambda lo, hi: torch.eye(5)[lo:hi]
    w = {"k": pick(0, 2), "v": pick(2, 3), "q": pick(3, 5), "g": torch.zeros(1, 5), "norm": torch.ones(1), "o": torch.eye(1)}
    m = dict(heads=1, dim=2, vdim=1, decay=[0.5])
    # token 0: S = [[2], [0]], o = q . S = 2;  token 1: S = [[1], [3]], o = 1 * 1 + 1 * 3 = 4; normed to +-1, gated by one half
    out = plain.lightning(h, w, m, 0.0)
    torch.testing.assert_close(out, torch.tensor([[0.5], [0.5]]), atol=1e-3, rtol=0)
    w["norm"] = torch.tensor([3.0])
    torch.testing.assert_close(plain.lightning(h, w, m, 0.0), torch.tensor([[1.5], [1.5]]), atol=3e-3, rtol=0)


def test_a_key_at_the_windows_edge_a_kept_key_and_a_far_key_decide_the_output():
    """The plain attentions with inputs made so that one key stands out: under a window it is seen from exactly `size`
    positions, a kept first token from every position, and without a window a key is seen from everywhere behind it."""
    n, size = 40, 7
    wide = lambda rows, cols, entries: torch.tensor([[entries.get((r, c), 0.0) for c in range(cols)] for r in range(rows)])

    def run(marked, keep, mask=True):
        h = torch.zeros(n, 3)
        h[:, 0] = 1.0                      # every token: the same query direction
        h[marked, 1] = 1.0                 # one position: a key along the queries, a value of its own
        m = dict(heads=1, kv_heads=1, dim=4, vdim=2, scale=40.0, rot=dict(dims=2, base=10000.0),
                 **({"mask": dict(size=size, keep_first=keep)} if mask else {}))
        # (dimension 2, beyond the rotated pair, carries the mark: the norm over the projection leaves its direction)
        w = {"q": wide(4, 3, {(2, 0): 1.0}), "k": wide(4, 3, {(2, 1): 1.0, (3, 0): 1.0}), "v": wide(2, 3, {(0, 1): 1.0, (1, 0): 0.01}),
             "q.norm": torch.ones(4), "k.norm": torch.ones(4), "o": torch.eye(2)}
        out = plain.attention(h, w, m, 1e-6)
        return (out[:, 0] > 0.5).nonzero().flatten().tolist()

    assert run(9, 2) == list(range(9, 9 + size))                 # a key behind the kept ones: `size` positions see it
    assert run(1, 2) == list(range(1, n))                        # a kept key: seen from everywhere
    assert run(2, 2) == list(range(2, 2 + size))                 # the first that is not kept
    assert run(1, 0) == list(range(1, 1 + size))
    assert run(3, 0, mask=False) == list(range(3, n))            # no window at all
