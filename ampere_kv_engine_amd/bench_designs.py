"""Prefill and decode throughput of the Keranex design (and, `--workload tukevik` / `lirulix` / `mekuvik`, of those designs) at sizes that resemble a real model's layers (random weights),
beside the dense Qwen3 decoder at equal width, depth, heads and active feed-forward width - the closest model the
engine has.  `python bench.py --workload keranex [--design-sizes s,m] [--layers L]` prints one JSON line per size:

  prefill  one request's 2,048-token prompt fed whole: tokens per second and milliseconds
  decode   `batch` requests with caches of `context` tokens, one token each per step, chosen greedily: tokens per second

A Keranex model here repeats the pattern [attention over a latent, the same, selective scan, attention reading the
second layer's latent], every layer with a routed feed-forward; its Qwen3 neighbour has as many layers of grouped-query
attention (a quarter as many kv heads) and a dense feed-forward as wide as the experts a token uses.
"""

from __future__ import annotations

import json
import time

PAGE_SIZE, PREFILL_TOKENS = 16, 2048

SIZES = {
    "s": dict(width=2048, vocab=32768, heads=16, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=768, window=1024,
              inner=4096, state=16, dt_rank=128, conv=4, experts=16, top=2, groups=4, keep=2, ff=1024),
    "m": dict(width=4096, vocab=65536, heads=32, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=1536, window=2048,
              inner=8192, state=16, dt_rank=256, conv=4, experts=32, top=4, groups=8, keep=4, ff=1024),
}


def keranex_config(size: dict, layers: int) -> dict:
    latent = lambda **more: dict(heads=size["heads"], dim=size["dim"], rot_dim=size["rot"], vdim=size["vdim"],
                                 kv_rank=size["kv_rank"], q_rank=size["q_rank"], mask=dict(size=size["window"]),
                                 scale=(size["dim"] + size["rot"]) ** -0.5, rot=dict(base=10000.0, dims=size["rot"]), **more)
    mlp = dict(kind="moe", expert=dict(ff=size["ff"]), router=dict(experts=size["experts"], top=size["top"],
               groups=dict(count=size["groups"], keep=size["keep"])))
    out = []
    for index in range(layers):
        place = index % 4
        if place == 2:
            out.append(dict(type="mamba1", mixer=dict(inner=size["inner"], state=size["state"], dt_rank=size["dt_rank"],
                                                      conv=size["conv"]), mlp=mlp))
        elif place == 3:
            out.append(dict(type="latent_attention", mixer=latent(kv_from=index - 2), mlp=mlp))
        else:
            out.append(dict(type="latent_attention", mixer=latent(), mlp=mlp))
    return dict(architecture="Keranex", vocab=size["vocab"], width=size["width"], norm=dict(eps=1e-5),
                embedding=dict(bigram=dict(buckets=size["vocab"] - 1, mul_prev=127, mul_cur=17)), layers=out)


# Tukevik at sizes of the same widths: the pattern [attention over chunks beside retention + dense feed-forward, recurrent
# unit + routed feed-forward, recurrent unit + dense, attention beside retention + routed]; a token uses `top` experts and
# the shared one, as wide together as the dense feed-forward.
TUKEVIK_SIZES = {
    "s": dict(width=2048, vocab=32768, heads=16, kv_heads=4, dim=128, vdim=128, chunk=4096, r_heads=4, r_dim=128, r_vdim=128,
              recurrent=2048, blocks=16, conv=4, experts=16, top=2, ff=1024, shared=1024, dense=3072),
    "m": dict(width=4096, vocab=65536, heads=32, kv_heads=8, dim=128, vdim=128, chunk=4096, r_heads=8, r_dim=128, r_vdim=128,
              recurrent=4096, blocks=16, conv=4, experts=32, top=4, ff=1024, shared=1024, dense=5120),
}


def tukevik_config(size: dict, layers: int) -> dict:
    parallel = dict(
        left=dict(heads=size["heads"], kv_heads=size["kv_heads"], dim=size["dim"], vdim=size["vdim"], mask=dict(size=size["chunk"]),
                  scale=size["dim"] ** -0.5, softcap=50.0), left_scale=0.7,
        right=dict(heads=size["r_heads"], dim=size["r_dim"], vdim=size["r_vdim"], rot=dict(base=1e4, dims=size["r_dim"]),
                   decay=[1.0 - 2.0 ** -(5 + h % 6) for h in range(size["r_heads"])]), right_scale=1.2)
    recurrent = dict(width=size["recurrent"], blocks=size["blocks"], conv=size["conv"])
    dense = dict(kind="dense", ff=size["dense"])
    routed = dict(kind="moe", expert=dict(ff=size["ff"]), router=dict(experts=size["experts"], top=size["top"]),
                  shared=dict(ff=size["shared"]))
    pattern = [("parallel", parallel, dense), ("rglru", recurrent, routed), ("rglru", recurrent, dense), ("parallel", parallel, routed)]
    return dict(architecture="Tukevik", vocab=size["vocab"], width=size["width"], norm=dict(eps=1e-6), residual_mult=0.6,
                layers=[dict(type=kind, mixer=mixer, mlp=mlp) for kind, mixer, mlp in (pattern[i % 4] for i in range(layers))])


# Lirulix at the same widths: the pattern [attention with a sink, delta rule, attention with a sink, differential
# attention over a window], every layer with a dense feed-forward, all layers inside one pass of the loop.  Beside it
# Tukevik (the closest design the engine has: attention with a sink on the same kernels, a mixer with a matrix state per
# head, float32 norms) with the same width, depth, heads and feed-forward width, its feed-forwards all dense.
LIRULIX_SIZES = {
    "s": dict(width=2048, vocab=32768, heads=16, kv_heads=4, dim=128, vdim=128, rot=64, d_heads=16, d_kv_heads=4, d_dim=64,
              d_vdim=128, window=1024, r_heads=16, r_kv_heads=16, r_dim=128, r_vdim=128, conv=4, decay_rank=64, gate_rank=64,
              ff=3072),
    "m": dict(width=4096, vocab=65536, heads=32, kv_heads=8, dim=128, vdim=128, rot=64, d_heads=32, d_kv_heads=8, d_dim=64,
              d_vdim=128, window=2048, r_heads=32, r_kv_heads=32, r_dim=128, r_vdim=128, conv=4, decay_rank=128, gate_rank=128,
              ff=5120),
}


def lirulix_config(size: dict, layers: int) -> dict:
    sink = dict(heads=size["heads"], kv_heads=size["kv_heads"], dim=size["dim"], vdim=size["vdim"], scale=size["dim"] ** -0.5,
                rot=dict(dims=size["rot"], base=1e6, scaling=dict(factor=4.0, original=4096, fast=32.0, slow=1.0)))
    two = dict(heads=size["d_heads"], kv_heads=size["d_kv_heads"], dim=size["d_dim"], vdim=size["d_vdim"], diff=0.3,
               scale=size["d_dim"] ** -0.5, mask=dict(size=size["window"]),
               rot=dict(dims=size["d_dim"], base=1e4, scaling=dict(factor=8.0, original=8192, low=1.0, high=4.0)))
    delta = dict(heads=size["r_heads"], kv_heads=size["r_kv_heads"], dim=size["r_dim"], vdim=size["r_vdim"], conv=size["conv"],
                 ranks=dict(decay=size["decay_rank"], gate=size["gate_rank"]))
    mlp = dict(kind="dense", ff=size["ff"])
    pattern = [("attention", sink), ("channel_delta", delta), ("attention", sink), ("attention_2", two)]
    return dict(architecture="Lirulix", vocab=size["vocab"], width=size["width"], norm=dict(eps=1e-6),
                layers=[dict(type=kind, mixer=mixer, mlp=mlp) for kind, mixer in (pattern[i % 4] for i in range(layers))],
                loop=dict(start=0, stop=layers, times=1))


def tukevik_beside_lirulix(size: dict, layers: int) -> dict:
    parallel = dict(
        left=dict(heads=size["heads"], kv_heads=size["kv_heads"], dim=size["dim"], vdim=size["vdim"], mask=dict(size=4096),
                  scale=size["dim"] ** -0.5, softcap=50.0), left_scale=0.7,
        right=dict(heads=size["r_heads"] // 4, dim=size["r_dim"], vdim=size["r_vdim"], rot=dict(base=1e4, dims=size["r_dim"]),
                   decay=[1.0 - 2.0 ** -(5 + h % 6) for h in range(size["r_heads"] // 4)]), right_scale=1.2)
    recurrent = dict(width=size["width"], blocks=16, conv=size["conv"])
    mlp = dict(kind="dense", ff=size["ff"])
    pattern = [("parallel", parallel), ("rglru", recurrent)]
    return dict(architecture="Tukevik", vocab=size["vocab"], width=size["width"], norm=dict(eps=1e-6), residual_mult=0.6,
                layers=[dict(type=kind, mixer=mixer, mlp=mlp) for kind, mixer in (pattern[i % 2] for i in range(layers))])


# Mekuvik at the same widths: the pattern [attention over a window that keeps the first tokens + dense feed-forward, linear
# attention + routed, attention over a latent + routed, linear attention + routed], one norm a layer, all layers inside
# one pass of the loop; a token uses `top` experts and the shared one, as wide together as the dense feed-forward.  Beside it
# Tukevik at its size of the same name (the closest design the engine has: the same attention kernels, retention on the
# same recurrence kernels, routed experts with a shared one through the same products) and Qwen3.
MEKUVIK_SIZES = {
    "s": dict(width=2048, vocab=32768, heads=16, kv_heads=4, dim=128, vdim=128, rot=64, window=1024, keep=4, l_heads=16, l_dim=128,
              l_vdim=128, m_heads=16, m_dim=128, m_rot=64, m_vdim=128, kv_rank=512, q_rank=768, experts=16, top=2, ff=1024,
              shared=1024, dense=3072),
    "m": dict(width=4096, vocab=65536, heads=32, kv_heads=8, dim=128, vdim=128, rot=64, window=2048, keep=4, l_heads=32, l_dim=128,
              l_vdim=128, m_heads=32, m_dim=128, m_rot=64, m_vdim=128, kv_rank=512, q_rank=1536, experts=32, top=4, ff=1024,
              shared=1024, dense=5120),
}


def mekuvik_config(size: dict, layers: int) -> dict:
    window = dict(heads=size["heads"], kv_heads=size["kv_heads"], dim=size["dim"], vdim=size["vdim"], scale=size["dim"] ** -0.5,
                  rot=dict(dims=size["rot"], base=1e6), mask=dict(size=size["window"], keep_first=size["keep"]))
    light = dict(heads=size["l_heads"], dim=size["l_dim"], vdim=size["l_vdim"],
                 decay=[1.0 - 2.0 ** -(3 + h % 8) for h in range(size["l_heads"])])
    latent = dict(heads=size["m_heads"], dim=size["m_dim"], rot_dim=size["m_rot"], vdim=size["m_vdim"], kv_rank=size["kv_rank"],
                  q_rank=size["q_rank"], scale=(size["m_dim"] + size["m_rot"]) ** -0.5,
                  rot=dict(dims=size["m_rot"], base=1e4, scaling=dict(factor=8.0, original=4096, fast=32.0, slow=1.0)))
    dense = dict(kind="dense", ff=size["dense"])
    routed = dict(kind="moe", expert=dict(ff=size["ff"]), router=dict(experts=size["experts"], top=size["top"]),
                  shared=dict(ff=size["shared"]))
    pattern = [("attention", window, dense), ("lightning", light, routed), ("latent_attention", latent, routed),
               ("lightning", light, routed)]
    return dict(architecture="Mekuvik", vocab=size["vocab"], width=size["width"], norm=dict(eps=1e-6), logit_scale=0.5,
                layers=[dict(type=kind, mixer=mixer, mlp=mlp) for kind, mixer, mlp in (pattern[i % 4] for i in range(layers))],
                loop=dict(start=0, stop=layers, times=1))


def qwen3_beside_tukevik(size: dict, layers: int) -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=layers, hidden_size=size["width"],
                num_attention_heads=size["heads"], num_key_value_heads=size["kv_heads"], head_dim=size["dim"],
                intermediate_size=size["dense"], vocab_size=size["vocab"], rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=True, hidden_act="silu")


def qwen3_config(size: dict, layers: int) -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=layers, hidden_size=size["width"],
                num_attention_heads=size["heads"], num_key_value_heads=max(size["heads"] // 4, 1), head_dim=128,
                intermediate_size=size["top"] * size["ff"], vocab_size=size["vocab"], rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")


def measure(config, batch: int, context: int, steps: int, warmup: int, graphs: bool = True) -> dict:
    import torch
    from .config import EngineConfig
    from .engine import LAST_TOKEN, Engine, StepEntry
    per_request = context + warmup + steps + 8
    pages = batch * ((per_request + PAGE_SIZE - 1) // PAGE_SIZE + 1) + PREFILL_TOKENS // PAGE_SIZE + 2
    engine = Engine.from_random(config, seed=0, engine_config=EngineConfig(
        dtype="bfloat16", page_size=PAGE_SIZE, num_pages=pages, max_seqs=batch + 1, max_batched_tokens=PREFILL_TOKENS,
        max_seq_len=max(per_request, PREFILL_TOKENS) + PAGE_SIZE, device="cuda:0", decode_graphs=graphs))
    for group in engine.cache.groups:       # any finite records: what they hold does not change the time
        group.pages.normal_(0.0, 0.5)
    generator = torch.Generator().manual_seed(0)
    sync = lambda: torch.cuda.synchronize(engine.device)
    vocab = engine.spec.vocab_size
    # ---- prefill
    samples = []
    for run in range(4):
        ids = torch.randint(0, vocab, (PREFILL_TOKENS,), generator=generator).tolist()
        seq = engine.open(f"p{run}")
        sync()
        started = time.perf_counter()
        engine.step([StepEntry(seq, ids, [PREFILL_TOKENS - 1])])
        sync()
        samples.append(time.perf_counter() - started)
        engine.close(seq)
    prefill = sorted(samples[1:])[1]
    # ---- decode
    seqs = [engine.open(f"d{i}") for i in range(batch)]
    for seq in seqs:
        engine.cache.reserve(seq, context - 1)
    first = torch.randint(0, vocab, (batch,), generator=generator).tolist()
    engine.choose(engine.step([StepEntry(seq, [token], [0]) for seq, token in zip(seqs, first)], borrow_logits=True))
    for _ in range(3 + warmup):
        engine.choose(engine.step([StepEntry(seq, LAST_TOKEN, [0]) for seq in seqs], borrow_logits=True))
    sync()
    started = time.perf_counter()
    for _ in range(steps):
        engine.choose(engine.step([StepEntry(seq, LAST_TOKEN, [0]) for seq in seqs], borrow_logits=True))
    sync()
    decode = (time.perf_counter() - started) / steps
    for seq in seqs:
        engine.close(seq)
    out = dict(prefill_tok_per_s=round(PREFILL_TOKENS / prefill, 1), prefill_ms=round(prefill * 1000, 3),
               decode_tok_per_s=round(batch / decode, 1), decode_ms_per_step=round(decode * 1000, 3),
               weight_gb_per_step=round(engine.model.weight_bytes_per_step() / 1e9, 3))
    del engine
    torch.cuda.empty_cache()
    return out


def design_workload(sizes: str, layers: int | None, batch: int, context: int, steps: int, warmup: int,
                    graphs: bool = True, only: str = "", design: str = "keranex") -> int:
    from .config import KeranexConfig, LirulixConfig, MekuvikConfig, Qwen3Config, TukevikConfig
    for name in [s for s in sizes.split(",") if s and design == "mekuvik"]:
        size, beside = MEKUVIK_SIZES[name], TUKEVIK_SIZES[name]
        count = layers or 8
        line = {"workload": "mekuvik", "sizes": name, "layers": count, "batch": batch, "context": context,
                "prefill_tokens": PREFILL_TOKENS, "dtype": "bf16", "data": "synthetic: random-init weights, random token ids",
                "shape": size}
        if only in ("", "mekuvik"):
            line["mekuvik"] = measure(MekuvikConfig.from_dict(mekuvik_config(size, count)), batch, context, steps, warmup, graphs)
        if only in ("", "tukevik"):
            line["tukevik_equal_size"] = measure(TukevikConfig.from_dict(tukevik_config(beside, count)), batch, context, steps, warmup, graphs)
        if only in ("", "qwen3"):
            line["qwen3_equal_size"] = measure(Qwen3Config.from_dict(qwen3_beside_tukevik(beside, count)), batch, context, steps, warmup, graphs)
        print(json.dumps(line), flush=True)
    if design == "mekuvik":
        return 0
    for name in [s for s in sizes.split(",") if s and design == "lirulix"]:
        size = LIRULIX_SIZES[name]
        count = layers or 8
        line = {"workload": "lirulix", "sizes": name, "layers": count, "batch": batch, "context": context,
                "prefill_tokens": PREFILL_TOKENS, "dtype": "bf16", "data": "synthetic: random-init weights, random token ids",
                "shape": size}
        if only in ("", "lirulix"):
            line["lirulix"] = measure(LirulixConfig.from_dict(lirulix_config(size, count)), batch, context, steps, warmup, graphs)
        if only in ("", "tukevik"):
            line["tukevik_equal_size"] = measure(TukevikConfig.from_dict(tukevik_beside_lirulix(size, count)), batch, context, steps, warmup, graphs)
        if only in ("", "qwen3"):
            line["qwen3_equal_size"] = measure(Qwen3Config.from_dict(qwen3_beside_tukevik(dict(size, dense=size["ff"]), count)), batch, context, steps, warmup, graphs)
        print(json.dumps(line), flush=True)
    if design == "lirulix":
        return 0
    for name in [s for s in sizes.split(",") if s and design == "tukevik"]:
        size = TUKEVIK_SIZES[name]
        count = layers or 8
        line = {"workload": "tukevik", "sizes": name, "layers": count, "batch": batch, "context": context,
                "prefill_tokens": PREFILL_TOKENS, "dtype": "bf16", "data": "synthetic: random-init weights, random token ids",
                "shape": size}
        if only in ("", "tukevik"):
            line["tukevik"] = measure(TukevikConfig.from_dict(tukevik_config(size, count)), batch, context, steps, warmup, graphs)
        if only in ("", "qwen3"):
            line["qwen3_equal_size"] = measure(Qwen3Config.from_dict(qwen3_beside_tukevik(size, count)), batch, context, steps, warmup, graphs)
        print(json.dumps(line), flush=True)
    if design == "tukevik":
        return 0
    for name in [s for s in sizes.split(",") if s]:
        size = SIZES[name]
        count = layers or 8
        line = {"workload": "keranex", "sizes": name, "layers": count, "batch": batch, "context": context,
                "prefill_tokens": PREFILL_TOKENS, "dtype": "bf16", "data": "synthetic: random-init weights, random token ids",
                "shape": size}
        if only in ("", "keranex"):
            line["keranex"] = measure(KeranexConfig.from_dict(keranex_config(size, count)), batch, context, steps, warmup, graphs)
        if only in ("", "qwen3"):
            line["qwen3_equal_size"] = measure(Qwen3Config.from_dict(qwen3_config(size, count)), batch, context, steps, warmup, graphs)
        print(json.dumps(line), flush=True)
    return 0
