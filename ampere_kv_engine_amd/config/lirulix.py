"""Typed configuration of the Lirulix decoder, read from the keys of its config.json.

A Lirulix model is a list of layers, each with a mixer of its own kind and sizes and a dense gated feed-forward (or
none):
  * `attention`: grouped-query attention with rotary positions over a part of the head, their frequencies stretched by
    a ramp between scaled and unscaled ones ("yarn"), and a learned sink per head in the softmax's denominator;
  * `attention_2`: differential attention - two maps per head over the same values, over a sliding window, with
    frequencies stretched piecewise by wavelength ("llama3"), the difference normed and gated per output value;
  * `channel_delta`: the gated delta rule with a decay per key channel behind short convolutions, its state in the
    request's slot.
The embedding is normed before the first layer; norm weights are stored around zero; `loop` names a run of layers that
is passed several times with the same weights, every pass with caches and states of its own and a vector of its own
added before its first layer.  Every size and every constant that can differ between models is a key of config.json
and travels from here into the part specifications; the two low ranks of a `channel_delta` mixer, which config.json
need not name (`mixer.ranks`), are read from the shapes of the checkpoint's tensors.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass

from .keranex import _get
from .qwen3 import ConfigError
from .specs import LayerSpec, ModelSpec, RunEntry, part

MIXER_TYPES = ("attention", "attention_2", "channel_delta")
UNIT_VECTOR_EPS = 1e-6          # q and k of the delta rule: x / sqrt(sum(x^2) + 1e-6), fixed by the design


def _checkpoint_shapes(folder: str) -> dict[str, tuple[int, ...]]:
    """Tensor name -> shape from the folder's safetensors (headers only), {} if it holds none."""
    from ..weights.loader import Checkpoint
    try:
        checkpoint = Checkpoint(folder)
    except FileNotFoundError:
        return {}
    return {name: checkpoint._meta[name][0] for name in checkpoint.names()}


@dataclass(frozen=True)
class LirulixConfig:
    raw: dict        # config.json as read, with the low ranks filled in (checked below; `to_dict` hands it back)

    architecture = "Lirulix"

    # ---- construction ---------------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: dict, shapes: dict | None = None) -> "LirulixConfig":
        """`shapes`: tensor shapes of the checkpoint, from which sizes that config.json does not name are taken."""
        raw = json.loads(json.dumps(raw))
        for index, layer in enumerate(raw.get("layers") or []):
            if not (isinstance(layer, dict) and layer.get("type") == "channel_delta" and isinstance(layer.get("mixer"), dict)):
                continue
            ranks = dict(layer["mixer"].get("ranks") or {})
            for key, tensor in (("decay", f"l{index}.mix.a1"), ("gate", f"l{index}.mix.g1")):
                if shapes is not None and tensor in shapes:
                    found = int(shapes[tensor][0])
                    if key in ranks and ranks[key] != found:
                        raise ConfigError(f"layers[{index}].mixer.ranks.{key} is {ranks[key]}, the checkpoint's {tensor} has {found} rows")
                    ranks[key] = found
            layer["mixer"]["ranks"] = ranks
        config = cls(raw=raw)
        config._check()
        return config

    @classmethod
    def from_folder(cls, folder: str) -> "LirulixConfig":
        with open(os.path.join(folder, "config.json")) as handle:
            return cls.from_dict(json.load(handle), _checkpoint_shapes(folder))

    def to_dict(self) -> dict:
        return json.loads(json.dumps(self.raw))

    @property
    def vocab_size(self) -> int:
        return self.raw["vocab"]

    @property
    def hidden_size(self) -> int:
        return self.raw["width"]

    @property
    def layers(self) -> list[dict]:
        return self.raw["layers"]

    def _check(self) -> None:
        raw = self.raw
        _get(raw, "vocab"), _get(raw, "width"), _get(raw, "norm.eps", float)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json key layers must be a non-empty list")
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}.type is {kind!r}; this design's mixers are {', '.join(MIXER_TYPES)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"{where}.mixer must be an object")
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _get(mixer, key)
            if mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"{where}.mixer.heads {mixer['heads']} is no multiple of kv_heads {mixer['kv_heads']}")
            if kind == "channel_delta":
                _get(mixer, "conv")
                for key in ("decay", "gate"):
                    if not isinstance(mixer["ranks"].get(key), int) or mixer["ranks"][key] <= 0:
                        raise ConfigError(f"{where}.mixer.ranks.{key} is named neither by config.json nor by a checkpoint's tensors")
            else:
                _get(mixer, "scale", float)
                dims = _get(mixer, "rot.dims")
                _get(mixer, "rot.base", float)
                if dims % 2 or dims > mixer["dim"]:
                    raise ConfigError(f"{where}.mixer.rot.dims must be even and at most dim {mixer['dim']}")
                scaling = mixer["rot"].get("scaling")
                if scaling is not None:
                    for key in ("factor", "original") + (("fast", "slow") if kind == "attention" else ("low", "high")):
                        _get(mixer, f"rot.scaling.{key}", float)
                if mixer.get("mask") is not None:
                    _get(mixer, "mask.size")
                if kind == "attention_2":
                    _get(mixer, "diff", float, positive=False)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp.kind must be dense")
                _get(mlp, "ff")
        loop = raw.get("loop")
        if loop is not None:
            start, stop, times = _get(raw, "loop.start", positive=False), _get(raw, "loop.stop"), _get(raw, "loop.times")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop.start .. loop.stop must name layers of the model, got {start} .. {stop} of {len(layers)}")

    # ---- the model this configuration describes -------------------------------------------------------
    def run_order(self) -> tuple[RunEntry, ...]:
        count, loop = len(self.layers), self.raw.get("loop")
        if loop is None:
            return tuple(RunEntry(i, i) for i in range(count))
        start, stop, times = loop["start"], loop["stop"], loop["times"]
        order = [RunEntry(i, i) for i in range(start)]
        for turn in range(times):
            order += [RunEntry(i, i, cache_copy=turn, adds_row=turn if i == start else None) for i in range(start, stop)]
        return tuple(order + [RunEntry(i, i) for i in range(stop, count)])

    @staticmethod
    def _rotation(rot: dict, kind: str):
        scaling = rot.get("scaling")
        if scaling is not None:
            scaling = dict(kind=kind, **{key: float(value) for key, value in scaling.items()})
        return part("rope_scaled", dims=rot["dims"], base=float(rot["base"]), scaling=scaling)

    def to_model_spec(self) -> ModelSpec:
        raw = self.raw
        hidden, eps = raw["width"], float(raw["norm"]["eps"])
        norm = part("rmsnorm", size=hidden, eps=eps, single_rounding=True, unit_offset=True)
        layers = []
        for index, layer in enumerate(self.layers):
            m, kind = layer["mixer"], layer["type"]
            window = m["mask"]["size"] if m.get("mask") is not None else None
            if kind == "attention":
                mixer = part("gated_attention", hidden_size=hidden, q_heads=m["heads"], kv_heads=m["kv_heads"],
                             head_dim=m["dim"], value_dim=m["vdim"], scale=float(m["scale"]), softcap=None, chunk=None,
                             window=window, sink="learned", unit_norm_eps=None, head_gate=False,
                             position=self._rotation(m["rot"], "yarn"), name="mix")
            elif kind == "attention_2":
                mixer = part("differential_attention", hidden_size=hidden, q_heads=m["heads"], kv_heads=m["kv_heads"],
                             head_dim=m["dim"], value_dim=m["vdim"], scale=float(m["scale"]), window=window,
                             constant=float(m["diff"]), eps=eps, position=self._rotation(m["rot"], "llama3"), name="mix")
            else:
                mixer = part("gated_delta_rule", hidden_size=hidden, heads=m["heads"], kv_heads=m["kv_heads"],
                             head_dim=m["dim"], value_dim=m["vdim"], taps=m["conv"], decay_rank=m["ranks"]["decay"],
                             gate_rank=m["ranks"]["gate"], unit_eps=UNIT_VECTOR_EPS, eps=eps, name="mix")
            mlp = layer.get("mlp")
            feed_forward = part("none") if mlp is None else part(
                "swiglu", hidden_size=hidden, intermediate_size=mlp["ff"], name="mlp", names=("gate", "up", "down"),
                activation="gelu_tanh")
            layers.append(LayerSpec(
                block=part("scaled_prenorm", hidden_size=hidden, norm=norm, residual_scale=1.0, names=("norm1", "norm2")),
                mixer=mixer, feed_forward=feed_forward, prefix=f"l{index}."))
        loop = raw.get("loop")
        return ModelSpec(
            architecture=self.architecture, vocab_size=raw["vocab"], hidden_size=hidden,
            embedding=part("normed_embedding", vocab_size=raw["vocab"], hidden_size=hidden, name="embed", norm=norm,
                           norm_name="embed.norm"),
            layers=tuple(layers), run_order=self.run_order(),
            final_norm=part("rmsnorm", size=hidden, eps=eps, single_rounding=True, unit_offset=True, name="final.norm"),
            head=part("linear_head", vocab_size=raw["vocab"], hidden_size=hidden, name="head"),
            eos_token_ids=tuple(raw.get("eos", ())) if isinstance(raw.get("eos"), list) else (),
            pass_vectors=part("row_table", rows=loop["times"], hidden_size=hidden, name="loop.step") if loop is not None else None,
        )
