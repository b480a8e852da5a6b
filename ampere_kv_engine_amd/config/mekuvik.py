"""Typed configuration of the Mekuvik decoder, read from the keys of its config.json.

A Mekuvik model is a list of layers.  Every layer has ONE norm whose output both of its branches read - a mixer and a
feed-forward (or none) - and their outputs are added to the residual sum together.  The mixers:
  * `lightning`: linear attention with a fixed decay per head - q, k and v behind silu, a state per head, the heads'
    outputs normed together with a weight and gated by a sigmoid;
  * `attention`: grouped-query attention whose queries and keys are normed over their whole projection, rotated over
    the first `rot.dims` dimensions of every head in interleaved pairs, over a sliding window that also keeps a request's
    first tokens;
  * `latent_attention`: attention whose keys and values are expanded from a compressed latent per token, with one
    rotated key part for all heads, stretched rotation frequencies and a sigmoid gate on the heads' outputs.
Feed-forwards are dense (`silu(gate) * up`) or routed (`moe`: the experts with the largest sigmoid scores, the score
multiplying what the expert reads, experts of the form down(gelu(up x)), plus a shared expert that every token uses).
`loop` names a run of layers that is passed several times with the same weights, every pass with caches and states of
its own; before every pass but the first the embedding's output is added to the residual sum.  The head is the
embedding table, and the logits are multiplied by `logit_scale`.  Every size and every constant that can differ between
models is a key of config.json and travels from here into the part specifications; a latent query's rank, if
config.json does not name it, is read from the checkpoint's tensor shapes.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass

from .keranex import _get
from .lirulix import _checkpoint_shapes
from .qwen3 import ConfigError
from .specs import LayerSpec, ModelSpec, RunEntry, part

MIXER_TYPES = ("lightning", "attention", "latent_attention")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class MekuvikConfig:
    raw: dict        # config.json as read (checked below; `to_dict` hands it back)

    architecture = "Mekuvik"

    # ---- construction ---------------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: dict, shapes: dict | None = None) -> "MekuvikConfig":
        """`shapes`: tensor shapes of the checkpoint, from which a size that config.json does not name is taken."""
        raw = json.loads(json.dumps(raw))
        for index, layer in enumerate(raw.get("layers") or []):
            if isinstance(layer, dict) and layer.get("type") == "latent_attention" and isinstance(layer.get("mixer"), dict):
                tensor = f"l{index}.mix.dq"
                if "q_rank" not in layer["mixer"] and shapes is not None and tensor in shapes:
                    layer["mixer"]["q_rank"] = int(shapes[tensor][0])
        config = cls(raw=raw)
        config._check()
        return config

    @classmethod
    def from_folder(cls, folder: str) -> "MekuvikConfig":
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

    @staticmethod
    def _check_rotation(mixer: dict, where: str, width: int) -> None:
        dims = _get(mixer, "rot.dims")
        _get(mixer, "rot.base", float)
        if dims % 2 or dims > width:
            raise ConfigError(f"{where}.mixer.rot.dims must be even and at most {width}")
        if mixer["rot"].get("scaling") is not None:
            for key in ("factor", "original", "fast", "slow"):
                _get(mixer, f"rot.scaling.{key}", float)

    def _check(self) -> None:
        raw = self.raw
        _get(raw, "vocab"), _get(raw, "width"), _get(raw, "norm.eps", float)
        if raw.get("logit_scale") is not None:
            _get(raw, "logit_scale", float)
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
            for key in ("heads", "dim", "vdim"):
                _get(mixer, key)
            if kind == "lightning":
                decay = mixer.get("decay")
                if (not isinstance(decay, list) or len(decay) != mixer["heads"]
                        or not all(isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay)):
                    raise ConfigError(f"{where}.mixer.decay must list one number for each of the {mixer['heads']} heads")
            elif kind == "attention":
                _get(mixer, "kv_heads"), _get(mixer, "scale", float)
                if mixer["heads"] % mixer["kv_heads"]:
                    raise ConfigError(f"{where}.mixer.heads {mixer['heads']} is no multiple of kv_heads {mixer['kv_heads']}")
                if mixer.get("rot") is not None:
                    self._check_rotation(mixer, where, mixer["dim"])
                if mixer.get("mask") is not None:
                    _get(mixer, "mask.size")
                    if mixer["mask"].get("keep_first") is not None:
                        _get(mixer, "mask.keep_first", positive=False)
                        if mixer["mask"]["keep_first"] < 0:
                            raise ConfigError(f"{where}.mixer.mask.keep_first must not be negative")
            else:
                for key in ("rot_dim", "kv_rank", "q_rank"):
                    if key == "q_rank" and key not in mixer:
                        raise ConfigError(f"{where}.mixer.q_rank is named neither by config.json nor by a checkpoint's tensors")
                    _get(mixer, key)
                _get(mixer, "scale", float)
                self._check_rotation(mixer, where, mixer["rot_dim"])
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                raise ConfigError(f"{where}.mlp.kind must be one of {', '.join(MLP_KINDS)}")
            if mlp["kind"] == "dense":
                _get(mlp, "ff")
            else:
                experts, top = _get(mlp, "router.experts"), _get(mlp, "router.top")
                _get(mlp, "expert.ff")
                if top > experts:
                    raise ConfigError(f"{where}.mlp.router: {top} experts a token cannot be chosen from {experts} experts")
                if mlp.get("shared") is not None:
                    _get(mlp, "shared.ff")
        loop = raw.get("loop")
        if loop is not None:
            start, stop = _get(raw, "loop.start", positive=False), _get(raw, "loop.stop")
            _get(raw, "loop.times")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop.start .. loop.stop must name layers of the model, got {start} .. {stop} of {len(layers)}")

    # ---- the model this configuration describes -------------------------------------------------------
    def run_order(self) -> tuple[RunEntry, ...]:
        """Layers start .. stop - 1 run `times` times in a row, every time with a cache of its own; every pass but the
        first begins by adding the embedding's output to the residual sum."""
        count, loop = len(self.layers), self.raw.get("loop")
        if loop is None:
            return tuple(RunEntry(i, i) for i in range(count))
        start, stop, times = loop["start"], loop["stop"], loop["times"]
        order = [RunEntry(i, i) for i in range(start)]
        for turn in range(times):
            order += [RunEntry(i, i, cache_copy=turn, adds_embedding=turn > 0 and i == start) for i in range(start, stop)]
        return tuple(order + [RunEntry(i, i) for i in range(stop, count)])

    @staticmethod
    def _rotation(rot: dict):
        scaling = rot.get("scaling")
        if scaling is not None:
            scaling = dict(kind="yarn", **{key: float(scaling[key]) for key in ("factor", "original", "fast", "slow")})
        return part("rope_scaled", dims=rot["dims"], base=float(rot["base"]), scaling=scaling, layout="interleaved")

    def to_model_spec(self) -> ModelSpec:
        raw = self.raw
        hidden, eps = raw["width"], float(raw["norm"]["eps"])
        norm = part("rmsnorm", size=hidden, eps=eps, single_rounding=True)
        layers = []
        for index, layer in enumerate(self.layers):
            m, kind = layer["mixer"], layer["type"]
            if kind == "lightning":
                mixer = part("retention", hidden_size=hidden, heads=m["heads"], head_dim=m["dim"], value_dim=m["vdim"],
                             decay=tuple(float(d) for d in m["decay"]), rotary_dims=0, rotary_base=0.0, key_scale=1.0,
                             eps=eps, input_activation="silu", norm="all_heads", gate="sigmoid", name="mix")
            elif kind == "attention":
                mask = m.get("mask")
                mixer = part("gated_attention", hidden_size=hidden, q_heads=m["heads"], kv_heads=m["kv_heads"],
                             head_dim=m["dim"], value_dim=m["vdim"], scale=float(m["scale"]), softcap=None, chunk=None,
                             window=mask["size"] if mask is not None else None,
                             keep_first=(mask.get("keep_first") or 0) if mask is not None else 0, sink=False,
                             unit_norm_eps=None, projection_norm_eps=eps, head_gate=False,
                             position=self._rotation(m["rot"]) if m.get("rot") is not None else None, name="mix")
            else:
                mixer = part("latent_attention", hidden_size=hidden, heads=m["heads"], head_dim=m["dim"],
                             rotated_dim=m["rot_dim"], value_dim=m["vdim"], kv_rank=m["kv_rank"], q_rank=m["q_rank"],
                             scale=float(m["scale"]), eps=eps, window=None, rotary_dims=m["rot"]["dims"],
                             position=self._rotation(m["rot"]), gate=True, name="mix")
            mlp = layer.get("mlp")
            if mlp is None:
                feed_forward = part("none")
            elif mlp["kind"] == "dense":
                feed_forward = part("swiglu", hidden_size=hidden, intermediate_size=mlp["ff"], name="mlp",
                                    names=("gate", "up", "down"))
            else:
                shared = mlp.get("shared")
                feed_forward = part("routed_experts", hidden_size=hidden, expert_size=mlp["expert"]["ff"],
                                    experts=mlp["router"]["experts"], top=mlp["router"]["top"], activation="gelu",
                                    weights="sigmoid_chosen", weight_on_input=True,
                                    shared_size=shared["ff"] if shared is not None else None, shared_gate=False, name="mlp")
            layers.append(LayerSpec(block=part("shared_norm", hidden_size=hidden, norm=norm, residual_scale=1.0, name="norm1"),
                                    mixer=mixer, feed_forward=feed_forward, prefix=f"l{index}."))
        scale = float(raw["logit_scale"]) if raw.get("logit_scale") is not None else 1.0
        return ModelSpec(
            architecture=self.architecture, vocab_size=raw["vocab"], hidden_size=hidden,
            embedding=part("embedding", vocab_size=raw["vocab"], hidden_size=hidden, name="embed"),
            layers=tuple(layers), run_order=self.run_order(),
            # logits = E norm(x) * logit_scale: the constant rides on the final norm's weight
            final_norm=part("rmsnorm", size=hidden, eps=eps, single_rounding=True, output_scale=scale, name="final.norm"),
            head=part("linear_head", vocab_size=raw["vocab"], hidden_size=hidden, name="head", tied_to="embed"),
            eos_token_ids=tuple(raw.get("eos", ())) if isinstance(raw.get("eos"), list) else (),
        )
