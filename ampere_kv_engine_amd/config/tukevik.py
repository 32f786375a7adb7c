"""Typed configuration of the Tukevik decoder, read from the keys of its config.json.

A Tukevik model is a list of layers, each with a mixer of its own kind and sizes and a feed-forward (or none):
  * `rglru`: a recurrent block - a gated branch beside a short causal convolution followed by a real-gated linear
    recurrent unit whose two gates are block-diagonal;
  * `parallel`: two mixers side by side that read the same input - `left`, grouped-query attention over chunks of
    positions with unit-normed queries and keys, a softcap on the scores, a sink in the softmax's denominator and a gate
    per head; `right`, retention with rotary positions and a fixed decay per head - added with a constant each.
Feed-forwards are dense (`silu(gate) * up`) or routed (`moe`: the top experts by logit, weighted by the softmax over the
chosen logits, plus a shared expert behind a sigmoid gate).  Every branch is added to the residual sum times
`residual_mult`; the head is the embedding table.  Every size and every constant that can differ between models is a
key of config.json and travels from here into the part specifications; nothing has a default in code.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass

from .keranex import _get
from .qwen3 import ConfigError
from .specs import LayerSpec, ModelSpec, RunEntry, part

MIXER_TYPES = ("rglru", "parallel")
MLP_KINDS = ("dense", "moe")
RGLRU_DECAY_CONSTANT = 8.0          # log a = -8 r softplus(lam): fixed by the design


@dataclass(frozen=True)
class TukevikConfig:
    raw: dict        # config.json as read (checked below; `to_dict` hands it back)

    architecture = "Tukevik"

    # ---- construction ---------------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: dict) -> "TukevikConfig":
        config = cls(raw=json.loads(json.dumps(raw)))
        config._check()
        return config

    @classmethod
    def from_folder(cls, folder: str) -> "TukevikConfig":
        with open(os.path.join(folder, "config.json")) as handle:
            return cls.from_dict(json.load(handle))

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
        _get(raw, "vocab"), _get(raw, "width"), _get(raw, "norm.eps", float), _get(raw, "residual_mult", float, positive=False)
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
            if kind == "rglru":
                width, blocks = _get(mixer, "width"), _get(mixer, "blocks")
                _get(mixer, "conv")
                if width % blocks:
                    raise ConfigError(f"{where}.mixer.width {width} is no multiple of its blocks {blocks}")
            else:
                for side in ("left", "right"):
                    if not isinstance(mixer.get(side), dict):
                        raise ConfigError(f"{where}.mixer.{side} must be an object")
                    _get(mixer, f"{side}_scale", float, positive=False)
                left, right = mixer["left"], mixer["right"]
                for key in ("heads", "kv_heads", "dim", "vdim"):
                    _get(left, key)
                _get(left, "scale", float)
                if left["heads"] % left["kv_heads"]:
                    raise ConfigError(f"{where}.mixer.left.heads {left['heads']} is no multiple of kv_heads {left['kv_heads']}")
                if left.get("softcap") is not None:
                    _get(left, "softcap", float)
                if left.get("mask") is not None:
                    _get(left, "mask.size")
                for key in ("heads", "dim", "vdim"):
                    _get(right, key)
                decay = right.get("decay")
                if (not isinstance(decay, list) or len(decay) != right["heads"]
                        or not all(isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay)):
                    raise ConfigError(f"{where}.mixer.right.decay must list one number for each of the {right['heads']} heads")
                if right.get("rot") is not None:
                    dims = _get(right, "rot.dims")
                    _get(right, "rot.base", float)
                    if dims % 2 or dims > right["dim"]:
                        raise ConfigError(f"{where}.mixer.right.rot.dims must be even and at most dim {right['dim']}")
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

    # ---- the model this configuration describes -------------------------------------------------------
    def to_model_spec(self) -> ModelSpec:
        raw = self.raw
        hidden, eps, mult = raw["width"], float(raw["norm"]["eps"]), float(raw["residual_mult"])
        norm = part("rmsnorm", size=hidden, eps=eps, single_rounding=True)
        layers = []
        for index, layer in enumerate(self.layers):
            m = layer["mixer"]
            if layer["type"] == "rglru":
                mixer = part("rglru", hidden_size=hidden, width=m["width"], blocks=m["blocks"], taps=m["conv"],
                             decay_constant=RGLRU_DECAY_CONSTANT, name="mix")
            else:
                left, right = m["left"], m["right"]
                mask, rot = left.get("mask"), right.get("rot")
                attention = part("gated_attention", hidden_size=hidden, q_heads=left["heads"], kv_heads=left["kv_heads"],
                                 head_dim=left["dim"], value_dim=left["vdim"], scale=float(left["scale"]),
                                 softcap=float(left["softcap"]) if left.get("softcap") is not None else None,
                                 chunk=mask["size"] if mask is not None else None, window=None, sink=True,
                                 unit_norm_eps=eps, head_gate=True, bias_suffix=".b", name="mix.left")
                retention = part("retention", hidden_size=hidden, heads=right["heads"], head_dim=right["dim"],
                                 value_dim=right["vdim"], decay=tuple(float(d) for d in right["decay"]),
                                 rotary_dims=rot["dims"] if rot is not None else 0,
                                 rotary_base=float(rot["base"]) if rot is not None else 0.0, eps=eps, name="mix.right")
                mixer = part("parallel", hidden_size=hidden,
                             branches=((attention, float(m["left_scale"])), (retention, float(m["right_scale"]))))
            mlp = layer.get("mlp")
            if mlp is None:
                feed_forward = part("none")
            elif mlp["kind"] == "dense":
                feed_forward = part("swiglu", hidden_size=hidden, intermediate_size=mlp["ff"], name="mlp",
                                    names=("gate", "up", "down"))
            else:
                shared = mlp.get("shared")
                feed_forward = part("routed_experts", hidden_size=hidden, expert_size=mlp["expert"]["ff"],
                                    experts=mlp["router"]["experts"], top=mlp["router"]["top"], activation="silu_gated",
                                    weights="softmax_chosen", router_bias=True,
                                    shared_size=shared["ff"] if shared is not None else None, name="mlp")
            layers.append(LayerSpec(
                block=part("scaled_prenorm", hidden_size=hidden, norm=norm, residual_scale=mult, names=("norm1", "norm2")),
                mixer=mixer, feed_forward=feed_forward, prefix=f"l{index}."))
        return ModelSpec(
            architecture=self.architecture, vocab_size=raw["vocab"], hidden_size=hidden,
            embedding=part("embedding", vocab_size=raw["vocab"], hidden_size=hidden, name="embed"),
            layers=tuple(layers), run_order=tuple(RunEntry(i, i) for i in range(len(layers))),
            final_norm=part("rmsnorm", size=hidden, eps=eps, single_rounding=True, name="final.norm"),
            head=part("linear_head", vocab_size=raw["vocab"], hidden_size=hidden, name="head", tied_to="embed"),
            eos_token_ids=tuple(raw.get("eos", ())) if isinstance(raw.get("eos"), list) else (),
        )
