"""Typed configuration of the Keranex decoder, read from the keys of its config.json.

A Keranex model is a list of layers, each with a mixer of its own kind and sizes - attention over a compressed
latent with a sliding window (`latent_attention`, which may read another layer's cache: `kv_from`) or a selective
scan (`mamba1`) - and a routed feed-forward (or none).  Every sublayer is normed before and after; the embedding
adds a row of a hashed table of token pairs.  Every size and every constant that can differ between models is a
key of config.json and travels from here into the part specifications; nothing has a default in code.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass

from .qwen3 import ConfigError
from .specs import LayerSpec, ModelSpec, RunEntry, part

MIXER_TYPES = ("latent_attention", "mamba1")


def _get(raw: dict, path: str, kind=int, positive: bool = True):
    """raw["a"]["b"] for path "a.b", with a message that names the path when it is absent or of the wrong type."""
    value = raw
    for key in path.split("."):
        if not isinstance(value, dict) or key not in value:
            raise ConfigError(f"config.json lacks {path}")
        value = value[key]
    if kind is int:
        if not isinstance(value, int) or isinstance(value, bool):
            raise ConfigError(f"config.json key {path} must be an integer, got {value!r}")
    elif kind is float:
        if not isinstance(value, (int, float)) or isinstance(value, bool):
            raise ConfigError(f"config.json key {path} must be a number, got {value!r}")
        value = float(value)
    if positive and value <= 0:
        raise ConfigError(f"config.json key {path} must be positive, got {value!r}")
    return value


@dataclass(frozen=True)
class KeranexConfig:
    raw: dict        # config.json as read (checked below; `to_dict` hands it back)

    architecture = "Keranex"

    # ---- construction ---------------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: dict) -> "KeranexConfig":
        config = cls(raw=json.loads(json.dumps(raw)))
        config._check()
        return config

    @classmethod
    def from_folder(cls, folder: str) -> "KeranexConfig":
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
        _get(raw, "vocab"), _get(raw, "width"), _get(raw, "norm.eps", float)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json key layers must be a non-empty list")
        bigram = raw.get("embedding", {}).get("bigram") if isinstance(raw.get("embedding"), dict) else None
        if bigram is not None:
            _get(bigram, "buckets"), _get(bigram, "mul_prev", positive=False), _get(bigram, "mul_cur", positive=False)
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            kind = layer.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}.type is {kind!r}; this design's mixers are {', '.join(MIXER_TYPES)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"{where}.mixer must be an object")
            if kind == "latent_attention":
                for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "mask.size", "rot.dims"):
                    _get(mixer, key)
                _get(mixer, "scale", float), _get(mixer, "rot.base", float)
                if mixer["rot"]["dims"] % 2 or mixer["rot"]["dims"] > mixer["rot_dim"]:
                    raise ConfigError(f"{where}.mixer.rot.dims must be even and at most rot_dim")
                source = mixer.get("kv_from")
                if source is not None:
                    if not isinstance(source, int) or not 0 <= source < len(layers) or source == index:
                        raise ConfigError(f"{where}.mixer.kv_from must name another layer")
                    other = layers[source]
                    if other.get("type") != "latent_attention" or other["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{where}.mixer.kv_from names layer {source}, which keeps no latent of its own")
                    if source > index:
                        raise ConfigError(f"{where}.mixer.kv_from names layer {source}, which runs later")
                    for key in ("kv_rank", "rot_dim"):
                        if other["mixer"].get(key) != mixer[key]:
                            raise ConfigError(f"{where}.mixer.{key} differs from that of layer {source}, whose latent it reads")
            else:
                for key in ("inner", "state", "dt_rank", "conv"):
                    _get(mixer, key)
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ConfigError(f"{where}.mlp.kind is {mlp.get('kind')!r}; this design's feed-forward is 'moe'")
                experts, top = _get(mlp, "router.experts"), _get(mlp, "router.top")
                count, keep = _get(mlp, "router.groups.count"), _get(mlp, "router.groups.keep")
                _get(mlp, "expert.ff")
                if experts % count or keep > count or top > keep * (experts // count):
                    raise ConfigError(f"{where}.mlp.router: {experts} experts in {count} groups of which {keep} are kept "
                                      f"cannot give {top} experts a token")

    # ---- the model this configuration describes -------------------------------------------------------
    def cache_window(self, owner: int) -> int:
        """Tokens that the layer which owns a latent cache must keep: the widest window among the layers that read it."""
        return max(self.layers[index]["mixer"]["mask"]["size"] for index in self.cache_readers(owner))

    def cache_readers(self, owner: int) -> list[int]:
        """The layers that read the records of layer `owner`: itself and those that name it as `kv_from`."""
        return [index for index, layer in enumerate(self.layers)
                if layer["type"] == "latent_attention" and (index == owner or layer["mixer"].get("kv_from") == owner)]

    def to_model_spec(self) -> ModelSpec:
        raw = self.raw
        hidden, eps = raw["width"], float(raw["norm"]["eps"])
        norm = part("rmsnorm", size=hidden, eps=eps, single_rounding=True)
        layers, order = [], []
        for index, layer in enumerate(self.layers):
            m = layer["mixer"]
            if layer["type"] == "latent_attention":
                source = m.get("kv_from")
                owner = index if source is None else source
                mixer = part("latent_attention", hidden_size=hidden, heads=m["heads"], head_dim=m["dim"],
                             rotated_dim=m["rot_dim"], value_dim=m["vdim"], kv_rank=m["kv_rank"], q_rank=m["q_rank"],
                             scale=float(m["scale"]), window=m["mask"]["size"], cache_window=self.cache_window(owner),
                             rotary_dims=m["rot"]["dims"], rotary_base=float(m["rot"]["base"]), eps=eps,
                             own_latent=source is None, name="mix",
                             reader_heads=tuple(self.layers[r]["mixer"]["heads"] for r in self.cache_readers(owner)))
                order.append(RunEntry(index, owner, writes_cache=source is None))
            else:
                mixer = part("selective_scan", hidden_size=hidden, inner=m["inner"], state=m["state"],
                             dt_rank=m["dt_rank"], taps=m["conv"], name="mix")
                order.append(RunEntry(index, index))
            mlp = layer.get("mlp")
            if mlp is None:
                feed_forward = part("none")
            else:
                r = mlp["router"]
                feed_forward = part("routed_experts", hidden_size=hidden, expert_size=mlp["expert"]["ff"],
                                    experts=r["experts"], top=r["top"], groups=r["groups"]["count"],
                                    groups_kept=r["groups"]["keep"], activation="relu_squared", name="mlp")
            layers.append(LayerSpec(
                block=part("sandwich", hidden_size=hidden, norm=norm, names=("norm1", "norm1b", "norm2", "norm2b")),
                mixer=mixer, feed_forward=feed_forward, prefix=f"l{index}."))
        bigram = raw.get("embedding", {}).get("bigram") if isinstance(raw.get("embedding"), dict) else None
        if bigram is None:
            embedding = part("embedding", vocab_size=raw["vocab"], hidden_size=hidden, name="embed")
        else:
            embedding = part("pair_hash_embedding", vocab_size=raw["vocab"], hidden_size=hidden, name="embed",
                             pair_name="bigram", buckets=bigram["buckets"], mul_prev=bigram["mul_prev"],
                             mul_cur=bigram["mul_cur"])
        return ModelSpec(
            architecture=self.architecture, vocab_size=raw["vocab"], hidden_size=hidden, embedding=embedding,
            layers=tuple(layers), run_order=tuple(order),
            final_norm=part("rmsnorm", size=hidden, eps=eps, single_rounding=True, name="final.norm"),
            head=part("linear_head", vocab_size=raw["vocab"], hidden_size=hidden, name="head", tied_to=None),
            eos_token_ids=tuple(raw.get("eos", ())) if isinstance(raw.get("eos"), list) else (),
        )
