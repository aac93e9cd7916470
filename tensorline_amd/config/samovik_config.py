"""Typed configuration of the Samovik decoder: a stack of layers of different kinds.

``config.json`` gives: ``architecture`` "Samovik", ``vocab``, ``width``, ``norm.eps``,
``token_side.dim`` (or no ``token_side``: no per-layer token input), and ``layers``, a list with one
entry per layer: ``type`` (``latent_attention``, ``lightning`` or ``wkv``), ``mixer`` (that mixer's
sizes and constants) and ``mlp`` (the routed feed-forward: ``kind`` "moe", ``router`` {experts, top},
``expert`` {ff, limit}, ``shared`` {ff, limit} or null; or null for a layer without feed-forward).
One size is not in config.json: the width of the decay's bottleneck in a ``wkv`` mixer is the first
dimension of its ``w1`` tensor; ``with_shapes`` takes it from the checkpoint's header, and a
configuration made by hand (random weights) names it ``decay_rank``.
"""
from __future__ import annotations

import copy
import json
import os
from dataclasses import dataclass, field
from typing import Any, Mapping

from tensorline_amd.config.model_config import ConfigError

MIXER_KEYS = {
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"),
    "lightning": ("heads", "dim", "vdim", "decay"),
    "wkv": ("heads", "dim"),
}


def _positive_int(where: str, d: Mapping[str, Any], key: str) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class SamovikConfig:
    vocab_size: int
    hidden_size: int
    layers: tuple = ()                      # the entries of config.json's ``layers``, checked
    norm_eps: float = 1e-6
    token_side_dim: int = 0                 # 0: no per-layer token input
    eos_token_id: tuple[int, ...] = ()
    max_position_embeddings: int = 1 << 30
    architecture: str = "Samovik"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False, hash=False)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "SamovikConfig":
        vocab, width = _positive_int("", d, "vocab"), _positive_int("", d, "width")
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        norm = d.get("norm") or {}
        if "eps" not in norm:
            raise ConfigError("config.json: norm.eps is missing")
        layers = []
        for i, layer in enumerate(raw_layers):
            where = f"layers[{i}]"
            kind = layer.get("type")
            if kind not in MIXER_KEYS:
                raise ConfigError(f"config.json: {where}.type {kind!r} is unknown; known: {', '.join(sorted(MIXER_KEYS))}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"config.json: {where}.mixer is missing")
            for key in MIXER_KEYS[kind]:
                if key not in mixer:
                    raise ConfigError(f"config.json: {where}.mixer.{key} is missing")
            for key in ("heads", "dim"):
                _positive_int(where + ".mixer", mixer, key)
            if kind == "lightning" and len(mixer["decay"]) != mixer["heads"]:
                raise ConfigError(f"config.json: {where}.mixer.decay must have one entry per head")
            if kind == "latent_attention":
                rot = mixer["rot"]
                if not isinstance(rot, dict) or "base" not in rot or int(rot.get("dims", mixer["rot_dim"])) != int(mixer["rot_dim"]):
                    raise ConfigError(f"config.json: {where}.mixer.rot must give 'base' and turn rot_dim dimensions")
                sc = rot.get("scaling")
                if sc and any(k not in sc for k in ("factor", "original", "fast", "slow")):
                    raise ConfigError(f"config.json: {where}.mixer.rot.scaling needs factor, original, fast and slow")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"config.json: {where}.mlp.kind {mlp.get('kind')!r} is unknown; known: moe")
                for part, keys in (("router", ("experts", "top")), ("expert", ("ff", "limit"))):
                    if not isinstance(mlp.get(part), dict) or any(k not in mlp[part] for k in keys):
                        raise ConfigError(f"config.json: {where}.mlp.{part} needs {' and '.join(keys)}")
                if mlp["router"]["top"] > mlp["router"]["experts"]:
                    raise ConfigError(f"config.json: {where}.mlp.router.top exceeds the number of experts")
                if mlp.get("shared") and any(k not in mlp["shared"] for k in ("ff", "limit")):
                    raise ConfigError(f"config.json: {where}.mlp.shared needs ff and limit")
            layers.append(copy.deepcopy(dict(layer)))
        side = d.get("token_side")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "token_side", "eos_token_id",
                 "max_position_embeddings"}
        return cls(vocab_size=vocab, hidden_size=width, layers=tuple(layers), norm_eps=float(norm["eps"]),
                   token_side_dim=_positive_int("token_side", side, "dim") if side else 0, eos_token_id=eos_ids,
                   max_position_embeddings=int(d.get("max_position_embeddings", 1 << 30)),
                   extra={k: v for k, v in d.items() if k not in known})

    @classmethod
    def from_json(cls, path: str | os.PathLike) -> "SamovikConfig":
        p = os.fspath(path)
        if os.path.isdir(p):
            p = os.path.join(p, "config.json")
        with open(p, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def needs_shapes(self) -> bool:
        return any(layer["type"] == "wkv" and "decay_rank" not in layer["mixer"] for layer in self.layers)

    def with_shapes(self, shapes: Mapping[str, tuple]) -> "SamovikConfig":
        """The sizes that only a tensor's shape gives, from ``shapes`` (tensor name -> shape)."""
        layers = copy.deepcopy(list(self.layers))
        for i, layer in enumerate(layers):
            if layer["type"] == "wkv" and "decay_rank" not in layer["mixer"]:
                name = f"l{i}.mix.w1"
                if name not in shapes or len(shapes[name]) != 2:
                    raise ConfigError(f"the checkpoint has no matrix {name!r} to read the decay's bottleneck width from")
                layer["mixer"]["decay_rank"] = int(shapes[name][0])
        return SamovikConfig(self.vocab_size, self.hidden_size, tuple(layers), self.norm_eps, self.token_side_dim,
                             self.eos_token_id, self.max_position_embeddings, self.architecture, self.extra)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                               "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(list(self.layers))}
        if self.token_side_dim:
            out["token_side"] = {"dim": self.token_side_dim}
        if self.eos_token_id:
            out["eos_token_id"] = list(self.eos_token_id)
        return out
