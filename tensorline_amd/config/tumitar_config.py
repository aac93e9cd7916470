"""Typed configuration of the Tumitar decoder: layers of two kinds of mixers, part of the stack run
several times over.

``config.json`` gives: ``architecture`` "Tumitar", ``vocab``, ``width``, ``norm.eps``,
``embedding.scale``, ``layers`` (one entry per layer: ``type`` "parallel" or "rglru", ``mixer`` with that
mixer's sizes and constants, ``mlp`` = {kind "dense", ff} or {kind "moe", router {experts, top, scale},
expert {ff}} or null), and optionally ``loop`` = {start, stop, times}: layers start .. stop - 1 run
``times`` times in a row with the same weights.
"""
from __future__ import annotations

import copy
import json
import os
from dataclasses import dataclass, field
from typing import Any, Mapping

from tensorline_amd.config.model_config import ConfigError

_LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
_RIGHT_KEYS = ("heads", "vdim", "state", "groups", "conv", "norm_groups")
_RGLRU_KEYS = ("width", "blocks", "conv")


def _positive_int(where: str, d: Mapping[str, Any], key: str) -> int:
    v = d.get(key) if isinstance(d, Mapping) else None
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


def _need(where: str, d: Any, keys) -> None:
    if not isinstance(d, Mapping):
        raise ConfigError(f"config.json: {where} is missing")
    for key in keys:
        if key not in d:
            raise ConfigError(f"config.json: {where}.{key} is missing")


@dataclass(frozen=True)
class TumitarConfig:
    vocab_size: int
    hidden_size: int
    layers: tuple = ()                      # the entries of config.json's ``layers``, checked
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    loop: tuple[int, int, int] | None = None    # (start, stop, times)
    eos_token_id: tuple[int, ...] = ()
    max_position_embeddings: int = 1 << 30
    architecture: str = "Tumitar"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False, hash=False)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TumitarConfig":
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
            kind, mixer = layer.get("type"), layer.get("mixer")
            if kind == "parallel":
                _need(where + ".mixer", mixer, ("left", "right", "left_scale", "right_scale"))
                _need(where + ".mixer.left", mixer["left"], _LEFT_KEYS)
                _need(where + ".mixer.right", mixer["right"], _RIGHT_KEYS)
                for key in ("heads", "kv_heads", "dim", "vdim"):
                    _positive_int(where + ".mixer.left", mixer["left"], key)
                for key in _RIGHT_KEYS:
                    _positive_int(where + ".mixer.right", mixer["right"], key)
                temp = mixer["left"].get("q_temp")
                if temp is not None:
                    _need(where + ".mixer.left.q_temp", temp, ("coef", "every"))
                    _positive_int(where + ".mixer.left.q_temp", temp, "every")
            elif kind == "rglru":
                _need(where + ".mixer", mixer, _RGLRU_KEYS)
                for key in _RGLRU_KEYS:
                    _positive_int(where + ".mixer", mixer, key)
            else:
                raise ConfigError(f"config.json: {where}.type {kind!r} is unknown; known: parallel, rglru")
            mlp = layer.get("mlp")
            if mlp is not None:
                mk = mlp.get("kind")
                if mk == "dense":
                    _positive_int(where + ".mlp", mlp, "ff")
                elif mk == "moe":
                    _need(where + ".mlp.router", mlp.get("router"), ("experts", "top", "scale"))
                    _need(where + ".mlp.expert", mlp.get("expert"), ("ff",))
                    if mlp["router"]["top"] > mlp["router"]["experts"]:
                        raise ConfigError(f"config.json: {where}.mlp.router.top exceeds the number of experts")
                else:
                    raise ConfigError(f"config.json: {where}.mlp.kind {mk!r} is unknown; known: dense, moe")
            layers.append(copy.deepcopy(dict(layer)))
        loop = d.get("loop")
        loop_t = None
        if loop:
            _need("loop", loop, ("start", "stop", "times"))
            start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= start < stop <= len(layers)) or times < 1:
                raise ConfigError(f"config.json: loop {loop!r} does not fit {len(layers)} layers")
            loop_t = (start, stop, times)
        emb = d.get("embedding") or {}
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "embedding", "loop", "eos_token_id",
                 "max_position_embeddings"}
        return cls(vocab_size=vocab, hidden_size=width, layers=tuple(layers), norm_eps=float(norm["eps"]),
                   embedding_scale=float(emb.get("scale", 1.0)), loop=loop_t, eos_token_id=eos_ids,
                   max_position_embeddings=int(d.get("max_position_embeddings", 1 << 30)),
                   extra={k: v for k, v in d.items() if k not in known})

    @classmethod
    def from_json(cls, path: str | os.PathLike) -> "TumitarConfig":
        p = os.fspath(path)
        if os.path.isdir(p):
            p = os.path.join(p, "config.json")
        with open(p, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def run_order(self) -> list[tuple[int, bool]]:
        """(layer, whether the embedding output is added in front of it) for every layer run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        order = [(i, False) for i in range(start)]
        for rep in range(times):
            order += [(i, rep > 0 and i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                               "layers": copy.deepcopy(list(self.layers))}
        if self.loop is not None:
            out["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.eos_token_id:
            out["eos_token_id"] = list(self.eos_token_id)
        return out
