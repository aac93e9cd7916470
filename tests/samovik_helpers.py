"""Shared by the Samovik tests: small configurations (none of them a real model's sizes), random
weights for the framework and for the plain implementation alike, and a runner of step lists."""
from __future__ import annotations

import copy

import numpy as np
import torch

from tensorline_amd.config.samovik_config import SamovikConfig


def _moe(experts, top, ff, limit, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}, "shared": shared}


def _latent(heads, dim, rot_dim, vdim, rank, base=5000.0, scaling=None, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
            "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
            "rot": {"base": base, "dims": rot_dim, "scaling": scaling}}


# all three mixers, two latent layers of different sizes (two cache groups), a layer without
# feed-forward, YaRN on one latent layer only
CFG_A = {"architecture": "Samovik", "vocab": 320, "width": 96, "norm": {"eps": 1e-5}, "token_side": {"dim": 8}, "layers": [
    {"type": "wkv", "mixer": {"heads": 3, "dim": 16, "decay_rank": 8}, "mlp": _moe(6, 2, 40, 3.0, {"ff": 56, "limit": 1.5})},
    {"type": "latent_attention", "mixer": _latent(3, 24, 8, 40, 48, scaling={"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}),
     "mlp": _moe(6, 2, 40, 3.0, {"ff": 56, "limit": 1.5})},
    {"type": "lightning", "mixer": {"heads": 2, "dim": 24, "vdim": 48, "decay": [0.9, 0.995]}, "mlp": None},
    {"type": "latent_attention", "mixer": _latent(2, 16, 16, 24, 64, base=300.0), "mlp": _moe(4, 3, 24, 7.0)},
]}
# sizes that are no multiple of 8, one head, as many choices as experts, one choice, no token input
CFG_B = {"architecture": "Samovik", "vocab": 131, "width": 72, "norm": {"eps": 1e-6}, "layers": [
    {"type": "latent_attention", "mixer": _latent(1, 20, 4, 12, 28, base=50.0), "mlp": _moe(3, 3, 20, 2.0)},
    {"type": "wkv", "mixer": {"heads": 2, "dim": 40, "decay_rank": 5}, "mlp": _moe(5, 1, 36, 1.0, {"ff": 12, "limit": 4.0})},
    {"type": "lightning", "mixer": {"heads": 3, "dim": 12, "vdim": 70, "decay": [0.5, 0.97, 1.0]}, "mlp": _moe(1, 1, 16, 2.0)},
]}
# no layer with a cache of tokens at all
CFG_C = {"architecture": "Samovik", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "token_side": {"dim": 4}, "layers": [
    {"type": "lightning", "mixer": {"heads": 2, "dim": 72, "vdim": 16, "decay": [0.8, 0.999]}, "mlp": _moe(4, 2, 32, 2.0)},
    {"type": "wkv", "mixer": {"heads": 1, "dim": 136, "decay_rank": 4}, "mlp": None},
]}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def one_layer(kind: str, mixer: dict, mlp=None, width: int = 64, vocab: int = 50, side: int = 0) -> dict:
    cfg = {"architecture": "Samovik", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
           "layers": [{"type": kind, "mixer": mixer, "mlp": mlp}]}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def typed(cfg: dict) -> SamovikConfig:
    return SamovikConfig.from_dict(copy.deepcopy(cfg))


def build(cfg: dict, dtype: str, seed: int = 0, device="cuda:0", edit=None):
    """(framework model, plain weights by name in float32).  Both hold the same bfloat16-rounded
    values; ``edit(weights)`` may change them first (the model is then loaded from the edited ones)."""
    from tensorline_amd.config.registry import get_architecture
    from tensorline_amd.engine.loading import TORCH_DTYPE
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor
    config = typed(cfg)
    model = DecoderModel(get_architecture("Samovik").build_spec(config), TORCH_DTYPE[dtype], device)
    w = {name: random_tensor(name, decl, seed, "cpu") for name, decl in model.tensor_decls().items()}
    if edit is not None:
        edit(w)
        for name in w:
            w[name] = w[name].to(torch.bfloat16).to(torch.float32)
    load_from_getter(model, lambda name, decl: w[name], device)
    return model, w


def run_steps(model, steps, page_size: int = 16, max_tokens: int = 512, max_requests: int = 4, graphs: bool = False,
              session=None) -> dict:
    """Run a list of {"entries": [{"id", "tokens", "want"}], "end": []}; returns id -> {position: logits row}."""
    from tensorline_amd.engine.replay import TraceSession
    s = session or TraceSession(model, max_tokens, page_size=page_size, max_requests=max_requests, graphs=graphs)
    got: dict = {}
    at: dict = {}
    for st in steps:
        logits = s.step(st["entries"], st.get("end", []))
        row = 0
        for e in st["entries"]:
            base = at.get(e["id"], 0)
            for wpos in e["want"]:
                got.setdefault(e["id"], {})[base + wpos] = logits[row]
                row += 1
            at[e["id"]] = base + len(e["tokens"])
        for rid in st.get("end", []):
            at.pop(rid, None)
    return got


def rel_error(got: np.ndarray, want: np.ndarray) -> float:
    """Root mean square of the difference (mean taken off) over that of the expected row."""
    d = np.asarray(got, np.float64) - np.asarray(want, np.float64)
    d = d - d.mean(-1, keepdims=True)
    w = np.asarray(want, np.float64)
    w = w - w.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / max(np.sqrt((w ** 2).mean()), 1e-30))


LIMIT = {"float32": 2e-5, "bfloat16": 4e-2}
