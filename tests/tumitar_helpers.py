"""Shared by the Tumitar tests: small configurations (none of them a real model's sizes) and random
weights for the framework and for the plain implementation alike."""
from __future__ import annotations

import copy

import torch

from tensorline_amd.config.tumitar_config import TumitarConfig


def _left(heads, kv_heads, dim, vdim, scale=None, coef=0.3, every=16):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
            "q_temp": {"coef": coef, "every": every}}


def _right(heads, vdim, state, groups, conv=4, norm_groups=1):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _parallel(left, right, left_scale=0.7, right_scale=1.25):
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def _moe(experts, top, ff, scale=1.5):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


# both mixers, both feed-forwards and a layer without one; the first two layers run twice
CFG_A = {"architecture": "Tumitar", "vocab": 320, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.75},
         "loop": {"start": 0, "stop": 2, "times": 2}, "layers": [
    {"type": "parallel", "mixer": _parallel(_left(4, 2, 24, 40, every=7), _right(4, 16, 24, 2, conv=4, norm_groups=2)), "mlp": _dense(136)},
    {"type": "rglru", "mixer": {"width": 64, "blocks": 4, "conv": 3}, "mlp": _moe(6, 2, 40)},
    {"type": "parallel", "mixer": _parallel(_left(2, 1, 16, 16, scale=0.4, coef=-0.1, every=3), _right(2, 40, 16, 1, conv=2), 1.0, 1.0), "mlp": None},
]}
# sizes that are no multiple of 8, one group, as many choices as experts, a loop of three passes in the middle
CFG_B = {"architecture": "Tumitar", "vocab": 131, "width": 72, "norm": {"eps": 1e-6}, "embedding": {"scale": 2.0},
         "loop": {"start": 1, "stop": 2, "times": 3}, "layers": [
    {"type": "rglru", "mixer": {"width": 90, "blocks": 3, "conv": 2}, "mlp": _moe(3, 3, 20, scale=0.5)},
    {"type": "parallel", "mixer": _parallel(_left(3, 3, 20, 12, every=5), _right(3, 10, 12, 1, conv=5, norm_groups=3), 0.3, 2.0), "mlp": _dense(50)},
    {"type": "rglru", "mixer": {"width": 36, "blocks": 1, "conv": 1}, "mlp": None},
]}
# head sizes the bfloat16 matrix-core attention takes (64 and 128), no loop, one choice of five experts
CFG_C = {"architecture": "Tumitar", "vocab": 200, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "layers": [
    {"type": "parallel", "mixer": _parallel(_left(6, 1, 64, 64, every=32), _right(2, 64, 64, 2, conv=4), 0.9, 0.6), "mlp": _moe(8, 2, 16, scale=1.0)},
    {"type": "parallel", "mixer": _parallel(_left(2, 2, 128, 96, scale=0.05, every=64), _right(8, 8, 40, 4, conv=3, norm_groups=4), 1.1, 0.4), "mlp": _moe(5, 1, 48, scale=2.5)},
]}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def one_layer(kind: str, mixer: dict, mlp=None, width: int = 64, vocab: int = 50, loop=None) -> dict:
    cfg = {"architecture": "Tumitar", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
           "layers": [{"type": kind, "mixer": mixer, "mlp": mlp}]}
    if loop:
        cfg["loop"] = loop
    return cfg


def typed(cfg: dict) -> TumitarConfig:
    return TumitarConfig.from_dict(copy.deepcopy(cfg))


def build(cfg: dict, dtype: str, seed: int = 0, device="cuda:0", edit=None):
    """(framework model, plain weights by name in float32).  Both hold the same bfloat16-rounded
    values; ``edit(weights)`` may change them first (the model is then loaded from the edited ones)."""
    from tensorline_amd.config.registry import get_architecture
    from tensorline_amd.engine.loading import TORCH_DTYPE
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor
    config = typed(cfg)
    model = DecoderModel(get_architecture("Tumitar").build_spec(config), TORCH_DTYPE[dtype], device)
    w = {name: random_tensor(name, decl, seed, "cpu") for name, decl in model.tensor_decls().items()}
    if edit is not None:
        edit(w)
        for name in w:
            w[name] = w[name].to(torch.bfloat16).to(torch.float32)
    load_from_getter(model, lambda name, decl: w[name], device)
    return model, w


def run_steps_with_routes(model, steps, page_size: int = 16, max_tokens: int = 512, max_requests: int = 4, graphs: bool = False):
    """Run a list of {"entries": [{"id", "tokens", "want"}], "end": []} eagerly.  Returns (id -> {position:
    logits row}, id -> one [tokens, top] tensor of chosen experts per run of a routed feed-forward, in the
    order the runs come in a step): what the framework's routers chose, for a plain run that is told to
    choose the same (a close call that falls the other way in bfloat16 changes every later position too)."""
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.ops import kernels
    assert not graphs, "a replayed graph does not call the router's entry again"
    s = TraceSession(model, max_tokens, page_size=page_size, max_requests=max_requests)
    got, at, routes, calls = {}, {}, {}, []
    route = kernels.moe_route

    def recording(logits, top, *a, **kw):
        ids, weights = route(logits, top, *a, **kw)
        calls.append(ids)
        return ids, weights
    kernels.moe_route = recording
    try:
        for st in steps:
            calls.clear()
            logits = s.step(st["entries"], st.get("end", []))
            chosen = [c.cpu() for c in calls]
            row = tok = 0
            for e in st["entries"]:
                base, n = at.get(e["id"], 0), len(e["tokens"])
                for wpos in e["want"]:
                    got.setdefault(e["id"], {})[base + wpos] = logits[row]
                    row += 1
                mine = routes.setdefault(e["id"], [[] for _ in chosen])
                for run, c in enumerate(chosen):
                    mine[run].append(c[tok:tok + n])
                tok += n
                at[e["id"]] = base + n
            for rid in st.get("end", []):
                at.pop(rid, None)
    finally:
        kernels.moe_route = route
    return got, {rid: [torch.cat(run) for run in runs] for rid, runs in routes.items()}


def random_config(rng) -> dict:
    """A configuration drawn from ``rng`` (a ``random.Random``): one to four layers of either kind in any
    order, sizes that are and are not multiples of 8 or 16, every head grouping, one to five taps, every kind
    of feed-forward, with or without a loop."""
    def divisor(n):
        return rng.choice([d for d in range(1, n + 1) if n % d == 0])

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return _dense(rng.choice([7, 24, 50, 136, 200]))
        experts = rng.randint(1, 9)
        return _moe(experts, rng.randint(1, experts), rng.choice([8, 20, 36, 64]), scale=rng.choice([0.5, 1.0, 2.5]))

    layers = []
    for _ in range(rng.randint(1, 4)):
        if rng.random() < 0.6:
            heads = rng.choice([1, 2, 3, 4, 6, 8])
            left = _left(heads, divisor(heads), rng.choice([8, 16, 20, 24, 32, 40, 64, 128]), rng.choice([8, 12, 16, 32, 48, 64, 128]),
                         scale=rng.choice([0.05, 0.125, 0.3]), coef=rng.choice([-0.1, 0.0, 0.3]), every=rng.choice([1, 2, 5, 16, 64]))
            rh = rng.choice([1, 2, 3, 4, 6])
            right = _right(rh, rng.choice([4, 8, 10, 16, 24, 64]), rng.choice([4, 8, 12, 16, 32, 64, 100]), divisor(rh),
                           conv=rng.randint(1, 5), norm_groups=divisor(rh))
            layers.append({"type": "parallel", "mixer": _parallel(left, right, rng.choice([0.3, 0.8, 1.0]), rng.choice([0.5, 1.0, 1.7])),
                           "mlp": mlp()})
        else:
            blocks = rng.randint(1, 5)
            layers.append({"type": "rglru", "mixer": {"width": blocks * rng.choice([4, 8, 10, 16, 30]), "blocks": blocks,
                                                      "conv": rng.randint(1, 5)}, "mlp": mlp()})
    cfg = {"architecture": "Tumitar", "vocab": rng.randint(50, 400), "width": rng.choice([24, 36, 50, 64, 72, 100, 128, 200]),
           "norm": {"eps": rng.choice([1e-5, 1e-6])}, "embedding": {"scale": rng.choice([0.5, 1.0, 3.0])}, "layers": layers}
    if rng.random() < 0.6:
        start = rng.randrange(len(layers))
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return cfg
