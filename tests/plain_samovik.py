"""The plain implementation of the Samovik decoder: slow, whole-sequence, one function per mechanism.

No cache, no batching, no kernels, no code shared with ``tensorline_amd``.  ``w`` is a dict of
tensors by checkpoint name, ``cfg`` the raw dictionary of config.json.  Everything runs in the dtype
of the tensors given (float32, or float64 for error budgets).  Every recurrent mixer is written as
the token-by-token loop of its definition and takes / returns its state, so a test can also drive
it one token at a time.
"""
from __future__ import annotations

import math

import torch


# ---- small pieces ------------------------------------------------------------------------------
def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_divide(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def dynamic_tanh(x, w, name):
    """tanh(alpha x) * weight + bias; no statistics of x are taken."""
    return torch.tanh(w[name + ".alpha"] * x) * w[name] + w[name + ".b"]


# ---- rotary positions with YaRN ------------------------------------------------------------------
def yarn_frequencies(rot: dict) -> tuple[torch.Tensor, float]:
    """(frequency per pair [dims/2] in float64, factor on cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot: dict):
    """x [T, heads, d]: the first rot['dims'] dimensions of every head are turned, dimension i
    paired with i + dims/2; the rest pass."""
    dims = int(rot["dims"])
    f, m = yarn_frequencies(rot)
    ang = (positions.to(torch.float32)[:, None] * f.to(torch.float32)[None, :]).to(x.dtype)   # angles in 32-bit
    if x.dtype == torch.float64:
        ang = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = (ang.cos() * m)[:, None, :], (ang.sin() * m)[:, None, :]
    u, v, rest = x[..., :dims // 2], x[..., dims // 2:dims], x[..., dims:]
    return torch.cat((u * cos - v * sin, v * cos + u * sin, rest), dim=-1)


# ---- mixers --------------------------------------------------------------------------------------
def latent_attention(h, w, p, m: dict, eps: float, positions=None):
    """h [T, width] of one sequence from its first token.  Keys and values are expanded from the
    normed latent; one rotated key part is shared by the heads."""
    T = h.shape[0]
    H, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T) if positions is None else positions
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], pos, m["rot"])
    dkv = h @ w[p + "dkv"].T
    c = rms_divide(dkv[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate(dkv[:, None, rank:], pos, m["rot"])                       # [T, 1, r]
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * float(m["scale"])
    mask = pos[None, :] <= pos[:, None]
    scores = scores.masked_fill(~mask[None], float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v)
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].T


def lightning(h, w, p, m: dict, eps: float, state=None):
    """Linear attention with one decay per head.  ``state`` [H, dim, vdim] or None (zeros);
    returns (output, state after the last token)."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    silu = torch.nn.functional.silu
    q = silu(h @ w[p + "q"].T).view(T, H, d)
    k = silu(h @ w[p + "k"].T).view(T, H, d)
    v = silu(h @ w[p + "v"].T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, d, dv, dtype=h.dtype) if state is None else state.clone()
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t, :, :, None] * v[t, :, None, :]
        out.append(torch.einsum("hij,hi->hj", S, q[t]))
    o = torch.stack(out).reshape(T, H * dv)
    o = rms_divide(o, eps) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, S


def wkv(h, w, p, m: dict, eps: float, state=None):
    """Time mixing with a decay per token and key channel and a bonus for the current token.
    ``state`` = (S [H, dim, dim], previous token's h [width]) or None; returns (output, state)."""
    T, W = h.shape
    H, d = int(m["heads"]), int(m["dim"])
    S, prev = (torch.zeros(H, d, d, dtype=h.dtype), torch.zeros(W, dtype=h.dtype)) if state is None else (state[0].clone(), state[1])
    before = torch.cat((prev[None], h[:-1]), dim=0)
    mix = {s: h + (before - h) * w[p + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ w[p + "r"].T).view(T, H, d)
    k = (mix["k"] @ w[p + "k"].T).view(T, H, d)
    v = (mix["v"] @ w[p + "v"].T).view(T, H, d)
    gate = torch.nn.functional.silu(mix["g"] @ w[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).view(T, H, d)
    u = w[p + "u"]
    out = []
    for t in range(T):
        kv = k[t, :, :, None] * v[t, :, None, :]
        out.append(torch.einsum("hij,hi->hj", S + u[:, :, None] * kv, r[t]))
        S = decay[t, :, :, None] * S + kv
    o = rms_divide(torch.stack(out), eps).reshape(T, H * d)
    o = o * w[p + "norm"] * gate
    return o @ w[p + "o"].T, (S, h[-1])


# ---- feed-forward ----------------------------------------------------------------------------------
def clamped_expert(h, w, p, limit: float):
    g = (h @ w[p + "gate"].T).clamp(max=limit)
    u = (h @ w[p + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def routed_experts(h, w, p, mlp: dict, margins: list | None = None):
    """The ``top`` experts with the largest router logits, weighted by the softmax over those logits
    alone, plus the shared expert if there is one.  ``margins`` receives, per token, by how much the
    last chosen logit leads the first one left out, over the largest logit's size (a close call, which
    rounding can turn, shows as a small number)."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h.to(torch.float32) @ w[p + "router"].to(torch.float32).T + w[p + "router.b"].to(torch.float32)
    if h.dtype == torch.float64:
        z = h @ w[p + "router"].T + w[p + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    if margins is not None and top < E:
        nxt = torch.topk(z, top + 1, dim=-1).values[:, -1]
        margins.append((val[:, -1] - nxt) / z.abs().max(-1).values)
    weight = torch.softmax(val, dim=-1).to(h.dtype)
    out = torch.zeros_like(h)
    for e in range(E):
        hit = idx == e                                           # [T, top]
        rows = hit.any(-1)
        if rows.any():
            y = clamped_expert(h[rows], w, f"{p}e{e}.", float(mlp["expert"]["limit"]))
            out[rows] += y * (weight[rows] * hit[rows]).sum(-1, keepdim=True)
    if mlp.get("shared"):
        out = out + clamped_expert(h, w, p + "shared.", float(mlp["shared"]["limit"]))
    return out


def token_side_input(x, tokens, w, layer: int, dim: int, eps: float):
    """The per-layer token input, added to the stream after the feed-forward."""
    p = f"l{layer}.side."
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w[p + "gate"].T) * e) @ w[p + "proj"].T
    return x + rms_divide(y, eps) * w[p + "norm"]


# ---- the whole model ---------------------------------------------------------------------------------
def forward(tokens, w, cfg: dict, per_layer: list | None = None, margins: list | None = None):
    """Logits [T, vocab] of one sequence from its first token.  ``per_layer``: a list that receives
    the residual stream after every layer; ``margins``: see ``routed_experts``, one entry per routed layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(cfg["norm"]["eps"])
    side = cfg.get("token_side")
    x = w["embed"][tokens]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = dynamic_tanh(x, w, p + "norm1")
        kind = layer["type"]
        if kind == "latent_attention":
            y = latent_attention(h, w, p + "mix.", layer["mixer"], eps)
        elif kind == "lightning":
            y, _ = lightning(h, w, p + "mix.", layer["mixer"], eps)
        elif kind == "wkv":
            y, _ = wkv(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(kind)
        x = x + y
        if layer.get("mlp"):
            x = x + routed_experts(dynamic_tanh(x, w, p + "norm2"), w, p + "mlp.", layer["mlp"], margins)
        if side:
            x = token_side_input(x, tokens, w, i, int(side["dim"]), eps)
        if per_layer is not None:
            per_layer.append(x)
    return dynamic_tanh(x, w, "final.norm") @ w["head"].T
