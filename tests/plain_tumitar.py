"""The plain implementation of the Tumitar decoder: slow, whole-sequence, one function per mechanism.

No cache, no batching, no kernels, no code shared with ``tensorline_amd``.  ``w`` is a dict of
tensors by checkpoint name, ``cfg`` the raw dictionary of config.json.  Everything runs in the dtype
of the tensors given (float32, or float64 for error budgets).  The recurrent mixers are written as
the token-by-token loops of their definitions and take / return their state, so a test can also
drive them one token at a time.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


# ---- small pieces ------------------------------------------------------------------------------
def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_divide(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_divide(x, eps) * weight


def causal_conv(x, taps, bias, before=None):
    """x [T, C]; taps [C, K], the last column is the current token's; ``before`` [K - 1, C] are the
    inputs ahead of x (zeros at a sequence's start).  Returns (out [T, C], the last K - 1 inputs)."""
    T, C = x.shape
    K = taps.shape[1]
    if before is None:
        before = x.new_zeros(K - 1, C)
    full = torch.cat((before, x), dim=0)                      # row t + K - 1 is x[t]
    out = bias.expand(T, C).clone()
    for j in range(K):
        out = out + full[j:j + T] * taps[:, j]
    return out, full[full.shape[0] - (K - 1):]


# ---- mixers --------------------------------------------------------------------------------------
def query_temperature(positions, coef, every):
    """1 + coef ln(floor((p + 1) / every) + 1) per position."""
    steps = torch.div(positions + 1, int(every), rounding_mode="floor")
    return 1.0 + float(coef) * torch.log(steps.to(torch.float64) + 1.0)


def sink_attention(h, w, p, m: dict, eps: float, positions=None):
    """h [T, width] of one sequence from its first token.  Grouped heads, biases, one RMS norm over
    all query rows and one over all key rows, a query factor that grows with the position, no
    rotation, and a softmax whose denominator has one added."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T) if positions is None else positions
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(k, w[p + "k.norm"], eps).view(T, G, d)
    if m.get("q_temp"):
        q = q * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"]).to(q.dtype)[:, None]
    q = q.view(T, H, d)
    out = h.new_zeros(T, H, dv)
    per = H // G
    for head in range(H):
        g = head // per
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])                       # [T, T]
        s = s.masked_fill(pos[None, :] > pos[:, None], float("-inf"))
        top = s.max(dim=1, keepdim=True).values.clamp_min(0.0)                # the sink's score is 0
        e = torch.exp(s - top)
        weights = e / (torch.exp(-top) + e.sum(dim=1, keepdim=True))
        out[:, head] = weights @ v[:, g]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def ssd_mixer(h, w, p, m: dict, eps: float, state=None):
    """Mamba-2's mixer.  ``state`` = (S [heads, N, vdim], the convolution's last inputs) or None."""
    T = h.shape[0]
    Hh, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = Hh * P
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    S, before = state if state is not None else (h.new_zeros(Hh, N, P), None)
    xbc, tail = causal_conv(xbc, w[p + "conv"], w[p + "conv.b"], before)
    xbc = F.silu(xbc)
    x = xbc[:, :inner].view(T, Hh, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = F.softplus(dt + w[p + "dt_bias"])                                    # [T, heads]
    rate = torch.exp(w[p + "A_log"])
    per = Hh // G
    y = h.new_zeros(T, Hh, P)
    S = S.clone()
    for t in range(T):
        for head in range(Hh):
            g = head // per
            S[head] = torch.exp(-rate[head] * dt[t, head]) * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S[head].T @ C[t, g] + w[p + "D"][head] * x[t, head]
    y = y.reshape(T, inner) * F.silu(z)
    parts = int(m["norm_groups"])
    y = rms_divide(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T, (S, tail)


def parallel_mixer(h, w, p, m: dict, eps: float, state=None, positions=None):
    left = sink_attention(h, w, p + "left.", m["left"], eps, positions)
    right, state = ssd_mixer(h, w, p + "right.", m["right"], eps, state)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right, state


def rglru_mixer(h, w, p, m: dict, state=None):
    """Griffin's recurrent block.  ``state`` = (S [width], the convolution's last inputs) or None."""
    T = h.shape[0]
    width, blocks = int(m["width"]), int(m["blocks"])
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = h @ w[p + "x"].T + w[p + "x.b"]
    S, before = state if state is not None else (h.new_zeros(width), None)
    u, tail = causal_conv(u, w[p + "conv"], w[p + "conv.b"], before)
    ub = u.view(T, blocks, width // blocks)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(T, width)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(T, width)
    log_a = -8.0 * r * F.softplus(w[p + "lam"])
    a = torch.exp(log_a)
    out = h.new_zeros(T, width)
    S = S.clone()
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[p + "o"].T, (S, tail)


# ---- feed-forwards -------------------------------------------------------------------------------
def dense_ff(h, w, p):
    return torch.relu(h @ w[p + "up"].T).pow(2) @ w[p + "down"].T


def router_choice(h, w, p, mlp: dict):
    """(chosen experts [T, top], their weights [T, top], all scores [T, experts])."""
    scores = torch.sigmoid(h @ w[p + "router"].T)
    top = scores.topk(int(mlp["router"]["top"]), dim=-1)
    return top.indices, top.values * float(mlp["router"]["scale"]), scores


def expert_ff(h, w, p):
    return (F.silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def routed_ff(h, w, p, mlp: dict, margins=None, forced=None):
    """``margins``: a list that gets, per call and token, how far the last chosen expert's logit lies above
    the best one left out, in units of the root mean square of the token's logits (infinite where every
    expert is chosen).  ``forced``: an iterator of [T, top] expert ids, one per call, to use in place of the router's
    own choice (weights are still those experts' own scores); ``margins`` then gets the regret instead: how
    far the worst forced expert's logit lies under the last one the router would have chosen, in the same
    units (0 where the sets agree)."""
    ids, weights, scores = router_choice(h, w, p, mlp)
    top = int(mlp["router"]["top"])
    z = h @ w[p + "router"].T
    ranked = z.sort(dim=-1, descending=True).values
    spread = z.pow(2).mean(dim=-1).sqrt()                     # the size of the token's logits (their root mean square)
    if forced is not None:
        ids = next(forced).long()
        weights = scores.gather(1, ids) * float(mlp["router"]["scale"])
        if margins is not None:
            margins.append((ranked[:, top - 1] - z.gather(1, ids).min(dim=-1).values).clamp_min(0.0) / spread)
    elif margins is not None:
        margins.append((ranked[:, top - 1] - ranked[:, top]) / spread if top < ranked.shape[1]
                       else torch.full((h.shape[0],), float("inf")))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(ids[t].tolist(), weights[t]):
            out[t] = out[t] + g * expert_ff(h[t:t + 1], w, f"{p}e{e}.")[0]
    return out


def feed_forward(h, w, p, mlp: dict, margins=None, forced=None):
    return dense_ff(h, w, p) if mlp["kind"] == "dense" else routed_ff(h, w, p, mlp, margins, forced)


# ---- the model -----------------------------------------------------------------------------------
def run_order(cfg: dict) -> list[tuple[int, bool]]:
    """(layer, whether the embedding output is added in front of it) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for rep in range(times):
        order += [(i, rep > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def layer_forward(x, w, cfg: dict, i: int, state=None, positions=None, margins=None, forced=None):
    layer, eps, p = cfg["layers"][i], float(cfg["norm"]["eps"]), f"l{i}."
    h = rms_norm(x, w[p + "norm1"], eps)
    if layer["type"] == "parallel":
        y, state = parallel_mixer(h, w, p + "mix.", layer["mixer"], eps, state, positions)
    else:
        y, state = rglru_mixer(h, w, p + "mix.", layer["mixer"], state)
    x = x + y
    if layer.get("mlp") is not None:
        x = x + feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"], margins, forced)
    return x, state


def forward(tokens, w, cfg: dict, return_layers: bool = False, margins=None, forced=None):
    """Logits [T, vocab] of one sequence from its first token; with ``return_layers`` also the
    residual stream after every layer run.  ``margins``, ``forced``: see ``routed_ff``."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x0 = w["embed"][ids] * float(cfg["embedding"]["scale"])
    x, seen = x0, []
    for i, again in run_order(cfg):
        if again:
            x = x + x0
        x, _ = layer_forward(x, w, cfg, i, margins=margins, forced=forced)
        seen.append(x)
    logits = rms_norm(x, w["final.norm"], float(cfg["norm"]["eps"])) @ w["embed"].T
    return (logits, seen) if return_layers else logits
