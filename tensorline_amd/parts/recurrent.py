"""Mixers that keep a matrix state per head and request instead of a cache of tokens.

Both run on one kernel (``kernels.linear_recurrence``): the state S [heads, key dim, value dim]
lives in float32 in the request's state slot, starts at zero, and is carried from token to token
and from step to step; a prompt portion is walked token by token in the order of the sequence.

``lightning_attention``: linear attention with a fixed decay per head.  With q = silu(W_q h), k =
silu(W_k h), v = silu(W_v h):  S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  the heads'
outputs side by side are RMS-normed as one vector, multiplied by sigmoid(W_g h) and projected.

``wkv``: time mixing in the manner of RWKV (Peng et al., "RWKV: Reinventing RNNs for the Transformer
Era", and its later versions with a data-dependent decay).  Each of r, k, v, g, w reads its own mix of
the token's input and the previous token's, h + (h' - h) mu_s.  The decay is per token and key
channel, w_t = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0));  o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,  S_t =
diag(w_t) S_(t-1) + k_t v_t^T.  Each head's output is divided by its own root mean square, then times
a weight and the gate silu(W_g mix_g), then projected.  The previous token's input is part of the
state: it sits behind S in the request's slot.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_mixer
from tensorline_amd.parts.spec import StateNeed, TensorDecl


def _check_key_dim(prefix: str, dk: int) -> None:
    if dk <= 0 or dk > 256:
        raise ValueError(f"{prefix}: a key size of {dk} per head is not served: the recurrence kernel takes up to 256")


@register_mixer("lightning_attention")
class LightningAttention(Part):
    """Parameters: ``heads``, ``dim`` (query/key size per head), ``vdim``, ``decay`` (one per head),
    ``eps``.  Tensors under the prefix: q, k, v, g, o, norm."""

    def __init__(self, hidden_size, prefix, dtype, device, heads: int, dim: int, vdim: int, decay, eps: float):
        super().__init__(hidden_size, prefix, dtype, device)
        self.heads, self.dim, self.vdim, self.eps = int(heads), int(dim), int(vdim), float(eps)
        _check_key_dim(prefix, self.dim)
        if len(decay) != self.heads:
            raise ValueError(f"{prefix}: {len(decay)} decays for {self.heads} heads")
        self.decay = torch.tensor([float(d) for d in decay], dtype=torch.float32, device=device)
        H = self.heads
        mk = lambda s, n_out: Linear(prefix + s, hidden_size, n_out, False, weight_name=prefix + s)
        self._parts = [mk("q", H * self.dim), mk("k", H * self.dim), mk("v", H * self.vdim), mk("g", H * self.vdim)]
        self.proj: Linear | None = None
        self.o_proj = Linear(prefix + "o", H * self.vdim, hidden_size, False, weight_name=prefix + "o")
        self.norm_w = None

    def tensors(self):
        out = {}
        for p in self._parts + [self.o_proj]:
            out.update(p.tensors())
        out[self.prefix + "norm"] = TensorDecl((self.heads * self.vdim,), "one_plus_normal", 0.1, "float32")
        return out

    def load(self, get: TensorGetter) -> None:
        for p in self._parts + [self.o_proj]:
            p.load(get)
        self.proj = fuse_linears(self.prefix + "qkvg", self._parts)
        for p in self._parts:
            p.weight = None
        self.o_proj.prepare()
        self.norm_w = get(self.prefix + "norm")

    def weight_tensors(self):
        return self.proj.tensors_kept() + self.o_proj.tensors_kept() + [self.norm_w]

    def library_products(self):
        return [(self.proj.weight, torch.float32), (self.o_proj.weight, torch.float32)]

    def cache_need(self):
        return None

    def state_need(self):
        return StateNeed((self.heads * self.dim * self.vdim,), "float32")

    def forward(self, h, ctx, cache):
        H, dk, dv = self.heads, self.dim, self.vdim
        proj = self.proj(h, out_dtype=torch.float32)
        q, k = proj[:, :H * dk], proj[:, H * dk:2 * H * dk]
        v, g = proj[:, 2 * H * dk:2 * H * dk + H * dv], proj[:, 2 * H * dk + H * dv:]
        o = kernels.linear_recurrence(q, k, v, ctx, cache.state, H, dk, dv, decay=self.decay, silu_inputs=True)
        y = kernels.gated_group_norm(o, self.norm_w, g, H * dv, self.eps, "sigmoid", self.dtype)
        return self.o_proj(y, out_dtype=torch.float32)


@register_mixer("wkv")
class WKV(Part):
    """Parameters: ``heads``, ``dim`` (key and value size per head), ``eps``.  Tensors under the prefix:
    mu.r, mu.k, mu.v, mu.g, mu.w, r, k, v, g, w1, w2, w0, u, norm, o; the width of w1 / w2 (the
    decay's low-rank bottleneck) is read from ``decay_rank``."""

    WAYS = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size, prefix, dtype, device, heads: int, dim: int, decay_rank: int, eps: float):
        super().__init__(hidden_size, prefix, dtype, device)
        self.heads, self.dim, self.decay_rank, self.eps = int(heads), int(dim), int(decay_rank), float(eps)
        _check_key_dim(prefix, self.dim)
        N = self.heads * self.dim
        mk = lambda s, n_in, n_out, **kw: Linear(prefix + s, n_in, n_out, False, weight_name=prefix + s, **kw)
        self.r, self.k, self.v, self.g = (mk(s, hidden_size, N) for s in "rkvg")
        self.w1 = mk("w1", hidden_size, self.decay_rank)
        self.w2 = Linear(prefix + "w2", self.decay_rank, N, True, weight_name=prefix + "w2", bias_name=prefix + "w0")
        self.o_proj = mk("o", N, hidden_size)
        self.mu = self.u = self.norm_w = None

    def _linears(self):
        return [self.r, self.k, self.v, self.g, self.w1, self.w2, self.o_proj]

    def tensors(self):
        out = {}
        for p in self._linears():
            out.update(p.tensors())
        for s in self.WAYS:
            out[self.prefix + "mu." + s] = TensorDecl((self.hidden_size,), "normal", 0.3, "float32")
        out[self.prefix + "u"] = TensorDecl((self.heads, self.dim), "normal", 0.3, "float32")
        out[self.prefix + "norm"] = TensorDecl((self.heads * self.dim,), "one_plus_normal", 0.1, "float32")
        return out

    def load(self, get: TensorGetter) -> None:
        for p in self._linears():
            p.load(get)
            p.prepare()
        self.mu = torch.stack([get(self.prefix + "mu." + s) for s in self.WAYS]).contiguous()
        self.u = get(self.prefix + "u")
        self.norm_w = get(self.prefix + "norm")

    def weight_tensors(self):
        out = [self.mu, self.u, self.norm_w]
        for p in self._linears():
            out += p.tensors_kept()
        return out

    def library_products(self):
        return [(p.weight, torch.float32) for p in (self.r, self.g, self.o_proj)]

    def cache_need(self):
        return None

    def state_need(self):
        # the matrix state of every head, then the previous token's input
        return StateNeed((self.heads * self.dim * self.dim + self.hidden_size,), "float32")

    def forward(self, h, ctx, cache):
        H, d = self.heads, self.dim
        f32 = torch.float32
        mix = kernels.token_shift(h, self.mu, ctx, cache.state, H * d * d)          # [5, T, width]: r, k, v, g, w
        r, k, v, g = (lin(mix[i], out_dtype=f32) for i, lin in enumerate((self.r, self.k, self.v, self.g)))
        wlog = self.w2(kernels.tanh_rows(self.w1(mix[4], out_dtype=f32), self.dtype), out_dtype=f32)
        o = kernels.linear_recurrence(r, k, v, ctx, cache.state, H, d, d, wlog=wlog, bonus=self.u)
        y = kernels.gated_group_norm(o, self.norm_w, g, d, self.eps, "silu", self.dtype)
        return self.o_proj(y, out_dtype=f32)
