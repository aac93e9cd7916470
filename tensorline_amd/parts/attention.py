"""Grouped-query attention over the paged cache.

One step: fused q/k/v projection (with bias), position encoding of queries and keys, write of the
new keys and values into the cache, causal attention of every token of the step over the cached
keys of its sequence, output projection (reference order: tensorline/paged.py:247-275).  All
attention, for a whole prompt, a portion of one or a single decoded token, reads the cache; the
step's own keys are in it before attention runs (paged.py:252-253).
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import build_part, register_mixer
from tensorline_amd.parts.spec import CacheNeed, PartSpec, TensorDecl, keys_and_values


@register_mixer("attention")
class PagedAttention(Part):
    """Parameters: head counts and size, whether q/k/v carry a bias, the position encoding, an
    optional ``window`` (a token sees only the last ``window`` keys, itself included), an optional
    ``scale`` (default head_dim^-1/2, tests/test_paged_attn.py:36), and ``kv_proj`` False for a
    layer that only reads keys and values another layer cached."""

    def __init__(self, hidden_size, prefix, dtype, device, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: PartSpec, qkv_bias: bool = True, out_bias: bool = False, window: int = 0,
                 scale: float | None = None, kv_proj: bool = True):
        super().__init__(hidden_size, prefix, dtype, device)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.num_heads, self.num_kv_heads, self.head_dim = int(num_heads), int(num_kv_heads), int(head_dim)
        # The kernels take head sizes in steps of 16.  Another size is served at the next step: the
        # projections get rows of zeros at the end of every head when they are loaded (and the output
        # projection columns of zeros), so the added dimensions of queries, keys and values are zero,
        # add nothing to a score and come out of the weighted sum as zeros that meet zero columns.
        self.kernel_dim = -(-self.head_dim // 16) * 16
        if self.head_dim <= 0 or not kernels.attention_takes_head_dim(self.kernel_dim):
            raise ValueError(f"{prefix}: a head size of {self.head_dim} is not served: the attention kernels take "
                             "up to 256")
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.kv_proj = bool(kv_proj)
        q_size, kv_size = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        self._projs = [Linear(prefix + "q_proj", hidden_size, q_size, qkv_bias)]
        if self.kv_proj:
            self._projs += [Linear(prefix + "k_proj", hidden_size, kv_size, qkv_bias),
                            Linear(prefix + "v_proj", hidden_size, kv_size, qkv_bias)]
        self.qkv: Linear | None = None
        self.o_proj = Linear(prefix + "o_proj", q_size, hidden_size, out_bias)
        self.position = build_part("position", position, head_dim=self.head_dim, device=device)

    # ---- weights -----------------------------------------------------------------------
    def tensors(self):
        out = {}
        for p in self._projs + [self.o_proj]:
            out.update(p.tensors())
        return out

    def _pad_heads(self, lin: Linear, heads: int, rows: bool) -> None:
        """Widen every head of a loaded projection from head_dim to kernel_dim with zeros: rows (and
        bias entries) of a q/k/v projection, columns of the output projection."""
        d, dp = self.head_dim, self.kernel_dim
        w = lin.weight
        if rows:
            wide = w.new_zeros(heads, dp, w.shape[1])
            wide[:, :d] = w.view(heads, d, w.shape[1])
            lin.weight, lin.out_features = wide.view(heads * dp, w.shape[1]), heads * dp
            if lin.bias is not None:
                b = lin.bias.new_zeros(heads, dp)
                b[:, :d] = lin.bias.view(heads, d)
                lin.bias = b.view(-1)
        else:
            wide = w.new_zeros(w.shape[0], heads, dp)
            wide[:, :, :d] = w.view(w.shape[0], heads, d)
            lin.weight, lin.in_features = wide.view(w.shape[0], heads * dp), heads * dp

    def load(self, get: TensorGetter) -> None:
        for p in self._projs:
            p.load(get)
        self.o_proj.load(get)
        if self.kernel_dim != self.head_dim:
            for i, p in enumerate(self._projs):
                self._pad_heads(p, self.num_heads if i == 0 else self.num_kv_heads, rows=True)
            self._pad_heads(self.o_proj, self.num_heads, rows=False)
        self.qkv = fuse_linears(self.prefix + "qkv_proj", self._projs)
        for p in self._projs:          # the fused copy is the one that is kept
            p.weight = p.bias = None
        self.o_proj.prepare()

    def weight_tensors(self):
        return self.qkv.tensors_kept() + self.o_proj.tensors_kept()

    # ---- what it keeps -------------------------------------------------------------------
    def cache_need(self) -> CacheNeed | None:
        return keys_and_values(self.num_kv_heads, self.kernel_dim, self.window)

    def state_need(self):
        return None

    # ---- one step ------------------------------------------------------------------------
    def library_products(self):
        return [(self.qkv.weight, self.dtype), (self.o_proj.weight, torch.float32)]

    @property
    def defers_norm(self) -> bool:
        return self.qkv.shuffled is not None and self.o_proj.shuffled is not None

    @staticmethod
    def step_vectors(facts) -> dict:
        """The one-token sequences of a step that also holds prompt portions, for the launch of their
        own that long contexts give them (``kernels.paged_attention``)."""
        singles = kernels.one_token_sequences(facts)
        return {"attention.single_seqs": singles} if singles else {}

    def forward(self, h, ctx, cache, sink=None):
        nkv_local = self.num_kv_heads if self.kv_proj else 0
        write = cache.write and self.kv_proj
        d = self.kernel_dim
        keys, values = cache.planes["k"], cache.planes["v"]
        qkv = None
        fused = getattr(self.position, "project_rotate_store", None)
        if fused is not None and write:
            qkv = fused(h, self.qkv, ctx.pos, self.num_heads, nkv_local, d, keys, values, cache.slots)
        if qkv is None:
            if self.qkv.bias is not None and getattr(self.position, "adds_bias", False):
                qkv = self.qkv(h, with_bias=False)           # the bias rides on the position encoding's pass
                self.position.apply_and_store(qkv, ctx.pos, self.num_heads, nkv_local, d,
                                              keys if write else None, values if write else None,
                                              cache.slots if write else None, bias=self.qkv.bias)
            else:
                qkv = self.qkv(h)
                self.position.apply_and_store(qkv, ctx.pos, self.num_heads, nkv_local, d,
                                              keys if write else None, values if write else None,
                                              cache.slots if write else None)
        o = kernels.paged_attention(qkv, keys, values, cache.tables, ctx.seq_of_token, ctx.pos,
                                    self.num_heads, self.num_kv_heads, d, self.scale,
                                    window=self.window, q_start=ctx.q_start, ctx_start=ctx.ctx_start,
                                    plan=ctx.facts, single_seqs=ctx.extra.get("attention.single_seqs"))
        return self.o_proj(o, out_dtype=torch.float32, sink=sink)


@register_mixer("normed_attention")
class NormedAttention(Part):
    """Grouped-query attention without rotation over the same paged cache, for designs that let
    positions in by other ways.  Parameters: ``heads``, ``kv_heads``, ``dim`` (query/key size per
    head), ``vdim`` (value size per head), ``scale`` of the scores, ``eps``;

    * ``qk_norm``: queries and keys are each RMS-normed over their whole projection, all heads at
      once, before they are split into heads (weights ``q.norm`` [heads*dim], ``k.norm``
      [kv_heads*dim]);
    * ``q_temp`` = {coef, every} or None: the query at position p is multiplied by
      ``1 + coef * ln(floor((p + 1) / every) + 1)``;
    * ``sink``: one is added to the softmax's denominator, ``p_j = exp(s_j) / (1 + sum exp(s))``: a key
      of score 0 that has no value;
    * ``window``: a token sees the last ``window`` keys only (0: all).

    Tensors under the prefix: q, k, v (with ``.b`` where ``bias``), q.norm, k.norm, o.  Projection
    sums, the norms and the factor are float32; what attention reads (queries, cached keys and
    values) is in the engine's dtype.  Keys and values share one head size in the cache,
    ``ceil16(max(dim, vdim))``: the shorter of the two is padded with zeros, which add nothing to a
    score and come out of the weighted sum as zeros that meet zero columns of ``o``."""

    def __init__(self, hidden_size, prefix, dtype, device, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 eps: float = 1e-6, bias: bool = True, qk_norm: bool = True, q_temp: dict | None = None, sink: bool = False,
                 window: int = 0):
        super().__init__(hidden_size, prefix, dtype, device)
        self.heads, self.kv_heads, self.dim, self.vdim = int(heads), int(kv_heads), int(dim), int(vdim)
        if min(self.heads, self.kv_heads, self.dim, self.vdim) <= 0 or self.heads % self.kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads of {dim} and {kv_heads} key/value heads of {vdim} do not fit")
        self.kernel_dim = -(-max(self.dim, self.vdim) // 16) * 16
        if not kernels.attention_takes_head_dim(self.kernel_dim):
            raise ValueError(f"{prefix}: a head size of {max(self.dim, self.vdim)} is not served: the attention kernels "
                             "take up to 256")
        self.scale, self.eps, self.window = float(scale), float(eps), int(window or 0)
        if self.scale <= 0.0:
            raise ValueError(f"{prefix}: the score scale {scale} must be positive")
        self.qk_norm, self.sink = bool(qk_norm), bool(sink)
        self.temp_coef = float(q_temp["coef"]) if q_temp else 0.0
        self.temp_every = int(q_temp["every"]) if q_temp else 0
        if q_temp and self.temp_every <= 0:
            raise ValueError(f"{prefix}: q_temp.every must be positive")
        mk = lambda s, n_in, n_out, b: Linear(prefix + s, n_in, n_out, b, weight_name=prefix + s, bias_name=prefix + s + ".b")
        self._projs = [mk("q", hidden_size, self.heads * self.dim, bias), mk("k", hidden_size, self.kv_heads * self.dim, bias),
                       mk("v", hidden_size, self.kv_heads * self.vdim, bias)]
        self.qkv: Linear | None = None
        self.o_proj = mk("o", self.heads * self.vdim, hidden_size, False)
        self.q_norm = self.k_norm = None

    def tensors(self):
        out = {}
        for p in self._projs + [self.o_proj]:
            out.update(p.tensors())
        if self.qk_norm:
            out[self.prefix + "q.norm"] = TensorDecl((self.heads * self.dim,), "one_plus_normal", 0.1, "float32")
            out[self.prefix + "k.norm"] = TensorDecl((self.kv_heads * self.dim,), "one_plus_normal", 0.1, "float32")
        return out

    def load(self, get: TensorGetter) -> None:
        for p in self._projs + [self.o_proj]:
            p.load(get)
        if self.kernel_dim != self.vdim:          # attention leaves kernel_dim columns per head: zero columns for the padding
            w, D = self.o_proj.weight, self.kernel_dim
            wide = w.new_zeros(w.shape[0], self.heads, D)
            wide[:, :, :self.vdim] = w.view(w.shape[0], self.heads, self.vdim)
            self.o_proj.weight, self.o_proj.in_features = wide.view(w.shape[0], self.heads * D), self.heads * D
        self.qkv = fuse_linears(self.prefix + "qkv", self._projs)
        for p in self._projs:
            p.weight = p.bias = None
        self.o_proj.prepare()
        if self.qk_norm:
            self.q_norm, self.k_norm = get(self.prefix + "q.norm"), get(self.prefix + "k.norm")

    def weight_tensors(self):
        return self.qkv.tensors_kept() + self.o_proj.tensors_kept() + [t for t in (self.q_norm, self.k_norm) if t is not None]

    def library_products(self):
        return [(lin.weight, torch.float32) for lin in (self.qkv, self.o_proj) if lin.weight is not None]

    def cache_need(self) -> CacheNeed | None:
        return keys_and_values(self.kv_heads, self.kernel_dim, self.window)

    def state_need(self):
        return None

    step_vectors = staticmethod(PagedAttention.step_vectors)

    def input_linear(self) -> Linear:
        """The product this mixer applies to its input first (float32 out).  A part that runs it beside
        another mixer may fuse the two products and hand each its columns (``forward_projected``)."""
        return self.qkv

    def forward(self, h, ctx, cache):
        return self.forward_projected(self.qkv(h, out_dtype=torch.float32), ctx, cache)

    def forward_projected(self, proj, ctx, cache):
        """``proj`` float32 [T, q | k | v] with the biases added; rows may be strided."""
        keys, values = cache.planes["k"], cache.planes["v"]
        q = kernels.qk_norm_store(proj, ctx.pos, self.q_norm, self.k_norm, self.eps, self.temp_coef, self.temp_every,
                                  keys, values, cache.slots, self.heads, self.kv_heads, self.dim, self.vdim, self.dtype)
        o = kernels.paged_attention(q, keys, values, cache.tables, ctx.seq_of_token, ctx.pos, self.heads, self.kv_heads,
                                    self.kernel_dim, self.scale, window=self.window, q_start=ctx.q_start,
                                    ctx_start=ctx.ctx_start, plan=ctx.facts,
                                    single_seqs=ctx.extra.get("attention.single_seqs"), sink=self.sink)
        return self.o_proj(o, out_dtype=torch.float32)
