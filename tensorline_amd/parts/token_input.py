"""A per-layer input from the token ids, added to the residual stream at the end of a layer.

One table holds a row per token with a slice of ``dim`` columns for every layer.  For layer i, with
x the stream after the layer's feed-forward:

    e = table[token][i dim : (i + 1) dim];   g = gelu_tanh(W_gate x) * e;   y = W_proj g;
    x <- x + y / sqrt(mean(y^2) + eps) * w

(gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))); the norm is a plain RMS norm whatever
the model's norm is.)  ``forward(x, pending, ctx)`` adds ``pending`` (the feed-forward's output) into the
float32 stream first, and returns the normed y for whoever runs next to add.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter
from tensorline_amd.parts.registry import register_token_input
from tensorline_amd.parts.spec import TensorDecl


@register_token_input("gated_token_slice")
class GatedTokenSlice(Part):
    """Parameters: ``table`` (the shared table's checkpoint name), ``vocab_size``, ``dim``, ``index`` (which
    slice), ``slices`` (how many the table holds), ``eps``.  Tensors under the prefix: gate, proj, norm."""

    def __init__(self, hidden_size, prefix, dtype, device, table: str, vocab_size: int, dim: int, index: int, slices: int,
                 eps: float):
        super().__init__(hidden_size, prefix, dtype, device)
        self.table_name, self.vocab_size = table, int(vocab_size)
        self.dim, self.index, self.slices, self.eps = int(dim), int(index), int(slices), float(eps)
        self.gate = Linear(prefix + "gate", hidden_size, self.dim, False, weight_name=prefix + "gate")
        self.proj = Linear(prefix + "proj", self.dim, hidden_size, False, weight_name=prefix + "proj")
        self.table = self.norm_w = None

    def tensors(self):
        return {**self.gate.tensors(), **self.proj.tensors(),
                self.prefix + "norm": TensorDecl((self.hidden_size,), "one_plus_normal", 0.1, "float32"),
                self.table_name: TensorDecl((self.vocab_size, self.slices * self.dim), "normal", 0.5, "compute")}

    def load(self, get: TensorGetter) -> None:
        self.gate.load(get)
        self.proj.load(get)
        self.gate.prepare()
        self.proj.prepare()
        self.norm_w = get(self.prefix + "norm")
        self.table = get(self.table_name)

    def weight_tensors(self):
        return self.gate.tensors_kept() + self.proj.tensors_kept() + [self.norm_w, self.table]

    def forward(self, x: torch.Tensor, pending: torch.Tensor | None, ctx) -> torch.Tensor:
        xa = kernels.add_cast(x, pending, self.dtype)
        g = kernels.gelu_token_gate(self.gate(xa, out_dtype=torch.float32), self.table, ctx.ids, self.index * self.dim)
        y = self.proj(g, out_dtype=torch.float32)
        return kernels.add_rmsnorm(y, None, self.norm_w, self.eps, torch.float32)
