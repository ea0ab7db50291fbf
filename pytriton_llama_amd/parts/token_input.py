"""A per-layer input that depends on the token alone."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, place, register_part
from .linear import LINEAR_LIBRARIES, linear


@register_part("embedding", "token_table")
class TokenTable(Part):
    """A table [vocab, columns] that several parts look their tokens up in (each its own
    columns). It computes nothing itself."""

    def __init__(self, vocab_size: int, columns: int, weight_name: str = "embed"):
        self.vocab_size, self.columns = int(vocab_size), int(columns)
        self.weight_name = weight_name
        self.weight: Optional[torch.Tensor] = None

    def param_sources(self) -> List[ParamSource]:
        return [ParamSource(self.weight_name, (self.vocab_size, self.columns))]

    def load(self, tensors, dtype, device) -> None:
        self.weight = place(tensors[self.weight_name], "matrix", dtype, device)


@register_part("stream_input", "gated_token_input")
class GatedTokenInput(Part):
    """x <- x + rmsnorm(P (gelu_tanh(G x) * e)) * w on a float32 residual stream x, where e is
    the token's vector: columns [first_column, first_column + dim) of its row of a shared
    TokenTable. G [dim, hidden], P [hidden, dim], w [hidden]; the norm is an RMS norm with
    eps inside the root. ``forward(stream, x_rounded, token_ids, pre)`` updates the stream in
    place and returns pre(stream) for a Dynamic-Tanh norm ``pre`` that follows (or None)."""
    kernel_libraries = ("stream",) + LINEAR_LIBRARIES

    def __init__(self, hidden_size: int, dim: int, table: TokenTable, first_column: int, eps: float,
                 gate_name: str = "gate", proj_name: str = "proj", norm_name: str = "norm"):
        self.hidden_size, self.dim = int(hidden_size), int(dim)
        self.table, self.first_column, self.eps = table, int(first_column), float(eps)
        if self.first_column < 0 or self.first_column + self.dim > table.columns:
            raise ValueError("the token's columns lie outside the table")
        self.names = (gate_name, proj_name, norm_name)
        self.gate = self.proj = self.norm_weight = None

    def param_sources(self) -> List[ParamSource]:
        g, p, n = self.names
        return [ParamSource(g, (self.dim, self.hidden_size)), ParamSource(p, (self.hidden_size, self.dim)),
                ParamSource(n, (self.hidden_size,), "vector")]

    def load(self, tensors, dtype, device) -> None:
        g, p, n = self.names
        self.gate = place(tensors[g], "matrix", dtype, device)
        self.proj = place(tensors[p], "matrix", dtype, device)
        self.norm_weight = place(tensors[n], "vector", dtype, device)

    def forward(self, stream: torch.Tensor, x: torch.Tensor, token_ids: torch.Tensor, pre=None,
                out_dtype: Optional[torch.dtype] = None):
        """``x``: the stream in the engine's dtype (the stream itself in float32)."""
        z = linear(x, self.gate)
        g = ops.gelu_gather_mul(z, self.table.weight, token_ids, self.first_column)
        y = linear(g, self.proj)
        out, _ = ops.stream_add_rmsnorm(stream, y, self.norm_weight, self.eps, pre, out_dtype)
        return out
