"""A per-layer input chosen by the token ("token_side"): with e = table[token][offset : offset + dim],
    y = W_proj (gelu_tanh(W_gate x) * e)
where x is what the sublayer reads (the stream itself in the design that has it).  The table [vocab, table_dim] is one
tensor that all layers share; each layer keeps only its own columns on the device.  It is a part of the "ffn" role that
also reads the step's token ids (``ctx.token_ids``).  The two products are the framework's (they stream the matrices for
few rows and use the library for many); one small kernel between them applies the activation and the table's row."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight


class TokenSide:
    graph_safe = True

    def __init__(self, spec, prefix: str) -> None:
        if spec.dim <= 0 or spec.offset < 0 or spec.offset + spec.dim > spec.table_dim:
            raise ValueError(f"columns [{spec.offset}, {spec.offset + spec.dim}) of a table of {spec.table_dim}")
        self.spec, self.prefix = spec, prefix

    def wanted(self) -> dict:
        s = self.spec
        return {s.table_name: ((s.vocab, s.table_dim), "embedding"), self.prefix + s.names[0]: ((s.dim, s.hidden), "linear"),
                self.prefix + s.names[1]: ((s.hidden, s.dim), "linear")}

    takes_layouts = True

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        self.table = get(s.table_name)[:, s.offset : s.offset + s.dim].to(device=device, dtype=dtype).contiguous()
        self.gate = LinearWeight(get(self.prefix + s.names[0]).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)
        self.proj = LinearWeight(get(self.prefix + s.names[1]).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def forward(self, ctx, x, out: torch.Tensor | None = None):
        n, take = x.shape[0], ctx.arena.take
        g = self.gate(x, out=take((n, self.gate.n), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        act = ops.gelu_gather_mul(g[:, : self.spec.dim], ctx.token_ids, self.table, take((n, self.spec.dim), x.dtype))
        return self.proj(act, out=out if out is not None else take((n, self.spec.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("ffn", "token_side", TokenSide)
