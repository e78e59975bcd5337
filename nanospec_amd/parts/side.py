"""A per-layer input chosen by the token ("token_side"): with e = table[token][offset : offset + dim],
    y = W_proj (gelu_tanh(W_gate x) * e)
where x is what the sublayer reads (the stream itself in the design that has it).  The table [vocab, table_dim] is one
tensor that all layers share; each layer keeps only its own columns on the device.  It is a part of the "ffn" role that
also reads the step's token ids (``ctx.token_ids``)."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry


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

    def load(self, get, dtype, device) -> None:
        s = self.spec
        self.table = get(s.table_name)[:, s.offset : s.offset + s.dim].to(device=device, dtype=dtype).contiguous()
        self.gate = get(self.prefix + s.names[0]).to(device=device, dtype=dtype).contiguous()
        self.proj = get(self.prefix + s.names[1]).to(device=device, dtype=dtype).contiguous()

    def forward(self, ctx, x, out: torch.Tensor | None = None):
        n = x.shape[0]
        return ops.token_side(x, ctx.token_ids, self.table, self.gate, self.proj,
                              out if out is not None else ctx.arena.take((n, self.spec.hidden), x.dtype))


registry.register("ffn", "token_side", TokenSide)
