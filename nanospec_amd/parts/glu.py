"""A dense gated feed-forward with clipped inputs ("clipped_glu"):
    g = min(W_gate h, limit);  u = clamp(W_up h, -limit, limit);  y = W_down (g sigmoid(alpha g) (u + shift))
Gate and up matrices are stacked at load time so that one product serves both; the activation is one kernel in 32-bit
(``ops.clipped_glu``, which the experts of a mixture share)."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight


class ClippedGLU:
    graph_safe = True
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        self.spec, self.prefix = spec, prefix
        self.gate_up: LinearWeight | None = None
        self.down: LinearWeight | None = None

    @property
    def _names(self):
        return tuple(self.prefix + n for n in self.spec.names)

    def wanted(self) -> dict:
        s = self.spec
        g, u, d = self._names
        ff = s.glu.intermediate
        return {g: ((ff, s.hidden), "linear"), u: ((ff, s.hidden), "linear"), d: ((s.hidden, ff), "linear")}

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        plain = layouts == "both"
        g, u, d = self._names
        gu = torch.cat([get(g), get(u)]).to(device=device, dtype=dtype).contiguous()
        self.gate_up = LinearWeight(gu, keep_plain=plain)
        self.down = LinearWeight(get(d).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def forward(self, ctx, x, out: torch.Tensor | None = None):
        s = self.spec
        n, take = x.shape[0], ctx.arena.take
        ff = s.glu.intermediate
        gu = self.gate_up(x, out=take((n, 2 * ff), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        act = ops.clipped_glu(gu, s.glu.limit, s.glu.alpha, out=take((n, ff), x.dtype), shift=s.glu.shift)
        return self.down(act, out=out if out is not None else take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("ffn", "clipped_glu", ClippedGLU)
