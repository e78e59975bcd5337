"""Two mixers side by side ("parallel"): both read the same input, y = left_scale * left(h) + right_scale * right(h).

Each of the two is a mixer of any registered kind with its own tensors (under the two prefixes) and its own needs of the
cache: the pair asks for a tuple of needs and is handed a tuple of views in the same order.  The sum is formed in 32-bit
by one kernel, which also adds the last bias of a mixer that leaves it to its caller.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry


class ParallelMixer:
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        self.spec, self.prefix = spec, prefix
        self.left = registry.build("mixer", spec.left, prefix + spec.prefixes[0])
        self.right = registry.build("mixer", spec.right, prefix + spec.prefixes[1])
        self.sides = (self.left, self.right)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.sides)

    def wanted(self) -> dict:
        out = {}
        for p in self.sides:
            out.update(p.wanted())
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        for p in self.sides:
            if getattr(p, "takes_layouts", False):
                p.load(get, dtype, device, layouts)
            else:
                p.load(get, dtype, device)

    def cache_need(self):
        return tuple(p.cache_need() for p in self.sides)

    def batch_plans(self) -> list:
        return [plan for p in self.sides for plan in getattr(p, "batch_plans", list)()]

    def step_buffers(self) -> dict:
        out = {}
        for p in self.sides:
            out.update(getattr(p, "step_buffers", dict)())
        return out

    def max_positions(self) -> int | None:
        limits = [p.max_positions() for p in self.sides if hasattr(p, "max_positions")]
        limits = [n for n in limits if n is not None]
        return min(limits) if limits else None

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None):
        n = x.shape[0]
        hidden = self.spec.left.hidden
        results, biases = [], []
        for part, view in zip(self.sides, cache):
            buf = ctx.arena.take((n, hidden), x.dtype)
            bias = getattr(part, "out_bias", None)
            if bias is not None:
                results.append(part.forward(ctx, x, view, owns_cache, out=buf, add_out_bias=False))
            else:
                results.append(part.forward(ctx, x, view, owns_cache, out=buf))
            biases.append(bias)
        return ops.scaled_sum(results[0], results[1], self.spec.left_scale, self.spec.right_scale,
                              out if out is not None else ctx.arena.take((n, hidden), x.dtype), bias=biases[0], bias_b=biases[1])


registry.register("mixer", "parallel", ParallelMixer)
