"""A mixture of small gated feed-forward experts with a router, and optionally one shared expert ("moe").

  z = W_r h + b                       router logits, in 32-bit
  the ``top`` largest logits are chosen; their weights are the soft-max over the chosen logits alone
  (``score`` = "sigmoid": s = sigmoid(z); the choice goes by s + correction, inside the ``keep_groups`` groups of neighbouring
  experts whose two largest choice scores add up highest; the weights are the chosen s, not renormalized)
  expert(h) = W_down (g sigmoid(alpha g) (u + shift)),  g = min(W_gate h, limit),  u = clamp(W_up h, -limit, limit)
  (limit infinite, alpha 1, shift 0: W_down (silu(W_gate h) * W_up h))
  y = sum over the chosen experts of weight * expert(h)  +  shared(h)

The experts' matrices are stacked at load time ([experts, ff, W] and [experts, W, ff]).  Steps of few rows run one
workgroup per (token, chosen expert), which streams that expert's matrices; steps of many rows sort the (token, expert)
pairs by expert on the device and run the experts as grouped products of 16-row tiles (``csrc/moe.hip``).  Nothing
depends on the host knowing which experts were chosen, so a step can be captured.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight


class MoE:
    graph_safe = True
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        if not 0 < spec.top <= spec.experts or spec.top > ops.MOE_MAX_TOP or spec.experts > ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{spec.top} of {spec.experts} experts (at most {ops.MOE_MAX_TOP} of {ops.MOE_MAX_EXPERTS})")
        if spec.score not in ("softmax", "sigmoid"):
            raise ValueError(f"score={spec.score!r}: use 'softmax' or 'sigmoid'")
        if spec.correction_name and spec.score != "sigmoid":
            raise ValueError("a correction on the choice belongs to sigmoid scores")
        if spec.groups < 1 or spec.experts % spec.groups or not 1 <= spec.keep_groups <= spec.groups or spec.top > spec.keep_groups * (spec.experts // spec.groups):
            raise ValueError(f"{spec.experts} experts in {spec.groups} groups of which {spec.keep_groups} are kept, {spec.top} chosen")
        self.spec, self.prefix = spec, prefix

    def _expert(self, e: int, which: int) -> str:
        return f"{self.prefix}{self.spec.expert_prefix}{e}.{self.spec.names[which]}"

    def _shared(self, which: int) -> str:
        return self.prefix + self.spec.shared_prefix + self.spec.names[which]

    def wanted(self) -> dict:
        s = self.spec
        ff = s.expert.intermediate
        out = {self.prefix + s.router_name: ((s.experts, s.hidden), "linear")}
        if s.router_bias_name:
            out[self.prefix + s.router_bias_name] = ((s.experts,), "bias")
        if s.correction_name:
            out[self.prefix + s.correction_name] = ((s.experts,), "bias")
        for e in range(s.experts):
            out[self._expert(e, 0)] = ((ff, s.hidden), "linear")
            out[self._expert(e, 1)] = ((ff, s.hidden), "linear")
            out[self._expert(e, 2)] = ((s.hidden, ff), "linear")
        if s.shared is not None:
            sf = s.shared.intermediate
            out[self._shared(0)] = ((sf, s.hidden), "linear")
            out[self._shared(1)] = ((sf, s.hidden), "linear")
            out[self._shared(2)] = ((s.hidden, sf), "linear")
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        stack = lambda which: torch.stack([get(self._expert(e, which)).to(device=device, dtype=dtype) for e in range(s.experts)]).contiguous()
        self.gate, self.up, self.down = stack(0), stack(1), stack(2)
        self.router = get(self.prefix + s.router_name).to(device=device, dtype=torch.float32).contiguous()
        f32 = lambda name: get(self.prefix + name).to(device=device, dtype=torch.float32).contiguous() if name else None
        self.router_bias, self.correction = f32(s.router_bias_name), f32(s.correction_name)
        self.shared_in = self.shared_out = None
        if s.shared is not None:
            gu = torch.cat([get(self._shared(0)), get(self._shared(1))]).to(device=device, dtype=dtype).contiguous()
            self.shared_in = LinearWeight(gu, keep_plain=plain)
            self.shared_out = LinearWeight(get(self._shared(2)).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def forward(self, ctx, x, out: torch.Tensor | None = None):
        s = self.spec
        n, take = x.shape[0], ctx.arena.take
        sel, wt = take((n, s.top), torch.int32), take((n, s.top), torch.float32)
        ops.moe_route(x, self.router, self.router_bias, s.top, sel, wt, logits=take((n, s.experts), torch.float32), sigmoid=s.score == "sigmoid",
                      correction=self.correction, groups=s.groups, keep=s.keep_groups)
        base = None
        if s.shared is not None:
            sf = s.shared.intermediate
            gu = self.shared_in(x, out=take((n, 2 * sf), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
            act = ops.clipped_glu(gu, s.shared.limit, s.shared.alpha, out=take((n, sf), x.dtype), shift=s.shared.shift)
            base = self.shared_out(act, out=take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        parts = ops.moe_experts(x, self.gate, self.up, self.down, sel, wt, s.expert.limit, s.expert.alpha, take, shift=s.expert.shift)
        return ops.moe_combine(parts, base, out if out is not None else take((n, s.hidden), x.dtype))


registry.register("ffn", "moe", MoE)
