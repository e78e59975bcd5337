"""Retention: linear attention with one fixed decay per head, no soft-max and no denominator ("retention").

h [tokens, hidden] is the mixer's input; H heads, D key channels, E value channels.  Per head:
  q = W_q h,  k = W_k h   [D];   v = W_v h   [E];   q and k rotated by their position, k then times key_scale
  S_t = decay S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t                      S [D, E] starts at zero
  y = W_o (o / rms(o) * silu(W_g h))                                     rms per head over E, no weight
S lives in 32-bit in the request's state slot and is carried from step to step.

One product reads h for q, k, v and the gate together (the matrices are stacked at load time); rotation and scaling
(``retention_prep``), the recurrence (``retention_scan``) and the gated norm (``gated_rms``) are 32-bit kernels.  The
recurrence walks every request's tokens of the step in order, so portions of prompts, single tokens and padding rows
(they own the pad slot) need nothing special.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight
from .needs import StateNeed


class Retention:
    graph_safe = True
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        if spec.heads <= 0 or spec.key_dim <= 0 or spec.value_dim <= 0 or len(spec.decay) != spec.heads:
            raise ValueError(f"retention of {spec.heads} heads of {spec.key_dim} x {spec.value_dim} with {len(spec.decay)} decays")
        if spec.key_dim > ops.RETENTION_MAX_KEY_DIM:
            raise ValueError(f"the recurrence takes key sizes up to {ops.RETENTION_MAX_KEY_DIM}")
        self.spec, self.prefix = spec, prefix
        self.position = registry.build("position", spec.position, prefix)
        if self.position.rotary_dim > spec.key_dim:
            raise ValueError("the rotary part of a head cannot be wider than the head")
        s = spec
        self.qk, self.vw = s.heads * s.key_dim, s.heads * s.value_dim
        # columns of the first product: q | k | v | gate
        self.k_at, self.v_at, self.g_at = self.qk, 2 * self.qk, 2 * self.qk + self.vw
        self.w_in: LinearWeight | None = None
        self.w_out: LinearWeight | None = None

    def _name(self, i: int) -> str:
        return self.prefix + self.spec.names[i]

    def wanted(self) -> dict:
        s = self.spec
        return {
            self._name(0): ((self.qk, s.hidden), "linear"), self._name(1): ((self.qk, s.hidden), "linear"),
            self._name(2): ((self.vw, s.hidden), "linear"), self._name(3): ((self.vw, s.hidden), "linear"),
            self._name(4): ((s.hidden, self.vw), "linear"), **self.position.wanted(),
        }

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        rows = -(-(self.g_at + self.vw) // 16) * 16
        w_in = torch.zeros((rows, s.hidden), dtype=dtype, device=device)
        for at, i in ((0, 0), (self.k_at, 1), (self.v_at, 2), (self.g_at, 3)):
            t = get(self._name(i))
            w_in[at : at + t.shape[0]].copy_(t)
        self.w_in = LinearWeight(w_in, keep_plain=plain)
        self.w_out = LinearWeight(get(self._name(4)).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)
        self.decay = torch.tensor([float(d) for d in s.decay], dtype=torch.float32, device=device)
        self.position.load(get, dtype, device)
        self._form = dict(interleaved=bool(getattr(self.position, "interleaved", False)), factor=float(getattr(self.position, "factor", 1.0)))

    def cache_need(self):
        s = self.spec
        return StateNeed((s.heads * s.key_dim * s.value_dim,), torch.float32)

    def max_positions(self) -> int | None:
        return self.position.max_positions

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None):
        s, pos = self.spec, self.position
        n, take = x.shape[0], ctx.arena.take
        if pos.max_positions is not None and ctx.max_position >= pos.max_positions:
            raise ValueError(f"position {ctx.max_position} is beyond the model's {pos.max_positions} positions")
        proj = self.w_in(x, out=take((n, self.w_in.n), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        qkv = ops.retention_prep(proj, (0, self.k_at, self.v_at), ctx.positions, pos.inv_freq, s.heads, s.key_dim, s.value_dim, pos.rotary_dim,
                                 s.key_scale, out=take((n, 2 * self.qk + self.vw), torch.float32), **self._form)
        o = ops.retention_scan(qkv, self.decay, cache.state, ctx.qo_indptr, ctx.state_slots, s.heads, s.key_dim, s.value_dim,
                               out=take((n, self.vw), torch.float32))
        gated = ops.gated_rms(o, proj[:, self.g_at : self.g_at + self.vw], None, s.norm_eps, s.heads, out=take((n, self.vw), x.dtype), silu=True)
        return self.w_out(gated, out=out if out is not None else take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("mixer", "retention", Retention)
