"""A matrix memory with exponential gates, the mLSTM of xLSTM ("matrix_memory").

h [tokens, hidden] is the mixer's input; H heads, D key channels, E value channels.  Per head:
  q = W_q h D^(-1/2),  k = W_k h   [D];   v = W_v h   [E]
  i = cap tanh((W_i h + b_i) / cap);   f = logsigmoid(cap tanh((W_f h + b_f) / cap))        the gates, in the logarithm
  m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n <- exp(f + m - m') n + exp(i - m') k
  o = S^T q / (max(|n . q|, exp(-m')) + den_eps)
  y = W_o (o / rms(o) * norm * sigmoid(W_g h))                   rms per head over E; the weight spans all heads' channels
S, n and m start at zero (m at 0, not at minus infinity) and live in 32-bit in the request's state slot.

One product reads h for q, k, v, the output gate and the two gate inputs together (the matrices are stacked at load
time); gates, recurrence (which leaves S^T q and the denominators) and the gated norm (which divides) are 32-bit kernels (``csrc/memory.hip``, ``gated_rms`` of ``csrc/delta.hip``).
The recurrence walks every request's tokens of the step in order, so portions of prompts, single tokens and padding rows
(they own the pad slot) need nothing special.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight
from .needs import StateNeed


def _forget_bias_law(shape, gen):
    """Forget gates that start mostly open: a memory that holds over dozens of tokens."""
    return torch.empty(shape, dtype=torch.float32, device=gen.device).uniform_(1.0, 4.0, generator=gen)


def _input_bias_law(shape, gen):
    return torch.empty(shape, dtype=torch.float32, device=gen.device).normal_(0.0, 0.5, generator=gen)


class MatrixMemory:
    graph_safe = True
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        if spec.heads <= 0 or spec.key_dim <= 0 or spec.value_dim <= 0 or not spec.gate_cap > 0:
            raise ValueError(f"a matrix memory of {spec.heads} heads of {spec.key_dim} x {spec.value_dim} with gates capped at {spec.gate_cap}")
        if spec.key_dim > ops.MEMORY_MAX_KEY_DIM:
            raise ValueError(f"the recurrence takes key sizes up to {ops.MEMORY_MAX_KEY_DIM}")
        self.spec, self.prefix = spec, prefix
        s = spec
        self.qk, self.vw = s.heads * s.key_dim, s.heads * s.value_dim
        # columns of the first product: q | k | v | output gate | input gate | forget gate
        self.k_at, self.v_at, self.g_at = self.qk, 2 * self.qk, 2 * self.qk + self.vw
        self.i_at = self.g_at + self.vw
        self.f_at = self.i_at + s.heads
        self.w_in: LinearWeight | None = None
        self.w_out: LinearWeight | None = None

    def _name(self, i: int) -> str:
        return self.prefix + self.spec.names[i]

    def wanted(self) -> dict:
        s = self.spec
        b = s.bias_suffix
        return {
            self._name(0): ((self.qk, s.hidden), "linear"), self._name(1): ((self.qk, s.hidden), "linear"),
            self._name(2): ((self.vw, s.hidden), "linear"), self._name(3): ((self.vw, s.hidden), "linear"),
            self._name(4): ((s.hidden, self.vw), "linear"), self._name(5): ((self.vw,), "norm"),
            self._name(6): ((s.heads, s.hidden), "linear"), self._name(6) + b: ((s.heads,), _input_bias_law),
            self._name(7): ((s.heads, s.hidden), "linear"), self._name(7) + b: ((s.heads,), _forget_bias_law),
        }

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        rows = -(-(self.f_at + s.heads) // 16) * 16
        w_in = torch.zeros((rows, s.hidden), dtype=dtype, device=device)
        for at, i in ((0, 0), (self.k_at, 1), (self.v_at, 2), (self.g_at, 3), (self.i_at, 6), (self.f_at, 7)):
            t = get(self._name(i))
            w_in[at : at + t.shape[0]].copy_(t)
        self.w_in = LinearWeight(w_in, keep_plain=plain)
        self.w_out = LinearWeight(get(self._name(4)).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)
        f32 = lambda name: get(name).to(device=device, dtype=torch.float32).contiguous()
        self.norm = f32(self._name(5))
        self.bias_i, self.bias_f = f32(self._name(6) + s.bias_suffix), f32(self._name(7) + s.bias_suffix)
        self.state_floats = ops.memory_state_floats(s.heads, s.key_dim, s.value_dim)

    def cache_need(self):
        s = self.spec
        return StateNeed((ops.memory_state_floats(s.heads, s.key_dim, s.value_dim),), torch.float32)

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None):
        s = self.spec
        n, take = x.shape[0], ctx.arena.take
        proj = self.w_in(x, out=take((n, self.w_in.n), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        den = take((n, s.heads), torch.float32)  # the read-out's denominators; the gated norm divides as it reads a head
        o = ops.memory_scan(proj, (0, self.k_at, self.v_at, self.i_at, self.f_at), self.bias_i, self.bias_f, cache.state, ctx.qo_indptr,
                            ctx.state_slots, s.heads, s.key_dim, s.value_dim, s.gate_cap, s.key_dim ** -0.5, den_eps=s.den_eps,
                            out=take((n, self.vw), torch.float32), den=den)
        gated = ops.gated_rms(o, proj[:, self.g_at : self.g_at + self.vw], self.norm, s.norm_eps, s.heads, out=take((n, self.vw), x.dtype),
                              den=den)
        return self.w_out(gated, out=out if out is not None else take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("mixer", "matrix_memory", MatrixMemory)
