"""Soft-max attention through latents (``config.spec.LatentAttentionSpec``): per token the cache holds one normed latent
c [kv_rank] and one rotated key part r [rot_dim] that all heads share, instead of keys and values per head.

With h the input, per head i (D unrotated, R rotated, E value channels, C = kv_rank):
    c_q = norm(W_dq h);  q_i = (W_uq c_q)_i = [q_i^plain (D) | q_i^rot (R)];  [c' | r'] = W_dkv h;  c = norm(c');  r = rotate(r')
    score_i(t, j) = (q_i^plain(t) . Uk_i c(j) + rotate(q_i^rot(t)) . r(j)) * scale,   Uk_i = rows i of W_uk  [D, C]
    out_i(t) = sigmoid(W_g h)_i * Uv_i sum_j p_i(t, j) c(j),                          Uv_i = rows i of W_uv  [E, C]
Because q . (Uk c) = (Uk^T q) . c and Uv sum p c is linear, the attention itself runs over ONE key/value head whose key is
[c | r] and whose value is c, with queries [Uk_i^T q_i^plain | rotate(q_i^rot)]: the paged cache, its manager and the
attention kernels serve it as they serve any layer with one key/value head, key size C + R and value size C.  What is
particular to the layer are three kernels around that (``csrc/latent.hip``) and three products:
    [W_dq; W_dkv; W_g] h  ->  latent_prep (norms, rotation of r, cache write, sigmoid)  ->  W_uq c_q  ->  latent_q_absorb
    ->  attention  ->  latent_out (through Uv_i, times the gate)  ->  W_o.
Norms, angles, rotations, the gate and the scores are 32-bit whatever the model's precision.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .attention import TILES, wide_attention
from .linear import LinearWeight
from .needs import PagedNeed


class LatentAttention:
    graph_safe = True
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        self.spec, self.prefix = spec, prefix
        self.position = registry.build("position", spec.position, prefix)
        if self.position.rotary_dim != spec.rot_dim or getattr(self.position, "interleaved", False):
            raise ValueError("the rotated part of a latent-attention head is rot_dim channels, paired i with i + rot_dim / 2")
        if spec.rot_dim % 2:
            raise ValueError(f"rot_dim={spec.rot_dim} must be even")
        self.first: LinearWeight | None = None
        self.sink_logits: torch.Tensor | None = None
        if not spec.q_rank and spec.gate:
            raise ValueError("a latent-attention layer without a query latent has no gate per head")

    @property
    def _n(self) -> dict:
        keys = ("dq", "dq_norm", "uq", "dkv", "dkv_norm", "uk", "uv", "g", "o")
        return {k: self.prefix + name for k, name in zip(keys, self.spec.names)}

    def wanted(self) -> dict:
        s, n = self.spec, self._n
        out = {
            n["uq"]: ((s.heads * (s.head_dim + s.rot_dim), s.q_rank or s.hidden), "linear"),
            n["dkv"]: ((s.kv_rank + s.rot_dim, s.hidden), "linear"), n["dkv_norm"]: ((s.kv_rank,), "norm"),
            n["uk"]: ((s.heads * s.head_dim, s.kv_rank), "linear"), n["uv"]: ((s.heads * s.value_dim, s.kv_rank), "linear"),
            n["o"]: ((s.hidden, s.heads * s.value_dim), "linear"),
        }
        if s.q_rank:
            out.update({n["dq"]: ((s.q_rank, s.hidden), "linear"), n["dq_norm"]: ((s.q_rank,), "norm")})
        if s.gate:
            out[n["g"]] = ((s.heads, s.hidden), "linear")
        if s.sink_name:
            out[self.prefix + s.sink_name] = ((s.heads,), "around_zero")
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s, n = self.spec, self._n
        plain = layouts == "both"
        to = lambda name: get(name).to(device=device, dtype=dtype).contiguous()
        # one product for everything that reads the layer's input: [W_dq; W_dkv; W_g]
        # (without a query latent the queries' matrix takes the place of W_dq in it, and there is no second product)
        self.q_cols = s.q_rank or s.heads * (s.head_dim + s.rot_dim)
        self.first = LinearWeight(torch.cat([to(n["dq"] if s.q_rank else n["uq"]), to(n["dkv"])] + ([to(n["g"])] if s.gate else [])).contiguous(),
                                  keep_plain=plain)
        self.dq_norm, self.dkv_norm = (to(n["dq_norm"]) if s.q_rank else None), to(n["dkv_norm"])
        self.uq = LinearWeight(to(n["uq"]), keep_plain=plain) if s.q_rank else None
        if s.sink_name:
            self.sink_logits = get(self.prefix + s.sink_name).to(device=device, dtype=torch.float32).contiguous()
        # the two per-head matrices, each in the layout its kernel walks: on the matrix cores (bfloat16, sizes that fit) every
        # head's matrix as [out, in] rows; otherwise as the plain kernels of ``csrc/latent.hip`` read them
        D, R, E, C = s.head_dim, s.rot_dim, s.value_dim, s.kv_rank
        # (without a query latent the queries are columns of the first product's rows, which must then start 16 bytes apart)
        self._mfma_q = (ops.headwise_takes(dtype, C, D, D + R, C + R) and s.hidden % 8 == 0 and s.q_rank % 8 == 0
                        and (s.q_rank > 0 or self.first.n % 8 == 0))
        self._mfma_o = ops.headwise_takes(dtype, E, C, C, E)
        uk, uv = to(n["uk"]), to(n["uv"])
        self.uk = uk.view(s.heads, D, C).transpose(1, 2).contiguous() if self._mfma_q else uk  # [heads, latent, dim] | [heads * dim, latent]
        self.uv = uv.view(s.heads, E, C) if self._mfma_o else uv.view(s.heads, E, C).transpose(1, 2).contiguous()  # [heads, value, latent] | [heads, latent, value]
        self.wo = LinearWeight(to(n["o"]), keep_plain=plain)
        self.position.load(get, dtype, device)
        self._factor = float(getattr(self.position, "factor", 1.0))

    def cache_need(self):
        s = self.spec
        return PagedNeed(1, s.kv_rank + s.rot_dim, s.window, s.kv_rank)

    def batch_plans(self) -> list:
        return [TILES]

    def max_positions(self) -> int | None:
        return self.position.max_positions

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None):
        s, pos = self.spec, self.position
        n = x.shape[0]
        if not owns_cache:
            raise ValueError("a latent-attention layer writes its own cache")
        if pos.max_positions is not None and ctx.max_position >= pos.max_positions:
            raise ValueError(f"position {ctx.max_position} is beyond the model's {pos.max_positions} positions")
        H, D, R, E, C = s.heads, s.head_dim, s.rot_dim, s.value_dim, s.kv_rank
        take = ctx.arena.take
        table = ctx.block_tables[cache.group]
        proj = self.first(x, out=take((n, self.first.n), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        gate = take((n, H), torch.float32) if s.gate else None
        if s.q_rank:
            cq = take((n, s.q_rank), x.dtype)
            ops.latent_prep(proj, self.dq_norm, self.dkv_norm, pos.inv_freq, self._factor, ctx.positions, ctx.token_req, table, cache.k, cache.v,
                            s.q_rank, C, R, H if s.gate else 0, s.norm_eps, cq, gate)
            q = self.uq(cq, out=take((n, H * (D + R)), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        else:
            # the queries are the first columns of the product; the rest of a row is [latent | rotated part]
            ops.latent_prep(proj[:, self.q_cols :], None, self.dkv_norm, pos.inv_freq, self._factor, ctx.positions, ctx.token_req, table, cache.k,
                            cache.v, 0, C, R, 0, s.norm_eps, None, None)
            q = proj[:, : self.q_cols]
        q_lat = take((n, H * (C + R)), x.dtype)
        if self._mfma_q:
            ops.headwise_product(q, D + R, self.uk, q_lat, C + R)
        ops.latent_q_absorb(q, None if self._mfma_q else self.uk, pos.inv_freq, self._factor, ctx.positions, H, D, R, C, out=q_lat)
        o_lat = take((n, H * C), x.dtype)
        if ops.wide_attention_takes(x.dtype, C + R, C, cache.k.shape[2]):
            wide_attention(ctx, q_lat, o_lat, cache, table, H, 1, C + R, C, s.softmax_scale, window=s.window, sink_logits=self.sink_logits)
        else:
            ops.attention_generic(q_lat, o_lat, cache.k, cache.v, ctx.token_req, ctx.positions, table, H, 1, C + R, s.softmax_scale,
                                  window=s.window, v_dim=C, sink_logits=self.sink_logits)
        att = take((n, H * E), x.dtype)
        if self._mfma_o:
            ops.headwise_product(o_lat, C, self.uv, att, E, gate=gate)
        else:
            ops.latent_out(o_lat, self.uv, gate, H, C, E, out=att)
        return self.wo(att, out=out if out is not None else take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("mixer", "latent_attention", LatentAttention)
