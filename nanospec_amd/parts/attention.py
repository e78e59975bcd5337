"""Grouped-query soft-max attention over the paged cache (reference: model/llama.py:161-184 and
model/attention.py).

Per step: one product for q, k and v together (the three checkpoint matrices are stacked at load
time), rotation of q and k fused with the write of k and v into the pages, attention of every token
over its request's pages, output projection.  float32 runs the plain attention kernel; bfloat16 runs
the matrix-core kernel: prompt portions as tiles of 16 tokens of one head, decode rows as tiles of
all heads of a group with the keys cut into ranges that are joined afterwards.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight
from .needs import PagedNeed

# How the matrix-core attention kernel is launched, from the counts of a step's batch and the size of the GPU
PORTION_RANGE_BLOCKS = 16  # the fewest 32-key blocks that a range of a prompt portion's keys is worth a workgroup of its own
PORTION_SINGLE_SET_BLOCKS = 128  # 32-key blocks of the longest row from which a workgroup is one set of waves instead of two
DECODE_WAVES_PER_UNIT = 4  # decode rows' keys are cut into ranges until about this many waves per compute unit are at work
LONG_ROW_KEYS = 8192  # rows that may reach this many keys get up to 32 ranges instead of 16
QKV_JOIN_MAX_RANGES = 4  # 17 to 128 rows: the kernel that joins the ranges of the q/k/v product, rotates and writes the cache reads
#                          every range, so more of them cost it what they gain the product


class TilePlan:
    """The batch as the matrix-core attention kernel walks it (a batch plan, see ``engine.context``): the requests that
    bring more than one token cut into tiles of ``TOKENS`` tokens, then the requests that bring exactly one, a tile each.
    A tile is ``ops.TILE_INTS`` ints: request, first token of the tile among the request's tokens of this step, row of the
    request's first token, tokens of the request in this step, keys after this step, and for one-token tiles the keys that
    all of them read in this step over all layers (by which the kernel chooses its loads: what cannot stay cached until
    the next step is read past the caches).  shape = (portion tiles, one-token tiles); a region of a fixed shape may hold
    more portion tiles than the batch needs: the rest bring no tokens and the kernel skips them."""

    key = "attention.tiles"
    TOKENS = 32

    def shape(self, lens) -> tuple[int, int]:
        return sum(-(-n // self.TOKENS) for n in lens if n != 1), sum(1 for n in lens if n == 1)

    def shape_captured(self, rows: int, tokens: int, portions: int) -> tuple[int, int]:
        # every portion may end in a tile that is not full
        return (-(-tokens // self.TOKENS) + portions if tokens else 0), rows

    def ints(self, shape) -> int:
        return ops.TILE_INTS * (shape[0] + shape[1])

    def fill(self, out: np.ndarray, shape, facts) -> None:
        tc, td = shape
        lens, indptr, kv, n = facts.lens, facts.indptr, facts.kv, facts.covered
        if tc:
            rows = [(b, t0, indptr[b], lens[b], kv[b], 0, 0, 0) for b in range(n) if lens[b] != 1 for t0 in range(0, lens[b], self.TOKENS)]
            rows += [(facts.n_reqs - 1, 0, 0, 0, 0, 0, 0, 0)] * (tc - len(rows))  # tiles without tokens
            out[: ops.TILE_INTS * tc] = np.asarray(rows, dtype=np.int32).reshape(-1)
        if td:
            req = np.nonzero(lens[:n] == 1)[0].astype(np.int32)
            d = np.zeros((td, ops.TILE_INTS), dtype=np.int32)
            k = len(req)
            d[:k, 0], d[:k, 2], d[:k, 3], d[:k, 4] = req, indptr[req], 1, kv[req]
            d[:k, 5] = min(int(kv[req].sum()) * facts.kv_layers, 2**31 - 1)
            out[ops.TILE_INTS * tc : ops.TILE_INTS * (tc + td)] = d.reshape(-1)

    @staticmethod
    def views(ctx):
        """-> (portion tiles, one-token tiles) as int32 [tiles, TILE_INTS] device views."""
        region, (tc, td) = ctx.plans[TilePlan.key]
        cut = ops.TILE_INTS * tc
        return region[:cut].view(tc, ops.TILE_INTS), region[cut : cut + ops.TILE_INTS * td].view(td, ops.TILE_INTS)


TILES = TilePlan()


@dataclass
class LaunchPlan:
    tiles: torch.Tensor  # int32 [n_tiles, 8]
    hp: int
    splits: int
    workspace: tuple | None
    qt: int = 1
    coop: bool = False


def launch_plans(ctx, group: int, kv_heads: int, head_dim: int, span: int = 0) -> list[LaunchPlan]:
    """How the matrix-core attention kernel is launched for a mixer with ``group`` query heads per key/value head, over
    the tile lists of the batch: prompt portions as 32-token tiles of one head, their keys cut into ranges when there
    are too few tiles to fill the GPU and many keys (a short portion late in a long prompt); decode rows with all heads
    of a group in one tile and the keys cut into ranges so that the launch fills the GPU.  ``span`` > 0: no query sees more
    than this many keys (a chunked mask), whatever the rows' lengths."""
    plans = []  # made afresh per call: the workspace lives in the caller's arena scope
    units = ops.compute_units(ctx.token_ids.device)
    chunk_tiles, decode_tiles = TilePlan.views(ctx)
    n_chunk_tiles, n_decode_tiles = chunk_tiles.shape[0], decode_tiles.shape[0]
    if n_chunk_tiles:
        tokens = TilePlan.TOKENS
        wgs = n_chunk_tiles * kv_heads * -(-group // 4)
        blocks = -(-(min(ctx.max_chunk_kv, span + tokens) if span else ctx.max_chunk_kv) // 32)
        # fewer workgroups than compute units (one fits a unit): cut the keys into ranges
        splits = max(1, min(16, units // wgs, blocks // PORTION_RANGE_BLOCKS))
        ws = None
        if splits > 1:
            cols = n_chunk_tiles * tokens * kv_heads * group
            ws = (ctx.arena.take((cols * splits * head_dim,), torch.float32), ctx.arena.take((cols * splits * 2,), torch.float32))
        # many workgroups with long rows of keys: one set of four waves per workgroup, two workgroups to a compute unit,
        # each with a barrier of its own (4 to 8% faster from 4,096 keys on; slower for short rows)
        single = splits == 1 and wgs >= 2 * units and blocks >= PORTION_SINGLE_SET_BLOCKS
        plans.append(LaunchPlan(chunk_tiles, 1, splits, ws, qt=tokens // 16, coop=single))
    if n_decode_tiles:
        hp = 1
        while hp < min(group, 16):
            hp *= 2
        # decode is bound by the latency of each wave's chain of loads: the four waves of a workgroup share a tile, and
        # the keys are cut into ranges until about a thousand waves are at work
        # (up to 32 ranges where requests may reach 8,192 keys and the tiles are few, a single request say: at 131,072
        # keys 86 against 132 us a layer; the kernel leaves the ranges beyond the sixteenth empty for shorter rows,
        # and where no request can be that long they are not launched: they would cost a captured step 1%)
        items = n_decode_tiles * kv_heads * -(-group // hp)
        longest = min(ctx.max_kv_len, span) if span else ctx.max_kv_len
        splits = max(1, min(32 if longest >= LONG_ROW_KEYS else 16, DECODE_WAVES_PER_UNIT * units // (4 * items)))
        # never ranges of fewer than 256 keys (in a captured step: of what its block tables can hold): short rows are
        # short chains already, and a single range needs no kernel to join it
        splits = max(1, min(splits, -(-longest // 256)))
        ws = None
        if splits > 1:
            cols = n_decode_tiles * (16 // hp) * kv_heads * group
            ws = (ctx.arena.take((cols * splits * head_dim,), torch.float32), ctx.arena.take((cols * splits * 2,), torch.float32))
        plans.append(LaunchPlan(decode_tiles, hp, splits, ws, coop=True))
    return plans


WIDE_RANGE_KEYS = 64  # the fewest keys that a range of a row's keys is worth a wave of its own in the two-size kernel


def wide_attention(ctx, q, out, cache, table, heads: int, kv_heads: int, head_dim: int, v_dim: int, scale: float, window: int = 0,
                   slope_exp: float = 0.0, sink_logits=None):
    """Launch ``ops.attention_wide`` (keys and values of two sizes on the matrix cores) over the tile lists of the batch:
    prompt portions as sets of 16 tokens of one head, decode rows with up to 16 heads of a group in one wave's columns and
    the keys cut into ranges until the launch fills the GPU (an item of that kernel is one wave)."""
    units = ops.compute_units(ctx.token_ids.device)
    group = heads // kv_heads
    chunk_tiles, decode_tiles = TilePlan.views(ctx)
    take = ctx.arena.take
    if chunk_tiles.shape[0]:
        qt = TilePlan.TOKENS // 16
        waves = chunk_tiles.shape[0] * qt * heads
        longest = min(ctx.max_chunk_kv, window + TilePlan.TOKENS) if window else ctx.max_chunk_kv
        splits = max(1, min(16, 4 * units // max(1, waves), longest // (4 * WIDE_RANGE_KEYS)))
        ws = None
        if splits > 1:
            cols = chunk_tiles.shape[0] * TilePlan.TOKENS * heads
            ws = (take((cols * splits * v_dim,), torch.float32), take((cols * splits * 2,), torch.float32))
        ops.attention_wide(q, out, cache.k, cache.v, chunk_tiles, table, heads, kv_heads, head_dim, v_dim, scale, window=window, hp=1,
                           splits=splits, workspace=ws, qt=qt, slope_exp=slope_exp, sink_logits=sink_logits)
    if decode_tiles.shape[0]:
        hp = 1
        while hp < min(group, 16):
            hp *= 2
        waves = decode_tiles.shape[0] * kv_heads * -(-group // hp)
        longest = min(ctx.max_kv_len, window) if window else ctx.max_kv_len
        # (wide heads: a block of 32 keys is a long chain of loads and products already, so ranges go down to one block)
        range_keys = WIDE_RANGE_KEYS // 2 if head_dim + v_dim > 512 else WIDE_RANGE_KEYS
        splits = max(1, min(32, 4 * units // max(1, waves), -(-longest // range_keys)))
        ws = None
        if splits > 1:
            cols = decode_tiles.shape[0] * (16 // hp) * heads
            ws = (take((cols * splits * v_dim,), torch.float32), take((cols * splits * 2,), torch.float32))
        ops.attention_wide(q, out, cache.k, cache.v, decode_tiles, table, heads, kv_heads, head_dim, v_dim, scale, window=window, hp=hp,
                           splits=splits, workspace=ws, qt=1, slope_exp=slope_exp, sink_logits=sink_logits)
    return out


class Attention:
    graph_safe = True
    ends_in_residual = True  # forward takes residual=IntoResidual
    takes_layouts = True  # load takes which copies of its matrices to keep

    def __init__(self, spec, prefix: str) -> None:
        if spec.heads % spec.kv_heads:
            raise ValueError(f"{spec.heads} heads are not a multiple of {spec.kv_heads} key/value heads")
        self.spec, self.prefix = spec, prefix
        self.position = registry.build("position", spec.position, prefix)
        if self.position.rotary_dim > spec.head_dim:
            raise ValueError("the rotary part of a head cannot be wider than the head")
        self.wqkv: LinearWeight | None = None
        self.wo: LinearWeight | None = None
        self.qkv_bias = self.q_norm = self.k_norm = self.v_mix = None
        self.out_bias: torch.Tensor | None = None  # the output projection's bias; a block may add it itself (add_out_bias=False)
        if spec.value_mix not in ("", "source", "mix"):
            raise ValueError(f"value_mix={spec.value_mix!r}: use '', 'source' or 'mix'")
        if (spec.bias or spec.whole_norm_eps is not None or spec.value_mix) and not spec.own_kv:
            raise ValueError("biases, whole-projection norms and mixed values belong to a layer with key/value projections of its own")
        if spec.whole_norm_eps is not None and spec.qk_norm_eps is not None:
            raise ValueError("a norm over the whole projection stands alone: no per-head unit norm beside it")
        if (spec.sink_name or spec.out_gate) and not spec.own_kv:
            raise ValueError("a learned sink and an output gate belong to a layer with key/value projections of its own")
        if spec.sink_name and spec.sink:
            raise ValueError("the soft-max has one sink: of score 0, or a learned one")
        self.sink_logits: torch.Tensor | None = None
        self.head_form = spec.head_norm_eps is not None or spec.value_is_key  # per-head norms with weights, values that are the keys
        if self.head_form and (spec.qk_norm_eps is not None or spec.whole_norm_eps is not None or spec.value_mix or not spec.own_kv):
            raise ValueError("per-head norms with weights and values that are the keys stand beside biases and a rotation only")
        if spec.value_is_key and spec.v_dim != spec.head_dim:
            raise ValueError("values that are the keys have the keys' size")
        self.q_head_norm = self.k_head_norm = None

    VALUES_KEY = "attention.values"  # where a "source" layer leaves its values of the step's tokens (``ctx.shared``)

    def step_buffers(self) -> dict:
        """Buffers that live as long as a step and that layers hand to each other: key -> columns per token."""
        s = self.spec
        return {self.VALUES_KEY: s.kv_heads * s.v_dim} if s.value_mix else {}

    @property
    def _names(self):
        p = self.prefix
        return tuple(p + name for name in self.spec.names)

    def wanted(self) -> dict:
        s = self.spec
        q, k, v, o = self._names
        out = {q: ((s.heads * s.head_dim, s.hidden), "linear"), o: ((s.hidden, s.heads * s.v_dim), "linear"), **self.position.wanted()}
        if s.own_kv:
            out[k] = ((s.kv_heads * s.head_dim, s.hidden), "linear")
            if not s.value_is_key:
                out[v] = ((s.kv_heads * s.v_dim, s.hidden), "linear")
        if s.bias:
            for name in (q, k, v, o):
                if name in out:
                    out[name + s.bias_suffix] = ((out[name][0][0],), "bias")
        if s.head_norm_eps is not None:
            out[q + s.head_norm_suffix] = ((s.head_dim,), "norm")
            out[k + s.head_norm_suffix] = ((s.head_dim,), "norm")
        if s.whole_norm_eps is not None:
            out[q + s.whole_norm_suffix] = ((s.heads * s.head_dim,), "norm")
            out[k + s.whole_norm_suffix] = ((s.kv_heads * s.head_dim,), "norm")
        if s.sink_name:
            out[self.prefix + s.sink_name] = ((s.heads,), "around_zero")
        if s.out_gate:
            out[self.prefix + s.gate_name] = ((s.heads * s.v_dim, s.hidden), "linear")
        if s.value_mix:
            # (a "source" layer's checkpoint holds the tensor too; it is not used there)
            out[self.prefix + s.value_mix_name] = ((), lambda shape, gen: torch.full(shape, 0.5, device=gen.device)
                                                   + 0.2 * torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device))
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        q, k, v, o = self._names
        rows = s.heads * s.head_dim + (s.kv_heads * (s.head_dim + (0 if s.value_is_key else s.v_dim)) if s.own_kv else 0)
        self.gate_at = rows  # the output gate's logits, if the layer has a gate, are the last columns of the first product
        stacked = (q,) if not s.own_kv else ((q, k) if s.value_is_key else (q, k, v))
        if s.out_gate:
            rows += s.heads * s.v_dim
            stacked += (self.prefix + s.gate_name,)
        wqkv = torch.empty((rows, s.hidden), dtype=dtype, device=device)
        at = 0
        for name in stacked:
            t = get(name)
            wqkv[at : at + t.shape[0]].copy_(t)
            at += t.shape[0]
        self.position.load(get, dtype, device)
        # how the position encoding pairs channels and scales cosine and sine (the kernels' ``RopeForm``)
        self._form = dict(interleaved=bool(getattr(self.position, "interleaved", False)), factor=float(getattr(self.position, "factor", 1.0)))
        to = lambda name: get(name).to(device=device, dtype=dtype).contiguous()
        if s.bias:
            if s.out_gate:
                raise ValueError("an output gate beside biased projections is not built")
            self.qkv_bias = torch.cat([to(name + s.bias_suffix) for name in stacked]).contiguous()
            self.out_bias = to(o + s.bias_suffix)
        if s.head_norm_eps is not None:
            self.q_head_norm, self.k_head_norm = to(q + s.head_norm_suffix), to(k + s.head_norm_suffix)
        if s.whole_norm_eps is not None:
            self.q_norm, self.k_norm = to(q + s.whole_norm_suffix), to(k + s.whole_norm_suffix)
        if s.value_mix == "mix":
            self.v_mix = to(self.prefix + s.value_mix_name).reshape(1)
        if s.sink_name:
            self.sink_logits = get(self.prefix + s.sink_name).to(device=device, dtype=torch.float32).contiguous()
        if s.general:
            # the general path: one product for what the layer projects, then norm / cache write and attention as kernels
            self.wqkv_rope = None
            self.wqkv = LinearWeight(wqkv, keep_plain=plain)
            self.wo = LinearWeight(get(o).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)
            return
        # for few rows the stacked matrix is streamed by a kernel that rotates and writes the cache in its epilogue; it
        # wants the rows tiled in an order of its own
        rot = self.position.rotary_dim
        self.wqkv_rope = None
        if dtype == torch.bfloat16 and s.hidden % 8 == 0 and s.head_dim % 16 == 0 and rot % 16 == 0:
            self.wqkv_rope = ops.TiledWeight(wqkv, ops.qkv_rope_row_order(s.heads, s.kv_heads, s.head_dim, rot, self._form["interleaved"]))
        # (without the plain layout the stacked matrix is also kept tiled in its own row order, for more than 16 rows)
        self.wqkv = LinearWeight(wqkv, keep_plain=plain, tiled=self.wqkv_rope is None or not plain)
        self.wo = LinearWeight(get(o).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def cache_need(self):
        s = self.spec
        if not s.own_kv:
            return None  # it reads the cache of the run-order entry that its LayerCall names
        return PagedNeed(s.kv_heads, s.head_dim, s.window, 0 if s.v_dim == s.head_dim else s.v_dim)

    def batch_plans(self) -> list:
        """What this mixer asks the batch builder to put on the device each step (``engine.context``)."""
        return [TILES]

    def max_positions(self) -> int | None:
        return self.position.max_positions

    def links_norms(self, rows: int) -> bool:
        """Whether, for this many rows, ``forward`` takes a ``PreNormed`` input and an ``IntoResidual`` ending."""
        if self.spec.general:
            return False
        first = self.wqkv_rope is not None or self.wqkv.links_norms(rows)
        return rows <= 16 and first and self.wo.links_norms(rows)

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None, residual=None, add_out_bias: bool = True):
        s = self.spec
        n = x.shape[0]
        pos = self.position
        if pos.max_positions is not None and ctx.max_position >= pos.max_positions:
            raise ValueError(f"position {ctx.max_position} is beyond the model's {pos.max_positions} positions")
        qkv = ctx.arena.take((n, self.wqkv.n), x.dtype)
        table = ctx.block_tables[cache.group]
        if s.general:
            return self._forward_general(ctx, x, cache, owns_cache, out, residual, qkv, table, add_out_bias)
        if self.wqkv_rope is not None and n <= 16 and ops.tiled_takes(x.x if isinstance(x, ops.PreNormed) else x, s.hidden):
            ops.linear_qkv_rope(x, self.wqkv_rope, qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v,
                                s.heads, s.kv_heads, s.head_dim, pos.rotary_dim, write_kv=owns_cache, **self._form)
        elif (self.wqkv_rope is not None and n <= ops.WIDE_TALL_ROWS and not isinstance(x, ops.PreNormed) and ops.tiled_takes(x[:1], s.hidden)
              and ops.wide_plan(self.wqkv_rope.n, s.hidden, n)[0] > 1):
            # 17 to 128 rows: the product streams the same tiled matrix with K cut into ranges, and the kernel that adds the
            # ranges rotates and writes the cache in the same pass (the library's product and a rotation kernel otherwise)
            ksplit, nt = ops.wide_plan(self.wqkv_rope.n, s.hidden, n)
            ksplit = min(ksplit, QKV_JOIN_MAX_RANGES)
            ws = ctx.arena.take((ksplit * n * self.wqkv_rope.n,), torch.float32)
            part = ops.linear_wide(x, self.wqkv_rope, workspace=ws, ksplit=ksplit, nt=nt, defer=True)
            ops.rope_kv_from_partial(part, qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v, s.heads, s.kv_heads,
                                     s.head_dim, pos.rotary_dim, write_kv=owns_cache, **self._form)
        else:
            self.wqkv(x, out=qkv, arena=ctx.arena, plain_copy=not ctx.captured)
            ops.rope_kv_write(qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v, s.heads, s.kv_heads,
                              s.head_dim, pos.rotary_dim, write_kv=owns_cache, **self._form)
        att = ctx.arena.take((n, s.heads * s.head_dim), x.dtype)
        page = cache.k.shape[2]
        if ops.mfma_attention_takes(x.dtype, s.head_dim, page):
            group = s.heads // s.kv_heads
            for plan in launch_plans(ctx, group, s.kv_heads, s.head_dim):
                ops.attention_mfma(qkv, att, cache.k, cache.v, plan.tiles, table, s.heads, s.kv_heads, s.head_dim,
                                   s.softmax_scale, window=s.window, hp=plan.hp, splits=plan.splits, workspace=plan.workspace,
                                   qt=plan.qt, coop=plan.coop)
        else:
            ops.attention_generic(qkv, att, cache.k, cache.v, ctx.token_req, ctx.positions, table, s.heads, s.kv_heads,
                                  s.head_dim, s.softmax_scale, window=s.window)
        if residual is not None:
            return self.wo.into_residual(att, residual, arena=ctx.arena, plain_copy=not ctx.captured)
        return self.wo(att, out=out, arena=ctx.arena, plain_copy=not ctx.captured)


    def _forward_general(self, ctx, x, cache, owns_cache, out, residual, qkv, table, add_out_bias=True):
        """Attention with any of the spec's options: values of another size than the keys, unit-RMS queries and keys, capped
        scores, a chunked mask, a sink, keys and values of another layer, biases, a norm over the whole of q and of k, a
        bias by distance, values mixed with an earlier layer's.  The cache holds keys as the scores meet them (after norm
        and rotation) and values as they are read (after mixing), so a layer that borrows them brings only its queries."""
        s, pos = self.spec, self.position
        n = x.shape[0]
        if s.own_kv != bool(owns_cache):
            raise ValueError("an attention layer writes the cache exactly if it has key/value projections of its own")
        if cache.k.shape[1:] != (s.kv_heads, cache.k.shape[2], s.head_dim) or cache.v.shape[2] != s.v_dim:
            raise ValueError("the cache that this layer reads has other heads or sizes than the layer")
        self.wqkv(x, out=qkv, arena=ctx.arena, plain_copy=not ctx.captured)
        if self.head_form:
            if pos.max_positions is not None and ctx.max_position >= pos.max_positions:
                raise ValueError(f"position {ctx.max_position} is beyond the model's {pos.max_positions} positions")
            ops.head_norm_rope_kv_write(qkv, ctx.positions, ctx.token_req, table, pos.inv_freq if pos.rotary_dim else None, cache.k, cache.v,
                                        s.heads, s.kv_heads, s.head_dim, s.v_dim, s.head_norm_eps or 0.0, pos.rotary_dim, bias=self.qkv_bias,
                                        q_weight=self.q_head_norm, k_weight=self.k_head_norm, value_is_key=s.value_is_key, **self._form)
        elif s.whole_norm_eps is not None and pos.rotary_dim:
            # a norm over the whole of q and of k, then the rotation, then the pages
            if s.bias or s.value_mix:
                raise ops.KernelRefused("rotation behind a whole-projection norm together with biases or mixed values is not built")
            ops.whole_norm_kv_write(qkv, ctx.positions, ctx.token_req, table, cache.k, cache.v, s.heads, s.kv_heads, s.head_dim, s.v_dim,
                                    s.whole_norm_eps, q_weight=self.q_norm, k_weight=self.k_norm, inv_freq=pos.inv_freq,
                                    rotary_dim=pos.rotary_dim, **self._form)
        elif pos.rotary_dim:
            if s.qk_norm_eps is not None or s.v_dim != s.head_dim or not s.own_kv:
                raise ops.KernelRefused("rotation together with unit-RMS queries and keys, another value size or borrowed keys is not built")
            if s.bias or s.value_mix:
                raise ops.KernelRefused("rotation together with biases or mixed values is not built")
            ops.rope_kv_write(qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v, s.heads, s.kv_heads,
                              s.head_dim, pos.rotary_dim, write_kv=True, **self._form)
        elif s.bias or s.whole_norm_eps is not None or s.value_mix:
            if s.qk_norm_eps is not None:
                raise ops.KernelRefused("a per-head unit norm together with biases, a whole-projection norm or mixed values is not built")
            shared = ctx.shared.get(self.VALUES_KEY) if s.value_mix else None
            if s.value_mix and shared is None:
                raise ops.KernelRefused("the step holds no buffer for the values that layers hand to each other")
            ops.whole_norm_kv_write(qkv, ctx.positions, ctx.token_req, table, cache.k, cache.v, s.heads, s.kv_heads, s.head_dim, s.v_dim,
                                    s.whole_norm_eps or 0.0, bias=self.qkv_bias, q_weight=self.q_norm, k_weight=self.k_norm,
                                    mix=self.v_mix, v_other=shared if s.value_mix == "mix" else None,
                                    v_keep=shared if s.value_mix == "source" else None)
        else:
            ops.unit_kv_write(qkv, ctx.positions, ctx.token_req, table, cache.k, cache.v, s.heads, s.kv_heads, s.head_dim, s.v_dim,
                              s.qk_norm_eps, own_kv=s.own_kv)
        att = ctx.arena.take((n, s.heads * s.v_dim), x.dtype)
        if s.v_dim == s.head_dim and not s.slope_exp and ops.mfma_attention_takes(x.dtype, s.head_dim, cache.k.shape[2]):
            # bfloat16 on the matrix cores: the tile kernels honour chunks, capped scores and the sink
            for plan in launch_plans(ctx, s.heads // s.kv_heads, s.kv_heads, s.head_dim, span=s.chunk):
                ops.attention_mfma(qkv, att, cache.k, cache.v, plan.tiles, table, s.heads, s.kv_heads, s.head_dim, s.softmax_scale,
                                   window=s.window, hp=plan.hp, splits=plan.splits, workspace=plan.workspace, qt=plan.qt, coop=plan.coop,
                                   chunk=s.chunk, cap=s.score_cap, sink=s.sink, sink_logits=self.sink_logits)
        elif not (s.chunk or s.score_cap or s.sink) and ops.wide_attention_takes(x.dtype, s.head_dim, s.v_dim, cache.k.shape[2]):
            # bfloat16, values of another size than the keys or a bias by distance: the two-size matrix-core kernel
            wide_attention(ctx, qkv, att, cache, table, s.heads, s.kv_heads, s.head_dim, s.v_dim, s.softmax_scale, window=s.window,
                           slope_exp=s.slope_exp, sink_logits=self.sink_logits)
        else:
            ops.attention_generic(qkv, att, cache.k, cache.v, ctx.token_req, ctx.positions, table, s.heads, s.kv_heads, s.head_dim,
                                  s.softmax_scale, window=s.window, v_dim=s.v_dim, chunk=s.chunk, cap=s.score_cap, sink=s.sink,
                                  slope_exp=s.slope_exp, sink_logits=self.sink_logits)
        if s.out_gate:
            ops.gate_mul(att, qkv[:, self.gate_at : self.gate_at + s.heads * s.v_dim], out=att)
        if residual is not None and self.out_bias is None:
            return self.wo.into_residual(att, residual, arena=ctx.arena, plain_copy=not ctx.captured)
        y = self.wo(att, out=out if out is not None else ctx.arena.take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        return ops.add_bias(y, self.out_bias) if (self.out_bias is not None and add_out_bias) else y


registry.register("mixer", "attention", Attention)
