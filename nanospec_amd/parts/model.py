"""A model built from a ``ModelSpec``: embedding, the layers in their run order, the last norm and
the output head (reference: model/llama.py:211-286).  Nothing here knows an architecture's name."""

from __future__ import annotations

import math
import sys

import torch

from ..kernels import ops
from ..weights import source as wsource
from . import registry
from .linear import LAYOUTS, LinearWeight
from .needs import PagedNeed, StateNeed


def _build_layers(spec):
    return [registry.build("block", layer, None) for layer in spec.layers]


def wanted_tensors(spec, layers=None) -> dict:
    """Every tensor the model reads from a checkpoint: name -> (shape, role)."""
    layers = layers if layers is not None else _build_layers(spec)
    out = {spec.embed_name: ((spec.vocab_size, spec.hidden), "embedding")}
    pair = getattr(spec, "pair_embedding", None)
    if pair is not None:
        out[pair.name] = ((pair.buckets + 1, spec.hidden), "embedding")
    for layer in layers:
        out.update(layer.wanted())
    passes = getattr(spec, "passes", None)
    if passes is not None:
        out[passes.name] = ((passes.times, spec.hidden), "embedding")
    out.update(registry.build("norm", spec.final_norm, spec.final_norm_name).wanted())
    out[spec.head_name] = ((spec.vocab_size, spec.hidden), "linear")
    return out


class DecoderModel:
    LAST_TOKEN = "last_token"  # model state: the last token that every request has brought so far

    def __init__(self, spec, config=None) -> None:
        self.spec, self.config = spec, config
        self.layers = _build_layers(spec)
        self.final_norm = registry.build("norm", spec.final_norm, spec.final_norm_name)
        self.embed: torch.Tensor | None = None
        self.head: LinearWeight | None = None
        self.dtype = self.device = None
        self._max_positions = "?"  # not asked yet
        # what every entry of the run order keeps in the cache
        self.cache_needs = [self.layers[c.layer].cache_need() if c.cache_from is None else None for c in spec.run_order]
        # the residual stream between the blocks: one tensor in the model's precision, or ``spec.streams`` copies in 32-bit
        forms = {getattr(layer, "stream_form", "single") for layer in self.layers}
        if len(forms) > 1 or (forms == {"streams"}) != bool(spec.streams):
            raise ValueError(f"the blocks carry the residual stream as {sorted(forms)}, the model as {'streams' if spec.streams else 'single'}")
        if spec.streams and not hasattr(self.final_norm, "read_streams"):
            raise ValueError("the last norm cannot read a 32-bit stream (it has no read_streams)")
        self.pair = getattr(spec, "pair_embedding", None)
        if self.pair is not None and not spec.streams:
            raise ValueError("a pair embedding is built for models that carry 32-bit streams")
        self.pair_table: torch.Tensor | None = None
        # a range of layers that runs several times: what each pass adds to the stream in front of it (``LayerCall.enters``)
        self.passes = getattr(spec, "passes", None)
        if self.passes is not None and not spec.streams:
            raise ValueError("passes over a range of layers are built for models that carry 32-bit streams")
        self.pass_rows: torch.Tensor | None = None
        # state of fixed size per request that belongs to no layer: name -> StateNeed (the cache storage keeps a tensor
        # [slots, *shape] for each, zeroed at admission, and the step's context hands them over as ``ctx.model_state``)
        self.state_needs = {self.LAST_TOKEN: StateNeed((1,), torch.int32)} if self.pair is not None else {}
        # buffers that live as long as a step and that layers hand to each other (``ctx.shared``): key -> columns per token
        self.step_buffers: dict[str, int] = {}
        for layer in self.layers:
            for part in getattr(layer, "parts", ()):
                for key, cols in getattr(part, "step_buffers", dict)().items():
                    if self.step_buffers.setdefault(key, cols) != cols:
                        raise ValueError(f"two layers want the step's buffer {key!r} with {self.step_buffers[key]} and {cols} columns")
        self._ones: torch.Tensor | None = None
        # for tests and debugging: called as layer_probe(run-order entry, float32 [tokens, hidden]) with the sum of the
        # streams after every entry (eager steps of models that carry 32-bit streams)
        self.layer_probe = None

    @property
    def graph_safe(self) -> bool:
        return all(layer.graph_safe for layer in self.layers)

    def batch_plans(self) -> list:
        """The batch plans of all layers' parts, one per key (``engine.context``)."""
        plans = {}
        for layer in self.layers:
            for plan in getattr(layer, "batch_plans", list)():
                plans.setdefault(plan.key, plan)
        return list(plans.values())

    def wanted(self) -> dict:
        return wanted_tensors(self.spec, self.layers)

    def load(self, source, dtype: torch.dtype, device, layouts: str = "auto") -> "DecoderModel":
        """Check the source against what the model wants (one error that lists everything wrong), then read
        each tensor once.  A head that is absent is the embedding table if the configuration ties them
        (reference: model/loader.py:62-70).  ``layouts``: "both" keeps every bfloat16 matrix in two layouts
        (``parts.linear.LAYOUTS``), "tiled" only in the re-laid one, "auto" chooses by the memory that is free."""
        spec = self.spec
        full = self.wanted()
        wanted = {k: v[0] for k, v in full.items()}
        wsource.check(source, wanted, optional={spec.head_name} if spec.tie_head else frozenset(), unread_prefixes=spec.unread_prefixes)
        self.dtype, self.device = dtype, torch.device(device)
        if layouts != "auto" and layouts not in LAYOUTS:
            raise ValueError(f"layouts={layouts!r}: use 'auto', 'both' or 'tiled'")
        if layouts == "auto":
            size = torch.finfo(dtype).bits // 8
            linear = sum(size * math.prod(d for d in shape if d is not None) for name, (shape, role) in full.items()
                         if role == "linear" and name != spec.head_name)
            free = torch.cuda.mem_get_info(self.device)[0]
            layouts = "both" if 2.2 * linear + size * 2 * spec.vocab_size * spec.hidden < 0.8 * free else "tiled"
            if layouts == "tiled" and dtype == torch.bfloat16:
                print(f"[nanospec_amd] {linear / 2**30:.0f} GiB of matrices, {free / 2**30:.0f} GiB free: keeping one layout; "
                      "steps of many tokens copy matrices into plain rows first and are slower", file=sys.stderr, flush=True)
        self.layouts = layouts
        get = source.get
        self.embed = get(spec.embed_name).to(device=device, dtype=dtype).contiguous()
        if spec.head_name in source.names():
            self.head = LinearWeight(get(spec.head_name).to(device=device, dtype=dtype).contiguous(), keep_plain=False)
        else:
            self.head = LinearWeight(self.embed, keep_plain=False)  # the embedding table is the head
        for layer in self.layers:
            if getattr(layer, "takes_layouts", False):
                layer.load(get, dtype, device, layouts)
            else:
                layer.load(get, dtype, device)
        self.final_norm.load(get, dtype, device)
        if self.pair is not None:
            self.pair_table = get(self.pair.name).to(device=device, dtype=dtype).contiguous()
        if self.passes is not None:
            self.pass_rows = get(self.passes.name).to(device=device, dtype=dtype).contiguous()
        if spec.streams:
            self._ones = torch.ones(spec.streams, dtype=torch.float32, device=device)
        # whoever runs the model works on a stream of their own: everything that loading enqueued (copies, re-laying of
        # matrices, random draws) is finished before anyone can read it
        torch.cuda.synchronize(self.device)
        return self

    # ------------------------------------------------------------------ positions

    @property
    def max_positions(self) -> int | None:
        """The positions the model's parts can encode; None if nothing bounds them."""
        if self._max_positions == "?":
            limits = [layer.max_positions() for layer in self.layers if hasattr(layer, "max_positions")]
            limits = [n for n in limits if n is not None]
            self._max_positions = min(limits) if limits else None
        return self._max_positions

    def check_positions(self, last_position: int) -> None:
        limit = self.max_positions
        if limit is not None and last_position >= limit:
            raise ValueError(f"position {last_position} is beyond the model's {limit} positions")

    # ------------------------------------------------------------------ one pass over the given tokens

    def forward_hidden(self, ctx, caches) -> tuple[torch.Tensor, torch.Tensor]:
        """Run the tokens of ``ctx`` through every entry of the run order.  -> (resid, delta): the stream
        before the last sum.  ``caches[i]`` is the cache view of run-order entry i (its own or the one
        it reads)."""
        n = ctx.n_tokens
        ctx.shared = {key: ctx.arena.take((n, cols), self.dtype) for key, cols in self.step_buffers.items()}
        if self.spec.streams:
            # copies of the stream in 32-bit, all equal to the embedding's output; blocks update them in place
            resid = ctx.arena.take((n, self.spec.streams, self.spec.hidden), torch.float32)
            if self.pair is not None:
                state = (getattr(ctx, "model_state", None) or {}).get(self.LAST_TOKEN)
                if state is None:
                    raise ValueError("the step's context holds no state for the tokens before its first ones (ctx.model_state)")
                ops.embed_pair_streams(self.embed, self.pair_table, ctx.token_ids, ctx.positions, ctx.token_req, ctx.qo_indptr,
                                       ctx.state_slots, state, resid, self.spec.embed_scale, self.pair.buckets, self.pair.mul_prev,
                                       self.pair.mul_cur)
            else:
                ops.embed_streams(self.embed, ctx.token_ids, resid, scale=self.spec.embed_scale)
            # a block leaves its last sublayer's output unwritten (``ops.PendingWrite``): the next read writes it in passing
            pending = None
            carry = ctx.arena.take((n, self.spec.hidden), self.dtype)
            for i, call in enumerate(self.spec.run_order):
                if call.enters is not None:
                    # a pass starts: what the layer before left unwritten goes into the streams, then the embedding's output
                    # (every pass but the first) and the pass's own row, each added in 32-bit
                    if pending is not None:
                        ops.stream_step(resid, pending)
                        pending = None
                    again = self.passes.add_embedding and call.enters > 0
                    if again and self.pair is not None:
                        raise ops.KernelRefused("a pass that adds the embedding's output again beside a pair embedding is not built")
                    ops.stream_add_rows(resid, self.embed if again else None, ctx.token_ids if again else None, self.pass_rows[call.enters],
                                        scale=self.spec.embed_scale)
                pending = self.layers[call.layer].forward(ctx, resid, pending, caches[i], call.cache_from is None, carry)
                if self.layer_probe is not None:
                    total = torch.empty((n, self.spec.hidden), dtype=torch.float32, device=resid.device)
                    self.final_norm.read_streams(ctx, resid, self._ones, out=ctx.arena.take((n, self.spec.hidden), self.dtype), sum_out=total,
                                                 pending=pending)
                    pending = None
                    self.layer_probe(i, total)
            return resid, pending
        resid = ctx.arena.take((n, self.spec.hidden), self.dtype)
        delta = ctx.arena.take((n, self.spec.hidden), self.dtype)
        ops.embed(self.embed, ctx.token_ids, out=resid, scale=self.spec.embed_scale)
        pending = None
        order = self.spec.run_order
        # buffers for what one block hands to the next (see PreNormBlock.forward)
        sums = ctx.arena.take((n, -(-self.spec.hidden // 16)), torch.float32)
        carry = ctx.arena.take((16 * n * self.spec.hidden,), torch.float32) if 16 < n <= ops.WIDE_TALL_ROWS and self.dtype == torch.bfloat16 else None
        for i, call in enumerate(order):
            layer = self.layers[call.layer]
            if getattr(layer, "links_blocks", False) and i + 1 < len(order):
                # the norm that reads this block's result is the next block's first
                nxt = getattr(self.layers[order[i + 1].layer], "entry_norm", None)
                out = layer.forward(ctx, resid, pending, caches[i], call.cache_from is None, delta, next_norm=nxt, next_sums=sums,
                                    next_carry=carry)
            else:
                if isinstance(pending, (ops.PreNormed, ops.Added)):
                    pending = None  # resid is whole already; a block that does not know the hand-over starts from it
                elif isinstance(pending, ops.PartialSums):
                    pending = ops.reduce_partial(pending, out=delta)
                out = layer.forward(ctx, resid, pending, caches[i], call.cache_from is None, delta)
            pending = out if out is not None else delta
        return resid, pending

    def logits(self, ctx, resid, delta, rows: torch.Tensor) -> torch.Tensor:
        """32-bit logits [len(rows), vocab] at the given token rows: last sum, last norm and head only there
        (reference: model/llama.py:284-286, engine/engine.py:382)."""
        n = rows.numel()
        if self.spec.streams:  # the streams are added up as the last norm reads them
            # (what the last block left unwritten is added for these rows as they are read, and not kept: nobody reads the
            # streams again)
            h = self.final_norm.read_streams(ctx, resid, self._ones, rows=rows, out=ctx.arena.take((n, self.spec.hidden), self.dtype),
                                             pending=delta, store=False)
        else:
            h = self.final_norm.forward(ctx, resid=resid, x=delta, rows=rows, out=ctx.arena.take((n, self.spec.hidden), self.dtype))
        out = self.head(h, out=ctx.arena.take((n, self.spec.vocab_size), torch.float32), out_f32=True, arena=ctx.arena)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap:
            ops.logit_transform(out, self.spec.logit_scale, self.spec.logit_softcap)
        return out
