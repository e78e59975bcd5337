"""The pre-norm residual block (reference: model/llama.py:198-208):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x)).

The stream is carried as ``resid`` plus a ``delta`` that has not been added yet, so that every sum is
done inside the norm kernel that follows it (the reference's fused form, model/llama.py:240-254)."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import IntoResidual

class PreNormBlock:
    def __init__(self, spec, prefix: str | None = None) -> None:
        p = spec.prefix if prefix is None else prefix
        self.spec = spec
        under = lambda given, part: p + (given if given is not None else part.kind + ".")
        self.mixer_norm = registry.build("norm", spec.mixer_norm, p + spec.mixer_norm_name)
        self.mixer = registry.build("mixer", spec.mixer, under(spec.mixer_prefix, spec.mixer))
        self.ffn_norm = registry.build("norm", spec.ffn_norm, p + spec.ffn_norm_name)
        self.ffn = registry.build("ffn", spec.ffn, under(spec.ffn_prefix, spec.ffn))
        self.parts = (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.parts)

    def wanted(self) -> dict:
        out = {}
        for p in self.parts:
            out.update(p.wanted())
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        for p in self.parts:
            if getattr(p, "takes_layouts", False):
                p.load(get, dtype, device, layouts)
            else:
                p.load(get, dtype, device)

    takes_layouts = True

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_plans(self) -> list:
        return [plan for p in self.parts for plan in getattr(p, "batch_plans", list)()]

    def max_positions(self) -> int | None:
        """The positions the block's parts can encode; None if nothing bounds them."""
        limits = [p.max_positions() for p in self.parts if hasattr(p, "max_positions")]
        limits = [n for n in limits if n is not None]
        return min(limits) if limits else None

    @property
    def entry_norm(self):
        """The norm that reads what the block before this one left (for blocks that ``links_blocks``)."""
        return self.mixer_norm

    links_blocks = True  # forward takes next_norm, next_sums and next_carry

    def forward(self, ctx, resid, delta, cache, owns_cache, delta_out, next_norm=None, next_sums=None, next_carry=None):
        """``delta``: what the block before left to be added: a tensor (None at the start), a ``PartialSums``, a
        ``PreNormed``, in which case ``resid`` is already whole and the first norm's input comes ready for a product that
        ``links_norms``, or an ``Added`` (``resid`` is whole, nothing else comes with it).  ``next_norm``: the norm that will read this block's result (the next block's first one), if it
        ``links_products``; ``next_sums`` (float32 [tokens, ceil(width / 16)]) and ``next_carry`` (float32, 16 * tokens *
        width, or None): buffers that live as long as the step.
        -> None, with the block's not yet added output in ``delta_out``; or that output in one of the forms of
        ``IntoResidual`` (a tensor is then ``delta_out``)."""
        n = resid.shape[0]
        mark = ctx.arena.mark()
        link = getattr(ctx, "link_norms", False) and resid.dtype == torch.bfloat16
        takes = lambda part: link and getattr(part, "links_norms", lambda rows: False)(n)  # a PreNormed input
        ends = lambda part: link and getattr(part, "ends_in_residual", False)
        lp = lambda norm: link and norm is not None and getattr(norm, "links_products", False) and norm.weight.dtype == resid.dtype
        buf = lambda: ctx.arena.take(resid.shape, resid.dtype)

        # first norm and mixer
        whole = (ops.PreNormed, ops.Added)  # forms in which resid already holds the sum
        if isinstance(delta, whole):
            h = delta if isinstance(delta, ops.PreNormed) and takes(self.mixer) else self.mixer_norm.forward(ctx, resid=resid, out=buf())
        else:
            h = self.mixer_norm.forward(ctx, resid=resid, x=delta, write_resid=delta is not None, out=buf())
        if ends(self.mixer) and lp(self.ffn_norm):
            a = self.mixer.forward(ctx, h, cache, owns_cache, residual=IntoResidual(resid, self.ffn_norm.weight, self.ffn_norm.spec.eps))
        else:
            a = self.mixer.forward(ctx, h, cache, owns_cache, out=buf())

        # second norm and feed-forward
        if isinstance(a, whole):
            h2 = a if isinstance(a, ops.PreNormed) and takes(self.ffn) else self.ffn_norm.forward(ctx, resid=resid, out=buf())
        else:
            h2 = self.ffn_norm.forward(ctx, resid=resid, x=a, write_resid=True, out=buf())
        if ends(self.ffn) and lp(next_norm) and next_sums is not None:
            # what the next block reads must outlive this block's scratch
            out = self.ffn.forward(ctx, h2, residual=IntoResidual(resid, next_norm.weight, next_norm.spec.eps, delta_out, next_sums,
                                                                 next_carry, outlives=True))
            ctx.arena.release(mark)
            return out
        self.ffn.forward(ctx, h2, out=delta_out)
        ctx.arena.release(mark)
        return None


registry.register("block", "prenorm", PreNormBlock)


class StreamBlock:
    """A pre-norm block over a 32-bit residual stream of S parallel copies x [tokens, S, width] (hyper-connections; S = 1
    without mixing tensors is the plain residual with its sum in 32-bit).  For each sublayer (mixer, then feed-forward
    if there is one):
        u = sum_s in[s] x_s;  y = sublayer(norm(u));  x_t <- sum_s mix[s, t] x_s + mult * out[t] * y   for all t at once
    The read is one kernel with the norm (``norm.read_streams``), the write another; sublayers compute in the model's
    precision and never see the streams."""

    stream_form = "streams"  # what ``forward`` takes as ``resid``: float32 [tokens, S, width], updated in place

    def __init__(self, spec, prefix: str | None = None) -> None:
        p = spec.prefix if prefix is None else prefix
        self.spec, self.prefix = spec, p
        self.copies = max(1, spec.streams)
        self.mixer_norm = registry.build("norm", spec.mixer_norm, p + spec.mixer_norm_name)
        self.mixer = registry.build("mixer", spec.mixer, p + spec.mixer_prefix)
        self.ffn = registry.build("ffn", spec.ffn, p + spec.ffn_prefix) if spec.ffn is not None else None
        self.ffn_norm = registry.build("norm", spec.ffn_norm, p + spec.ffn_norm_name) if spec.ffn is not None else None
        # norms behind the sublayers (x <- x + post_norm(sublayer(norm(x)))), applied as the output is written into the streams
        post = lambda given, name: registry.build("norm", given, p + name) if given is not None else None
        self.mixer_post = post(getattr(spec, "mixer_post_norm", None), getattr(spec, "mixer_post_norm_name", ""))
        self.ffn_post = post(getattr(spec, "ffn_post_norm", None), getattr(spec, "ffn_post_norm_name", "")) if spec.ffn is not None else None
        # a third sublayer behind the feed-forward (a part of the "ffn" role: it sees the step's context and its input)
        extra = getattr(spec, "extra", None)
        self.extra = registry.build("ffn", extra, p + spec.extra_prefix) if extra is not None else None
        self.extra_norm = registry.build("norm", spec.extra_norm, p + spec.extra_norm_name) if extra is not None else None
        self.extra_post = post(spec.extra_post_norm, spec.extra_post_norm_name) if extra is not None else None
        self.parts = tuple(x for x in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post,
                                       self.extra_norm, self.extra, self.extra_post) if x is not None)
        self.dtype = None
        for norm in (self.mixer_norm, self.ffn_norm, self.extra_norm):
            if norm is not None and not hasattr(norm, "read_streams"):
                raise ValueError(f"a norm of kind {norm.spec.kind!r} cannot read a 32-bit stream (it has no read_streams)")
        for norm in (self.mixer_post, self.ffn_post, self.extra_post):
            if norm is not None and not hasattr(norm, "behind"):
                raise ValueError(f"a norm of kind {norm.spec.kind!r} cannot stand behind a sublayer of a 32-bit stream (it has no behind)")
        self._hc: list = []  # per sublayer: (in [S], mix [S, S], mult * out [S]) float32 on the device

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.parts)

    def _hc_names(self):
        if self.extra is not None:
            raise ValueError("hyper-connected streams with a third sublayer are not built")
        return [self.prefix + q + t for q in self.spec.hc_names[: 2 if self.ffn is not None else 1] for t in ("in", "out", "mix")]

    def wanted(self) -> dict:
        out = {}
        for p in self.parts:
            out.update(p.wanted())
        if self.spec.streams:
            S = self.copies
            # laws under which random streams neither die out nor blow up: read about the mean, write about evenly,
            # mix close to the identity
            law = lambda mean, std: (lambda shape, gen: mean + std * torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device))
            for name in self._hc_names():
                if name.endswith("mix"):
                    out[name] = ((S, S), lambda shape, gen: torch.eye(S, device=gen.device) * 0.9 + 0.1 / S
                                 + 0.05 * torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device))
                else:
                    out[name] = ((S,), law(1.0 / S if name.endswith("in") else 1.0, 0.1))
        return out

    takes_layouts = True

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        for p in self.parts:
            if getattr(p, "takes_layouts", False):
                p.load(get, dtype, device, layouts)
            else:
                p.load(get, dtype, device)
        S, m = self.copies, float(self.spec.mult)
        self.dtype = dtype
        self._hc = []
        f32 = lambda t: t.to(device=device, dtype=torch.float32).contiguous()
        for q in range(3 if self.extra is not None else (2 if self.ffn is not None else 1)):
            if self.spec.streams:
                pre = self.prefix + self.spec.hc_names[q]
                self._hc.append((f32(get(pre + "in")), f32(get(pre + "mix")), f32(get(pre + "out")) * m))
            else:
                self._hc.append((torch.ones(1, device=device), torch.ones((1, 1), device=device), torch.full((1,), m, device=device)))

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_plans(self) -> list:
        return [plan for p in self.parts for plan in getattr(p, "batch_plans", list)()]

    def max_positions(self) -> int | None:
        limits = [p.max_positions() for p in self.parts if hasattr(p, "max_positions")]
        limits = [n for n in limits if n is not None]
        return min(limits) if limits else None

    @staticmethod
    def _sublayer(part, post_norm, ctx, h, *cache, out):
        """Run a sublayer.  -> (its output, what the output passes on its way into the streams: an ``ops.PostNorm`` or None).
        A sublayer whose last projection has a bias (``out_bias``) leaves it to that place, where it is added in 32-bit."""
        bias = getattr(part, "out_bias", None)
        if bias is not None:
            y = part.forward(ctx, h, *cache, out=out, add_out_bias=False)
        else:
            y = part.forward(ctx, h, *cache, out=out)
        if post_norm is not None:
            return y, post_norm.behind(bias)
        return y, (ops.PostNorm(bias=bias) if bias is not None else None)

    def forward(self, ctx, resid, delta, cache, owns_cache, delta_out):
        """``resid``: float32 [tokens, S, width], updated in place.  ``delta``: None, or the ``ops.PendingWrite`` that the block
        before left (its last sublayer's output, not yet in the streams): it is written by the kernel that reads for this
        block's mixer.  ``delta_out``: None, or a buffer [tokens, width] in the model's dtype that outlives the block: the
        last sublayer's output is then left there, unwritten, and returned as a ``PendingWrite``.  (``delta`` may lie in the
        same buffer: it is used up before anything is put there.)"""
        n, S, W = resid.shape
        if S != self.copies:
            raise ValueError(f"the block is built for {self.copies} streams, the model carries {S}")
        mark = ctx.arena.mark()
        dtype = self.dtype
        a, mix, gain = self._hc[0]
        h = self.mixer_norm.read_streams(ctx, resid, a, out=ctx.arena.take((n, W), dtype), pending=delta)
        later = [(self.ffn_norm, self.ffn, self.ffn_post, 1)] if self.ffn is not None else []
        if self.extra is not None:
            later.append((self.extra_norm, self.extra, self.extra_post, 2))
        y, post = self._sublayer(self.mixer, self.mixer_post, ctx, h, cache, owns_cache,
                                 out=delta_out if not later and delta_out is not None else ctx.arena.take((n, W), dtype))
        pending = ops.PendingWrite(y, mix, gain, post)
        for at, (norm, part, post_norm, q) in enumerate(later):
            a, mix, gain = self._hc[q]
            h = norm.read_streams(ctx, resid, a, out=h, pending=pending)
            y, post = self._sublayer(part, post_norm, ctx, h, out=delta_out if (delta_out is not None and at == len(later) - 1) else y)
            pending = ops.PendingWrite(y, mix, gain, post)
        if delta_out is None:
            ops.stream_step(resid, pending)
            pending = None
        ctx.arena.release(mark)
        return pending


registry.register("block", "streams", StreamBlock)
