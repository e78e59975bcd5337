"""RMS norm (reference: model/llama.py:86-95), with the residual sum of the surrounding block fused in."""

from __future__ import annotations

import torch

from ..kernels import ops
from .registry import register


class RMSNorm:
    graph_safe = True
    # y = weight * r / rms(r): linear in 1/rms(r), so a product that follows can apply that factor to its sums and a
    # product that precedes can gather the sum of squares (``parts.linear.IntoResidual``)
    links_products = True

    def __init__(self, spec, name: str) -> None:
        self.spec, self.name = spec, name
        self.weight: torch.Tensor | None = None
        # a weight kept as the factor minus one: the factor is 1 + w, which the kernels form in 32-bit from the stored value (1 + w
        # rounded to bfloat16 would lose most of w)
        self.offset = 1.0 if getattr(spec, "unit_offset", False) else 0.0
        if self.offset:
            self.links_products = False  # the products that fold a norm in multiply by the stored weight

    def wanted(self) -> dict:
        return {self.name: ((self.spec.dim,), "around_zero" if self.offset else "norm")}

    def load(self, get, dtype, device) -> None:
        self.weight = get(self.name).to(device=device, dtype=dtype).contiguous()

    def forward(self, ctx, resid=None, x=None, rows=None, write_resid=False, out=None) -> torch.Tensor:
        if self.offset:
            raise ops.KernelRefused("a norm whose weight is kept as the factor minus one reads a 32-bit stream (blocks of kind 'streams')")
        return ops.rmsnorm(self.weight, self.spec.eps, resid=resid, x=x, rows=rows, write_resid=write_resid, out=out)

    def read_streams(self, ctx, streams: torch.Tensor, coeff: torch.Tensor, rows=None, out=None, sum_out=None, pending=None,
                     store: bool = True) -> torch.Tensor:
        """The norm of one mix of a 32-bit residual stream's copies: u = sum_s coeff[s] streams[:, s]; weight * u / rms(u),
        in the weight's dtype (``streams`` float32 [tokens, S, dim]; see ``parts.block.StreamBlock``).  ``pending``: a
        sublayer's output that is still to be written into the streams (``ops.PendingWrite``); it is written in the same
        pass, before the read (with ``rows`` and ``store`` = False: for those rows only and without keeping it)."""
        return ops.stream_step(streams, pending, coeff, self.weight, self.spec.eps, rows=rows, out=out, sum_out=sum_out, store=store,
                               w_offset=self.offset)

    def behind(self, bias: torch.Tensor | None = None) -> "ops.PostNorm":
        """This norm as the one BEHIND a sublayer, applied to the sublayer's output (plus ``bias``) on its way into a 32-bit
        stream: what ``ops.PendingWrite`` carries."""
        return ops.PostNorm(bias, self.weight, self.spec.eps, self.offset)


class NoNorm:
    """No norm: a sublayer behind it reads the mix of a 32-bit stream's copies itself, rounded to the model's precision."""

    graph_safe = True
    links_products = False
    weight = None

    def __init__(self, spec, name: str) -> None:
        self.spec, self.name = spec, name
        self.dtype: torch.dtype | None = None

    def wanted(self) -> dict:
        return {}

    def load(self, get, dtype, device) -> None:
        self.dtype = dtype

    def forward(self, ctx, resid=None, x=None, rows=None, write_resid=False, out=None) -> torch.Tensor:
        raise ops.KernelRefused("a read without a norm is built for 32-bit streams (blocks of kind 'streams')")

    def read_streams(self, ctx, streams: torch.Tensor, coeff: torch.Tensor, rows=None, out=None, sum_out=None, pending=None,
                     store: bool = True) -> torch.Tensor:
        return ops.stream_step(streams, pending, coeff, None, 0.0, rows=rows, out=out, sum_out=sum_out, store=store, dtype=self.dtype)


register("norm", "rmsnorm", RMSNorm)
register("norm", "none", NoNorm)
