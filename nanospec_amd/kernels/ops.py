"""Python faces of the HIP kernels.  Each function checks on the host that the operands have the
shapes, strides and types the kernel and its grid assume, then launches on the current stream.

A size a kernel does not take raises ``KernelRefused`` with the reason; nothing is computed
elsewhere instead.  Tensors are torch tensors on the GPU; only their addresses cross into C.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_size_t, c_uint32, c_void_p

import torch

from . import build

F32, BF16 = 0, 1


class KernelRefused(Exception):
    """A kernel was asked for a size or type it does not take."""


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelRefused(f"kernels take float32 or bfloat16 tensors, not {t.dtype}")


def _ptr(t):
    return c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # the handle without building a Stream object
_device_index = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream's handle; asked for at every launch, so by the shortest way that torch offers."""
    if _raw_stream is not None and _device_index is not None:
        return c_void_p(_raw_stream(_device_index()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelRefused("kernels run on GPU tensors only; there is no CPU path")


def _check(code: int, what: str) -> None:
    if code != 0:
        lib = build.core()
        lib.ns_error_string.restype = ctypes.c_char_p
        msg = lib.ns_error_string(c_int(code)).decode()
        raise KernelRefused(f"{what}: {msg} (code {code})")


_units: dict[int, int] = {}


def compute_units(device) -> int:
    """Compute units of the GPU a tensor lives on (256 on an MI355X); launch heuristics count workgroups against it."""
    index = torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if index not in _units:
        _units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _units[index]


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelRefused(f"{name} must be a contiguous int32 tensor")
    return t


# ------------------------------------------------------------------------------------------------ elementwise


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None, scale: float = 1.0) -> torch.Tensor:
    """out[i] = table[ids[i]] (times ``scale``, in 32-bit, rounded once).  ``ids`` int32; the caller has checked 0 <= id < vocab."""
    _gpu(table, ids)
    _i32(ids, "ids")
    n, hidden = ids.numel(), table.shape[1]
    if out is None:
        out = torch.empty((n, hidden), dtype=table.dtype, device=table.device)
    if not table.is_contiguous() or out.shape != (n, hidden) or out.dtype != table.dtype or not out.is_contiguous():
        raise KernelRefused("embed: table and out must be contiguous [*, hidden] of one dtype")
    _check(build.core().ns_embed(_ptr(out), _ptr(table), _ptr(ids), c_int(n), c_int(hidden), c_float(scale), c_int(_dtype_code(table)),
                                 _stream()), "embed")
    return out


def logit_transform(logits: torch.Tensor, scale: float = 1.0, softcap: float = 0.0) -> torch.Tensor:
    """32-bit logits in place: times ``scale``; with ``softcap`` > 0 then softcap * tanh(logit / softcap)."""
    _gpu(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1 or softcap < 0:
        raise KernelRefused("logit_transform takes float32 [rows, vocab] and a cap that is not negative")
    _check(build.core().ns_logit_transform(_ptr(logits), c_int(logits.shape[0]), c_int(logits.shape[1]), c_int(logits.stride(0)),
                                           c_float(scale), c_float(softcap), _stream()), "logit_transform")
    return logits


class PartialSums:
    """A product whose K was cut into ranges that have not been added up yet (``linear_wide(..., defer=True)``):
    ``ws`` holds float32 [ksplit, rows, n].  ``rmsnorm`` adds them while it reads them; ``reduce_partial`` makes the tensor."""

    def __init__(self, ws: torch.Tensor, ksplit: int, rows: int, n: int, dtype: torch.dtype) -> None:
        self.ws, self.ksplit, self.rows, self.n, self.dtype = ws, ksplit, rows, n, dtype
        self.shape = (rows, n)


def reduce_partial(p: PartialSums, out: torch.Tensor | None = None) -> torch.Tensor:
    """The sum of the ranges, in order, rounded to the product's dtype."""
    _gpu(p.ws, out)
    if out is None:
        out = torch.empty((p.rows, p.n), dtype=p.dtype, device=p.ws.device)
    if out.shape != (p.rows, p.n) or out.stride(1) != 1 or out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelRefused("reduce_partial: out has the wrong shape or dtype")
    _check(build.core().ns_wide_reduce(_ptr(out), _ptr(p.ws), c_int(p.rows), c_int(p.n), c_int(out.stride(0)), c_int(p.ksplit),
                                       c_int(1 if out.dtype == torch.float32 else 0), _stream()), "reduce_partial")
    return out


def rmsnorm(weight: torch.Tensor, eps: float, resid: torch.Tensor | None = None, x: "torch.Tensor | PartialSums | None" = None,
            rows: torch.Tensor | None = None, write_resid: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[i] = weight * norm(resid[r] + x[r]) with r = rows[i] (or i).  With ``write_resid`` the sum
    is also stored back into ``resid`` (not with ``rows``).  ``x`` may be a ``PartialSums``."""
    if isinstance(x, PartialSums):
        p, dim = x, weight.numel()
        ok = (weight.dtype == torch.bfloat16 and p.dtype == torch.bfloat16 and p.n == dim and dim % 4 == 0 and dim <= 16384
              and (resid is None or (resid.shape == (p.rows, dim) and resid.is_contiguous() and resid.dtype == weight.dtype)))
        if not ok:
            x = reduce_partial(p)
        else:
            _gpu(weight, resid, rows, p.ws)
            if rows is not None:
                _i32(rows, "rows")
            n = rows.numel() if rows is not None else p.rows
            if out is None:
                out = torch.empty((n, dim), dtype=weight.dtype, device=weight.device)
            if out.shape != (n, dim) or not out.is_contiguous() or out.dtype != weight.dtype:
                raise KernelRefused("rmsnorm: out has the wrong shape")
            _check(build.core().ns_rmsnorm_partial(_ptr(out), _ptr(resid), _ptr(p.ws), c_size_t(p.rows * dim), c_int(p.ksplit), _ptr(weight),
                                                   _ptr(rows), c_int(n), c_int(dim), c_float(eps), c_int(1 if write_resid else 0),
                                                   c_int(_dtype_code(weight)), _stream()), "rmsnorm")
            return out
    src = resid if resid is not None else x
    if src is None:
        raise KernelRefused("rmsnorm needs resid or x")
    _gpu(weight, resid, x, rows)
    dim = weight.numel()
    for t in (resid, x):
        if t is not None and (t.dim() != 2 or t.shape[1] != dim or not t.is_contiguous() or t.dtype != weight.dtype):
            raise KernelRefused(f"rmsnorm: operands must be contiguous [*, {dim}] of the weight's dtype")
    if resid is not None and x is not None and resid.shape != x.shape:
        raise KernelRefused("rmsnorm: resid and x differ in shape")
    if rows is not None:
        _i32(rows, "rows")
    n = rows.numel() if rows is not None else src.shape[0]
    if out is None:
        out = torch.empty((n, dim), dtype=weight.dtype, device=weight.device)
    if out.shape != (n, dim) or not out.is_contiguous() or out.dtype != weight.dtype:
        raise KernelRefused("rmsnorm: out has the wrong shape")
    _check(build.core().ns_rmsnorm(_ptr(out), _ptr(resid), _ptr(x), _ptr(weight), _ptr(rows), c_int(n), c_int(dim), c_float(eps),
                                   c_int(1 if write_resid else 0), c_int(_dtype_code(weight)), _stream()), "rmsnorm")
    return out


def _check_pages(block_table, k_cache, v_cache, kv_heads: int, head_dim: int, dtype, what: str) -> int:
    """What the kernels that write keys and values into pages assume of the pools and the block table.  -> page size.
    (Positions and request indices inside the batch are the batch builder's: a kernel computes
    ``block_table[token_req[t]][position // page]`` without asking whether the table is that wide.)"""
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelRefused(f"{what}: key pages are [pages, kv_heads, page, head_dim], value pages [pages, kv_heads, head_dim, page]")
    page = k_cache.shape[2]
    if (k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, head_dim, page)
            or k_cache.dtype != dtype or v_cache.dtype != dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
        raise KernelRefused(f"{what}: cache pages do not fit heads, head size or dtype")
    _i32(block_table, "block_table")
    if block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelRefused(f"{what}: block_table is int32 [requests, pages] with unit stride along a row")
    return page


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, token_req: torch.Tensor, block_table: torch.Tensor,
                  inv_freq: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, heads: int, kv_heads: int,
                  head_dim: int, rotary_dim: int, write_kv: bool = True, interleaved: bool = False, factor: float = 1.0) -> None:
    """Rotate q in place inside ``qkv`` [N, (heads + 2 kv_heads) * head_dim]; rotate k and write k and v of
    every token into the pages ``block_table[token_req[t], position // page]``.
    k_cache [pages, kv_heads, page, head_dim]; v_cache [pages, kv_heads, head_dim, page].
    ``interleaved``: pair j of the rotary part is channels (2j, 2j + 1) instead of (j, j + rotary_dim / 2); ``factor``
    multiplies cosine and sine."""
    _gpu(qkv, positions, token_req, block_table, inv_freq, k_cache, v_cache)
    n = positions.numel()
    width = (heads + 2 * kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[0] != n or qkv.shape[1] != width or qkv.stride(1) != 1:
        raise KernelRefused(f"rope_kv_write: qkv must be [{n}, {width}]")
    _i32(positions, "positions"), _i32(token_req, "token_req")
    if token_req.numel() != n:
        raise KernelRefused("rope_kv_write: token_req is per token")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(1, rotary_dim // 2):
        raise KernelRefused("rope_kv_write: inv_freq must hold rotary_dim/2 float32 values")
    page = _check_pages(block_table, k_cache, v_cache, kv_heads, head_dim, qkv.dtype, "rope_kv_write")
    _check(build.core().ns_rope_kv_write(_ptr(qkv), c_int(qkv.stride(0)), _ptr(positions), _ptr(token_req), _ptr(block_table),
                                         c_int(block_table.stride(0)), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), c_int(n),
                                         c_int(heads), c_int(kv_heads), c_int(head_dim), c_int(rotary_dim), c_int(1 if interleaved else 0),
                                         c_float(factor), c_int(page), c_int(1 if write_kv else 0), c_int(_dtype_code(qkv)), _stream()),
           "rope_kv_write")


def silu_mul(gu: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[n, i] = silu(gu[n, i]) * gu[n, I + i] for gu [N, 2 I]."""
    _gpu(gu)
    n, two_i = gu.shape
    inter = two_i // 2
    if two_i % 2 or not gu.is_contiguous():
        raise KernelRefused("silu_mul: gu must be contiguous [N, 2 I]")
    if out is None:
        out = torch.empty((n, inter), dtype=gu.dtype, device=gu.device)
    _check(build.core().ns_silu_mul(_ptr(out), _ptr(gu), c_int(n), c_int(inter), c_int(_dtype_code(gu)), _stream()), "silu_mul")
    return out


def fill_u32(t: torch.Tensor, value: int = 0) -> None:
    """Set every 32-bit word of ``t`` (a kernel, so that it may be part of a captured graph)."""
    _gpu(t)
    nbytes = t.numel() * t.element_size()
    if nbytes % 4 or not t.is_contiguous():
        raise KernelRefused("fill_u32: the tensor must be contiguous and a whole number of 32-bit words")
    _check(build.core().ns_fill_u32(_ptr(t), c_uint32(value), c_size_t(nbytes // 4), _stream()), "fill_u32")


def scatter_i32(dst: torch.Tensor, dst_idx: torch.Tensor, src: torch.Tensor, src_idx: torch.Tensor) -> None:
    """dst[dst_idx[i]] = src[src_idx[i]] for int32 tensors on the GPU (indices are trusted: the caller built them)."""
    _gpu(dst, dst_idx, src, src_idx)
    for name, t in (("dst", dst), ("dst_idx", dst_idx), ("src", src), ("src_idx", src_idx)):
        _i32(t, name)
    if dst_idx.numel() != src_idx.numel():
        raise KernelRefused("scatter_i32: one source index per destination index")
    _check(build.core().ns_scatter_i32(_ptr(dst), _ptr(dst_idx), _ptr(src), _ptr(src_idx), c_int(dst_idx.numel()), _stream()), "scatter_i32")


# ------------------------------------------------------------------------------------------------ matrix products


def _check_linear(x, w, out, out_f32):
    _gpu(x, w, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or not w.is_contiguous() or x.dtype != w.dtype:
        raise KernelRefused(f"linear: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit (w is [out, in], one dtype)")
    m, n = x.shape[0], w.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    if out is None:
        out = torch.empty((m, n), dtype=want, device=x.device)
    if out.shape != (m, n) or out.dtype != want or out.stride(1) != 1:
        raise KernelRefused("linear: out has the wrong shape or dtype")
    return out


def linear_generic(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None, out_f32: bool = False) -> torch.Tensor:
    """x @ w.T with the plain tiled kernel: any sizes, float32 or bfloat16, 32-bit accumulation in a fixed order."""
    out = _check_linear(x, w, out, out_f32)
    m, k = x.shape
    _check(build.core().ns_gemm_generic(_ptr(out), _ptr(x), _ptr(w), c_int(m), c_int(w.shape[0]), c_int(k), c_int(x.stride(0)),
                                        c_int(out.stride(0)), c_int(1 if out_f32 else 0), c_int(_dtype_code(x)), _stream()), "linear_generic")
    return out


SKINNY_MAX_ROWS = 64
WIDE_TALL_ROWS = 128  # ``linear_wide`` with one matrix and one row tile per wave takes this many rows


class TiledWeight:
    """A bfloat16 weight matrix [N, K] re-laid for the streaming matrix-core kernel:
    wt[rt][kt][i][lane = 16 g + r][e] = w[16 rt + r][128 kt + 32 g + 8 i + e], rows padded to a multiple of 16 and
    k to a multiple of 128 with zeros, so that every load of a wave is one contiguous kilobyte."""

    def __init__(self, w: torch.Tensor, row_order: torch.Tensor | None = None) -> None:
        """``row_order``: the rows of ``w`` in the order in which they are laid out (a permutation), for kernels whose
        epilogue wants particular rows together in a tile."""
        if w.dtype != torch.bfloat16 or w.dim() != 2 or not w.is_cuda:
            raise KernelRefused("TiledWeight takes a bfloat16 matrix on the GPU")
        if row_order is not None:
            w = w[row_order.to(w.device)]
        self.n, self.k = w.shape
        n_pad, k_pad = -(-self.n // 16) * 16, -(-self.k // 128) * 128
        if (n_pad, k_pad) != (self.n, self.k):
            wp = torch.zeros((n_pad, k_pad), dtype=w.dtype, device=w.device)
            wp[: self.n, : self.k] = w
        else:
            wp = w
        # (rt, r, kt, g, i, e) -> (rt, kt, i, g, r, e)
        self.data = wp.view(n_pad // 16, 16, k_pad // 128, 4, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous()

    def rows(self, start: int, stop: int) -> "TiledWeight":
        """The sub-matrix of rows [start, stop); both must be multiples of 16 (or stop the last row)."""
        if start % 16 or (stop % 16 and stop != self.n):
            raise KernelRefused("row slices of a tiled weight start and end at multiples of 16")
        out = object.__new__(TiledWeight)
        out.n, out.k = stop - start, self.k
        out.data = self.data[start // 16 : -(-stop // 16)]
        return out


def untile(w: TiledWeight, out: torch.Tensor, k0: int = 0, k1: int | None = None) -> torch.Tensor:
    """Columns ``k0`` to ``k1`` (all by default; ``k0`` a multiple of 128, ``k1`` one or the last column) of the matrix of
    ``w`` in plain rows, into ``out`` [n, k1 - k0] (bfloat16, unit stride along a row): what a library product over many
    rows reads, made for the one product where only the re-laid copy is kept."""
    _gpu(out)
    k1 = w.k if k1 is None else k1
    if (out.dtype != torch.bfloat16 or out.dim() != 2 or out.shape != (w.n, k1 - k0) or out.stride(1) != 1 or out.stride(0) % 8
            or out.data_ptr() % 16 or w.k % 8):
        raise KernelRefused(f"untile: out must be bfloat16 [{w.n}, {k1 - k0}] with rows a multiple of 8 elements apart, 16-byte "
                            f"aligned, and k a multiple of 8")
    if not 0 <= k0 < k1 <= w.k or k0 % 128 or (k1 % 128 and k1 != w.k):
        raise KernelRefused("untile: the columns start at a multiple of 128 and end at one or at the last column")
    _check(build.core().ns_untile_bf16(_ptr(out), _ptr(w.data), c_int(w.n), c_int(w.k), c_int(k0), c_int(k1), c_int(out.stride(0)),
                                       _stream()), "untile")
    return out


def tiled_takes(x: torch.Tensor, k: int, max_rows: int = SKINNY_MAX_ROWS) -> bool:
    return (x.dtype == torch.bfloat16 and x.shape[0] <= max_rows and k % 8 == 0 and x.stride(0) % 8 == 0
            and x.stride(1) == 1 and x.data_ptr() % 16 == 0)


class PreNormed:
    """The input of an RMS norm's consumer when the norm has no kernel of its own: ``x`` = r * weight [rows, dim] in bfloat16
    (r the rows to normalise), and ``ssq`` [rows, parts], float32, whose sum over parts is each row's sum of r^2.  The
    consumer multiplies its sums by rsqrt(sum / dim + eps): y = w * r / rms(r) is linear in 1/rms(r).  Made by
    ``linear_resid_norm``; taken by ``linear_tiled`` and ``linear_qkv_rope`` for at most 16 rows."""

    def __init__(self, x: torch.Tensor, ssq: torch.Tensor, dim: int, eps: float) -> None:
        self.x, self.ssq, self.dim, self.eps = x, ssq, dim, eps
        self.shape, self.dtype = x.shape, x.dtype


class Added:
    """What a part returns instead of its output when it has already added that output to the residual stream in place
    (a library product with the stream as its addend): nothing is left to add and no statistics come with it."""


def _prenorm_args(pre: "PreNormed | None", m: int, what: str):
    if pre is None:
        return c_void_p(None), c_int(0), c_int(0), c_float(0.0)
    if (pre.ssq.dtype != torch.float32 or pre.ssq.dim() != 2 or pre.ssq.shape[0] != m or not pre.ssq.is_contiguous() or m > 16
            or not pre.ssq.is_cuda):
        raise KernelRefused(f"{what}: the sums of squares must be float32 [rows, parts] for at most 16 rows")
    return _ptr(pre.ssq), c_int(pre.ssq.shape[1]), c_int(pre.dim), c_float(pre.eps)


GATED_HALF_ROWS = 4  # up to this many rows the gated product runs half a row tile of each matrix per workgroup (with more,
#                      reading x in twice as many workgroups costs what the even spread gains)


def linear_tiled(x: "torch.Tensor | PreNormed", w: TiledWeight, w2: TiledWeight | None = None, out: torch.Tensor | None = None,
                 out_f32: bool = False, waves: int = 0, halves: bool | None = None, act: str | None = None,
                 bias: torch.Tensor | None = None, bias2: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 x @ w.T for at most 64 rows from a tiled weight; with ``w2``: silu(x @ w.T) * (x @ w2.T).  ``bias`` (and, with
    ``w2``, ``bias2``): bfloat16 [N], added to the 32-bit sums before anything else happens to them.  ``x`` may be a
    ``PreNormed`` (at most 16 rows).  ``halves`` (with ``w2``, at most 16 rows): a workgroup takes 8 rows of each matrix
    instead of 16, which spreads a number of row tiles that is no multiple of the compute units evenly; None: by rows.
    ``act`` (one of ``ACTIVATIONS``, not with ``w2`` or 32-bit results): the activation of the result, which is rounded to
    bfloat16 first, so that the values are those of ``activation`` after this product."""
    if act is not None and (w2 is not None or out_f32 or act not in ACTIVATIONS):
        raise KernelRefused("linear_tiled: an activation goes with one matrix, a bfloat16 result and a known name")
    pre = x if isinstance(x, PreNormed) else None
    if pre is not None:
        x = pre.x
    _gpu(x, out)
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k):
        raise KernelRefused(f"linear_tiled takes bfloat16 x [rows <= {SKINNY_MAX_ROWS}, {w.k}] with an inner size that is a "
                            f"multiple of 8; got {tuple(x.shape)} {x.dtype}")
    m = x.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    if out is None:
        out = torch.empty((m, w.n), dtype=want, device=x.device)
    if out.shape != (m, w.n) or out.dtype != want or out.stride(1) != 1:
        raise KernelRefused("linear_tiled: out has the wrong shape or dtype")
    if w2 is not None and (w2.n != w.n or w2.k != w.k):
        raise KernelRefused("linear_tiled: w2 must match w")
    for b in (bias, bias2):
        if b is not None and (not b.is_cuda or b.shape != (w.n,) or b.dtype != torch.bfloat16 or not b.is_contiguous()):
            raise KernelRefused(f"linear_tiled: a bias is bfloat16 [{w.n}]")
    if bias2 is not None and w2 is None:
        raise KernelRefused("linear_tiled: a second bias goes with a second matrix")
    if waves == 0:  # with more than 8 rows eight waves were never behind four at the shapes measured
        waves = 8 if w.k >= 8192 or ((w.n // 16 < 512 or m > 8) and w.k >= 2048) else 4
    if halves is None:  # (with 3 or 4 rows only where whole row tiles would not spread evenly over 256 compute units)
        halves = m <= 2 or (m <= GATED_HALF_ROWS and -(-w.n // 16) % 256 != 0)
    epi = (5 if act is not None else 0) if w2 is None else (4 if halves and m <= 16 and not out_f32 else 1)
    _check(build.core().ns_gemm_tiled_bf16(_ptr(out), _ptr(x), _ptr(w.data), _ptr(w2.data if w2 is not None else None), c_int(m),
                                           c_int(w.n), c_int(w.k), c_int(x.stride(0)), c_int(out.stride(0)),
                                           c_int(epi), c_int(1 if out_f32 else 0), c_int(waves),
                                           *_prenorm_args(pre, m, "linear_tiled"), c_int(ACTIVATIONS[act] if act is not None else 0),
                                           _ptr(bias), _ptr(bias2), _stream()),
           "linear_tiled")
    return out


def linear_resid_norm(x: torch.Tensor, w: TiledWeight, resid: torch.Tensor, next_weight: torch.Tensor, eps: float,
                      x_next: torch.Tensor | None = None, ssq: torch.Tensor | None = None, waves: int = 0) -> PreNormed:
    """A block's contribution to the residual stream, for at most 16 rows: resid += x @ w.T in place (the product and
    the sum rounded to bfloat16 in turn, as separate kernels would), and what the RMS norm that follows needs from it:
    -> PreNormed(resid * next_weight, per-workgroup sums of resid^2)."""
    _gpu(x, resid, next_weight, x_next, ssq)
    m = x.shape[0]
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k) or m > 16:
        raise KernelRefused(f"linear_resid_norm takes at most 16 bfloat16 rows of {w.k} values; got {tuple(x.shape)} {x.dtype}")
    if resid.shape != (m, w.n) or resid.dtype != torch.bfloat16 or resid.stride(1) != 1:
        raise KernelRefused("linear_resid_norm: resid must be bfloat16 [rows, out features]")
    if next_weight.shape != (w.n,) or next_weight.dtype != torch.bfloat16 or not next_weight.is_contiguous():
        raise KernelRefused("linear_resid_norm: the next norm's weight must be bfloat16 [out features]")
    parts = -(-w.n // 16)
    if x_next is None:
        x_next = torch.empty_like(resid)
    if ssq is None:
        ssq = torch.empty((m, parts), dtype=torch.float32, device=x.device)
    if (x_next.shape != resid.shape or x_next.dtype != resid.dtype or x_next.stride() != resid.stride()
            or ssq.shape != (m, parts) or ssq.dtype != torch.float32 or not ssq.is_contiguous()):
        raise KernelRefused("linear_resid_norm: x_next must be laid out like resid, ssq float32 [rows, ceil(out features / 16)]")
    if waves == 0:
        waves = 8 if w.k >= 8192 or (w.n // 16 < 512 and w.k >= 2048) else 4
    _check(build.core().ns_gemm_resid_norm_bf16(_ptr(resid), _ptr(x_next), _ptr(ssq), _ptr(next_weight), _ptr(x), _ptr(w.data),
                                                c_int(m), c_int(w.n), c_int(w.k), c_int(x.stride(0)), c_int(resid.stride(0)),
                                                c_int(waves), _stream()), "linear_resid_norm")
    return PreNormed(x_next, ssq, w.n, eps)


def _wide_cost(tiles: int, per_group: int, ksplit: int, k_tiles: int, units: int) -> int:
    """What the busiest compute unit streams, in row tiles times k tiles: a product of few rows takes as long as that."""
    groups = -(-tiles // per_group)
    return -(-groups * ksplit // units) * per_group * -(-k_tiles // ksplit)


def wide_plan(n: int, k: int, rows: int = SKINNY_MAX_ROWS, units: int | None = None) -> tuple[int, int]:
    """(ranges K is cut into, 16-row tiles per wave) of ``linear_wide``: two tiles per wave when there are rows enough
    (and at most 64 rows of x), then as many ranges as give every compute unit about one workgroup, with at least four k
    tiles of 128 per range (more, shorter ranges were measured slower once the kernel that joins them is counted: 37 against
    31 us for the down-projection of the 8B shape at 64 rows with 10 and with 4 ranges).  With one tile per wave and up to
    64 rows a workgroup may have three waves instead of four (``wide_waves``); the ranges are chosen for whichever of the
    two leaves the busiest compute unit the least to stream.  ``units``: the GPU's compute units (the current device's by
    default)."""
    units = units or compute_units(torch.cuda.current_device())
    nt = 2 if n >= 8192 and rows <= SKINNY_MAX_ROWS else 1
    k_tiles = -(-k // 128)
    most = max(1, min(16, k_tiles // 4))
    ranges = lambda per_group: max(1, min(most, round(units / -(-n // (16 * per_group)))))
    if nt != 1 or rows > SKINNY_MAX_ROWS:
        return ranges(4 * nt), nt
    tiles = -(-n // 16)
    four, three = ranges(4), ranges(3)
    return (three if _wide_cost(tiles, 3, three, k_tiles, units) < _wide_cost(tiles, 4, four, k_tiles, units) else four), nt


def wide_waves(n: int, k: int, rows: int, ksplit: int, nt: int, gated: bool = False, units: int | None = None) -> tuple[int, bool]:
    """(waves per workgroup, by half tiles) of ``linear_wide`` for a product cut as given: what deals the row tiles most
    evenly to the compute units.  One matrix, one tile per wave, up to 64 rows: three waves instead of four where that
    leaves the busiest unit less.  Gate and up in one range: four waves of a whole tile of each (8 half tiles a workgroup),
    seven or four waves of half a tile of each (7 or 4 a workgroup); at the 8B shape 1,792 half tiles are 7 for each of 256
    units instead of 8 for each of 224 (42 against 51 us at 64 rows; the 1B shape's 1,024 as 4 for each: 17 against 25 us)."""
    units = units or compute_units(torch.cuda.current_device())
    if nt != 1 or (rows > SKINNY_MAX_ROWS and not gated):
        return 4, False
    tiles, k_tiles = -(-n // 16), -(-k // 128)
    if gated:
        if rows > SKINNY_MAX_ROWS:  # 65 to 128 rows: only half tiles hold the sums of both matrices
            return (7 if -(-(-(-2 * tiles // 7)) // units) * 7 <= -(-(-(-2 * tiles // 4)) // units) * 4 else 4), ksplit == 1
        if ksplit != 1 or -(-tiles // 4) >= units:  # (whole tiles fill the GPU: measured level or ahead, 163 against 166 us at the 70B shape)
            return 4, False
        options = [(-(-(-(-tiles // 4)) // units) * 8, 4, False), (-(-(-(-2 * tiles // 7)) // units) * 7, 7, True),
                   (-(-(-(-2 * tiles // 4)) // units) * 4, 4, True)]
        _, waves, halves = min(options, key=lambda o: o[0])  # (the first of equals: the fewest workgroups, each reads x)
        return waves, halves
    three = _wide_cost(tiles, 3, ksplit, k_tiles, units) < _wide_cost(tiles, 4, ksplit, k_tiles, units)
    return (3 if three else 4), False


def linear_wide(x: "torch.Tensor | PreNormed", w: TiledWeight, w2: TiledWeight | None = None, out: torch.Tensor | None = None,
                out_f32: bool = False, workspace: torch.Tensor | None = None, ksplit: int = 0, nt: int = 0, defer: bool = False,
                waves: int = 0, halves: bool | None = None):
    """bfloat16 x @ w.T for up to 64 rows from a tiled weight (up to 128 with ``nt=1`` and no ``w2``), with the tile of x
    shared through LDS by the four waves of
    a workgroup and K cut into ``ksplit`` ranges that a second kernel adds up; with ``w2``: silu(x @ w.T) * (x @ w2.T).
    ``workspace``: float32, (2 if w2 else 1) * ksplit * rows * w.n values (none for a single range).  ``defer`` (not with
    ``w2``): with more than one range the second kernel is left out and a ``PartialSums`` over the workspace comes back.
    ``waves``, ``halves``: waves per workgroup and whether gate and up go by half tiles (``wide_waves`` by default).
    ``x`` may be a ``PreNormed`` (at most 16 rows, one range)."""
    pre = x if isinstance(x, PreNormed) else None
    if pre is not None:
        x = pre.x
    _gpu(x, out, workspace)
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k, WIDE_TALL_ROWS):
        raise KernelRefused(f"linear_wide takes bfloat16 x [rows <= {WIDE_TALL_ROWS}, {w.k}] with an inner size that is a "
                            f"multiple of 8; got {tuple(x.shape)} {x.dtype}")
    m = x.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    plan = wide_plan(w.n, w.k, m)
    ksplit, nt = ksplit or plan[0], nt or plan[1]
    if not waves:
        waves, dealt_halves = wide_waves(w.n, w.k, m, ksplit, nt, gated=w2 is not None)
        halves = dealt_halves if halves is None else halves
    halves = bool(halves)
    if m > SKINNY_MAX_ROWS and ((w2 is not None and not halves) or nt != 1):
        raise KernelRefused(f"linear_wide takes more than {SKINNY_MAX_ROWS} rows only with one row tile per wave, and two matrices only by half tiles")
    defer = defer and ksplit > 1 and w2 is None and not out_f32
    if out is None and not defer:
        out = torch.empty((m, w.n), dtype=want, device=x.device)
    if not defer and (out.shape != (m, w.n) or out.dtype != want or out.stride(1) != 1):
        raise KernelRefused("linear_wide: out has the wrong shape or dtype")
    if w2 is not None and (w2.n != w.n or w2.k != w.k or out_f32):
        raise KernelRefused("linear_wide: w2 must match w and the gated result is bfloat16")
    need = (2 if w2 is not None else 1) * ksplit * m * w.n if ksplit > 1 else 0  # a single range writes the result itself
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.float32, device=x.device)
    if need and (workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous()):
        raise KernelRefused("linear_wide: workspace too small")
    if pre is not None and (ksplit != 1 or defer):
        raise KernelRefused("linear_wide: a pre-normed input goes with one range of K")
    if halves and (w2 is None or ksplit != 1 or nt != 1 or waves not in (4, 7)):
        raise KernelRefused("linear_wide: half tiles go with two matrices, one range, one tile per wave, 4 or 7 waves")
    if not halves and waves != 4 and not (waves == 3 and w2 is None and nt == 1 and m <= SKINNY_MAX_ROWS):
        raise KernelRefused("linear_wide: workgroups of 4 waves, or of 3 for one matrix with one tile per wave and up to 64 rows")
    _check(build.core().ns_gemm_wide_dealt_bf16(_ptr(None if defer else out), _ptr(workspace if need else None), _ptr(x), _ptr(w.data),
                                                _ptr(w2.data if w2 is not None else None), c_int(m), c_int(w.n), c_int(w.k), c_int(x.stride(0)),
                                                c_int(w.n if defer else out.stride(0)), c_int(1 if w2 is not None else 0),
                                                c_int(1 if out_f32 else 0), c_int(ksplit), c_int(nt), c_int(1 if defer else 0),
                                                c_int(waves), c_int(1 if halves else 0), *_prenorm_args(pre, m, "linear_wide"), _stream()),
           "linear_wide")
    return PartialSums(workspace, ksplit, m, w.n, x.dtype) if defer else out


def rows_plan(n: int, k: int, rows: int, gated: bool = False, units: int | None = None) -> tuple[int, int]:
    """(ranges K is cut into, 16-row tiles per wave) of ``linear_rows``: the most tiles per wave, then ranges of K until
    the workgroups fill the GPU, with at least eight k tiles of 128 per range."""
    units = units or compute_units(torch.cuda.current_device())
    nt = 2 if gated else 4
    groups = -(-n // (64 * nt)) * -(-rows // 128)
    k_tiles = -(-k // 128)
    return max(1, min(16, k_tiles // 8, units // groups)), nt


def linear_rows(x: torch.Tensor, w: TiledWeight, w2: TiledWeight | None = None, out: torch.Tensor | None = None,
                out_f32: bool = False, workspace: torch.Tensor | None = None, ksplit: int = 0, nt: int = 0):
    """bfloat16 x @ w.T for any number of rows from a tiled weight: the kernel of ``linear_wide`` over blocks of 128 rows,
    with ``nt`` (2 or 4; 1 or 2 with ``w2``) row tiles of the weight per wave.  For models that keep the tiled layout only:
    the platform's library is twice as fast where the plain layout is there for it.  Arguments as ``linear_wide``."""
    _gpu(x, out, workspace)
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k, x.shape[0]):
        raise KernelRefused(f"linear_rows takes bfloat16 x [rows, {w.k}] with an inner size that is a multiple of 8; got "
                            f"{tuple(x.shape)} {x.dtype}")
    m = x.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    plan = rows_plan(w.n, w.k, m, w2 is not None)
    ksplit, nt = ksplit or plan[0], nt or plan[1]
    if out is None:
        out = torch.empty((m, w.n), dtype=want, device=x.device)
    if out.shape != (m, w.n) or out.dtype != want or out.stride(1) != 1:
        raise KernelRefused("linear_rows: out has the wrong shape or dtype")
    if w2 is not None and (w2.n != w.n or w2.k != w.k or out_f32):
        raise KernelRefused("linear_rows: w2 must match w and the gated result is bfloat16")
    need = (2 if w2 is not None else 1) * ksplit * m * w.n if ksplit > 1 else 0
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.float32, device=x.device)
    if need and (workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous()):
        raise KernelRefused("linear_rows: workspace too small")
    _check(build.core().ns_gemm_rows_bf16(_ptr(out), _ptr(workspace if need else None), _ptr(x), _ptr(w.data),
                                          _ptr(w2.data if w2 is not None else None), c_int(m), c_int(w.n), c_int(w.k), c_int(x.stride(0)),
                                          c_int(out.stride(0)), c_int(1 if w2 is not None else 0),
                                          c_int(1 if out_f32 else 0), c_int(ksplit), c_int(nt), c_int(0), _stream()),
           "linear_rows")
    return out


def qkv_rope_row_order(heads: int, kv_heads: int, head_dim: int, rotary_dim: int, interleaved: bool = False) -> torch.Tensor:
    """The row order of a stacked [q; k; v] matrix for ``linear_qkv_rope``: per head 16-row tiles; in the rotary part of a
    q or k head a tile holds the first channels of 8 rotary pairs and then their second channels (pair j is channels j and
    j + rotary_dim/2, or 2j and 2j + 1 with ``interleaved``), elsewhere 16 consecutive channels."""
    order = []
    half = rotary_dim // 2
    first, second = ((lambda j: 2 * j), (lambda j: 2 * j + 1)) if interleaved else ((lambda j: j), (lambda j: j + half))
    for g in range(heads + 2 * kv_heads):
        base = g * head_dim
        rot = rotary_dim if g < heads + kv_heads else 0
        for jt in range(rot // 16):
            order += [base + first(jt * 8 + e) for e in range(8)] + [base + second(jt * 8 + e) for e in range(8)]
        for d0 in range(rot, head_dim, 16):
            order += [base + d0 + e for e in range(16)]
    return torch.tensor(order, dtype=torch.int64)


def qkv_rope_takes(x: torch.Tensor, head_dim: int, rotary_dim: int) -> bool:
    return x.dtype == torch.bfloat16 and x.shape[0] <= 16 and head_dim % 16 == 0 and rotary_dim % 16 == 0


def linear_qkv_rope(x: "torch.Tensor | PreNormed", w: TiledWeight, q_out: torch.Tensor, positions, token_req, block_table, inv_freq,
                    k_cache, v_cache, heads: int, kv_heads: int, head_dim: int, rotary_dim: int, write_kv: bool = True,
                    waves: int = 0, interleaved: bool = False, factor: float = 1.0) -> None:
    """The stacked q/k/v product of at most 16 tokens with rotation and cache write fused into its epilogue: q goes rotated
    into ``q_out`` [M, >= heads * head_dim], k rotated into its K page slot, v into the transposed V page.  ``w`` is the
    stacked matrix tiled in ``qkv_rope_row_order`` (of the same ``interleaved``).  ``x`` may be a ``PreNormed``."""
    pre = x if isinstance(x, PreNormed) else None
    if pre is not None:
        x = pre.x
    _gpu(x, q_out, positions, token_req, block_table, inv_freq, k_cache, v_cache)
    m = x.shape[0]
    if not (tiled_takes(x, w.k) and qkv_rope_takes(x, head_dim, rotary_dim)) or x.shape[1] != w.k:
        raise KernelRefused("linear_qkv_rope takes at most 16 bfloat16 rows and head and rotary sizes that are multiples of 16")
    if w.n != (heads + 2 * kv_heads) * head_dim:
        raise KernelRefused("linear_qkv_rope: the weight does not hold heads + 2 kv_heads heads")
    if q_out.dtype != torch.bfloat16 or q_out.shape[0] != m or q_out.shape[1] < heads * head_dim or q_out.stride(1) != 1:
        raise KernelRefused("linear_qkv_rope: q_out must be bfloat16 [rows, >= heads * head_dim]")
    _i32(positions, "positions"), _i32(token_req, "token_req")
    page = _check_pages(block_table, k_cache, v_cache, kv_heads, head_dim, torch.bfloat16, "linear_qkv_rope")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(1, rotary_dim // 2) or positions.numel() != m or token_req.numel() != m:
        raise KernelRefused("linear_qkv_rope: positions, token_req are per row; inv_freq holds rotary_dim / 2 float32 values")
    if waves == 0:
        waves = 8 if w.k >= 2048 else 4
    _check(build.core().ns_gemm_qkv_rope_bf16(_ptr(q_out), _ptr(x), _ptr(w.data), c_int(m), c_int(w.k), c_int(x.stride(0)),
                                              c_int(q_out.stride(0)), _ptr(positions), _ptr(token_req), _ptr(block_table),
                                              c_int(block_table.stride(0)), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), c_int(heads),
                                              c_int(kv_heads), c_int(head_dim), c_int(rotary_dim), c_int(1 if interleaved else 0),
                                              c_float(factor), c_int(page),
                                              c_int(1 if write_kv else 0), c_int(waves), *_prenorm_args(pre, m, "linear_qkv_rope"),
                                              _stream()), "linear_qkv_rope")


def rope_kv_from_partial(p: PartialSums, q_out: torch.Tensor, positions, token_req, block_table, inv_freq, k_cache, v_cache,
                         heads: int, kv_heads: int, head_dim: int, rotary_dim: int, write_kv: bool = True, interleaved: bool = False,
                         factor: float = 1.0) -> None:
    """Rotation and cache write for a stacked q/k/v product whose K ranges are not added up yet (``linear_wide(...,
    defer=True)`` from a weight tiled in ``qkv_rope_row_order`` of the same ``interleaved``): one pass adds the ranges, rotates, and writes q into
    ``q_out`` [rows, >= heads * head_dim], k into its K page slot and v into the transposed V page."""
    _gpu(p.ws, q_out, positions, token_req, block_table, inv_freq, k_cache, v_cache)
    m = p.rows
    if p.dtype != torch.bfloat16 or head_dim % 16 or rotary_dim % 16 or p.n != (heads + 2 * kv_heads) * head_dim:
        raise KernelRefused("rope_kv_from_partial takes a bfloat16 product of heads + 2 kv_heads heads, head and rotary sizes multiples of 16")
    if q_out.dtype != torch.bfloat16 or q_out.shape[0] != m or q_out.shape[1] < heads * head_dim or q_out.stride(1) != 1:
        raise KernelRefused("rope_kv_from_partial: q_out must be bfloat16 [rows, >= heads * head_dim]")
    _i32(positions, "positions"), _i32(token_req, "token_req")
    page = _check_pages(block_table, k_cache, v_cache, kv_heads, head_dim, torch.bfloat16, "rope_kv_from_partial")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(1, rotary_dim // 2) or positions.numel() != m or token_req.numel() != m:
        raise KernelRefused("rope_kv_from_partial: positions, token_req are per row; inv_freq holds rotary_dim / 2 float32 values")
    if p.ws.dtype != torch.float32 or p.ws.numel() < p.ksplit * m * p.n:
        raise KernelRefused("rope_kv_from_partial: the partial sums are too few")
    _check(build.core().ns_rope_kv_partial(_ptr(q_out), c_int(q_out.stride(0)), _ptr(p.ws), c_int(p.ksplit), c_int(m), c_int(p.n),
                                           _ptr(positions), _ptr(token_req), _ptr(block_table), c_int(block_table.stride(0)),
                                           _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), c_int(heads), c_int(kv_heads), c_int(head_dim),
                                           c_int(rotary_dim), c_int(1 if interleaved else 0), c_float(factor), c_int(page),
                                           c_int(1 if write_kv else 0), _stream()), "rope_kv_from_partial")


# ------------------------------------------------------------------------------------------------ attention


def _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim, v_dim: int | None = None):
    _gpu(q, out, k_cache, v_cache)
    v_dim = head_dim if v_dim is None else v_dim
    page = k_cache.shape[2] if k_cache.dim() == 4 else 0
    if (k_cache.dim() != 4 or k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, v_dim, page)
            or not k_cache.is_contiguous() or not v_cache.is_contiguous() or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype):
        raise KernelRefused("attention: cache pages do not fit heads, head size or dtype")
    if q.stride(1) != 1 or q.shape[1] < heads * head_dim:
        raise KernelRefused("attention: q rows must hold heads * head_dim contiguous values")
    if out.shape != (q.shape[0], heads * v_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelRefused("attention: out must be contiguous [tokens, heads * value size]")
    if heads % kv_heads:
        raise KernelRefused(f"attention: {heads} heads are not a multiple of {kv_heads} key/value heads")
    return page


def attention_generic(q, out, k_cache, v_cache, token_req, positions, block_table, heads: int, kv_heads: int, head_dim: int,
                      scale: float, window: int = 0, v_dim: int | None = None, chunk: int = 0, cap: float = 0.0,
                      sink: bool = False, slope_exp: float = 0.0, sink_logits: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of every token's query over its request's pages; any key and value size up to 1024, either
    dtype.  ``chunk`` > 0: a query sees no key before the start of its own chunk of positions; ``cap`` > 0: scores become
    cap * tanh(score / cap); ``sink``: one more term of score 0 without a value in the soft-max's denominator;
    ``slope_exp`` > 0: head h of H loses 2^(-slope_exp (h + 1) / H) times its distance to the key from every score.
    ``sink_logits`` (float32 [heads]): the one more term is exp(sink_logits[h]), not scaled, instead of exp(0)."""
    v_dim = head_dim if v_dim is None else v_dim
    page = _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim, v_dim)
    if sink_logits is not None and (_f32(sink_logits, "sink_logits").numel() != heads):
        raise KernelRefused(f"attention_generic: sink_logits holds one float32 value for each of the {heads} heads")
    _i32(token_req, "token_req"), _i32(positions, "positions"), _i32(block_table, "block_table")
    if head_dim > 1024 or v_dim > 1024:
        raise KernelRefused(f"attention_generic takes key and value sizes up to 1024, not {head_dim} and {v_dim}")
    n = q.shape[0]
    _check(build.core().ns_attn_generic(_ptr(out), _ptr(q), c_int(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(token_req),
                                        _ptr(positions), _ptr(block_table), c_int(block_table.stride(0)), c_int(n), c_int(heads),
                                        c_int(kv_heads), c_int(head_dim), c_int(v_dim), c_int(page), c_float(scale), c_int(window),
                                        c_int(chunk), c_float(cap), c_int(1 if sink else 0), _ptr(sink_logits), c_float(slope_exp), c_int(_dtype_code(q)),
                                        _stream()), "attention_generic")
    return out


def unit_kv_write(qkv: torch.Tensor, positions, token_req, block_table, k_cache, v_cache, heads: int, kv_heads: int, head_dim: int,
                  v_dim: int, eps: float | None, own_kv: bool = True) -> None:
    """For attention without rotation.  A row of ``qkv`` is q [heads, head_dim] and, with ``own_kv``, k [kv_heads, head_dim]
    and v [kv_heads, v_dim].  With ``eps`` not None every head's q (in place) and k are divided by their root mean square,
    x / sqrt(mean(x^2) + eps); k and v of every token go into the pages ``block_table[token_req[t], position // page]``:
    k_cache [pages, kv_heads, page, head_dim], v_cache [pages, kv_heads, v_dim, page]."""
    _gpu(qkv, positions, token_req, block_table, k_cache, v_cache)
    n = positions.numel()
    width = heads * head_dim + (kv_heads * (head_dim + v_dim) if own_kv else 0)
    if qkv.dim() != 2 or qkv.shape[0] != n or qkv.shape[1] < width or qkv.stride(1) != 1:
        raise KernelRefused(f"unit_kv_write: qkv must be [{n}, {width}]")
    _i32(positions, "positions"), _i32(token_req, "token_req"), _i32(block_table, "block_table")
    if token_req.numel() != n or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelRefused("unit_kv_write: token_req is per token, block_table int32 [requests, pages]")
    page = k_cache.shape[2] if k_cache.dim() == 4 else 0
    if (k_cache.dim() != 4 or k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, v_dim, page)
            or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
        raise KernelRefused("unit_kv_write: cache pages do not fit heads, sizes or dtype")
    _check(build.core().ns_unit_kv_write(_ptr(qkv), c_int(qkv.stride(0)), _ptr(positions), _ptr(token_req), _ptr(block_table),
                                         c_int(block_table.stride(0)), _ptr(k_cache), _ptr(v_cache), c_int(n), c_int(heads), c_int(kv_heads),
                                         c_int(head_dim), c_int(v_dim), c_int(page), c_float(-1.0 if eps is None else eps),
                                         c_int(1 if own_kv else 0), c_int(_dtype_code(qkv)), _stream()), "unit_kv_write")


def mfma_attention_takes(dtype, head_dim: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and page_size >= 4 and page_size & (page_size - 1) == 0


TILE_INTS = 8  # ints per attention tile descriptor: request, first token, first row, tokens, keys, 0, 0, 0


def attention_mfma(q, out, k_cache, v_cache, tiles, block_table, heads: int, kv_heads: int, head_dim: int, scale: float,
                   window: int = 0, hp: int = 1, splits: int = 1,
                   workspace: tuple[torch.Tensor, torch.Tensor] | None = None, qt: int = 1, coop: bool = False,
                   short_offsets: bool = True, chunk: int = 0, cap: float = 0.0, sink: bool = False,
                   sink_logits: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 attention on the matrix cores for the tiles described in ``tiles`` (int32 [n_tiles, 8]: request, first
    token of the tile among the request's tokens of this step, row of the request's first token in ``q``, tokens of the
    request in this step, keys after this step, three zeros).  ``hp`` heads of a group times 16/hp tokens make a tile;
    with ``qt`` = 2 (only with hp = 1) a tile is 32 tokens.  ``splits`` > 1 cuts the keys of every tile
    into that many ranges (at most 64) and needs ``workspace`` = (part_o, part_ml) float32 tensors.  With ``coop`` the four
    waves of a workgroup share each tile and range (for decode, where a wave's chain of loads is what takes the time); with
    ``qt`` = 2 it asks for workgroups of one set of four waves instead of two (for long rows of keys).  A pool within
    4 GiB is addressed with 32-bit offsets from its start; ``short_offsets`` = False keeps every address 64 bits wide
    whatever the pool's size (the form that larger pools take).  ``chunk``, ``cap``, ``sink``, ``sink_logits``: as for
    ``attention_generic``; with any of them the tiles are walked by the kernels that do not share keys through LDS."""
    page = _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim)
    if sink_logits is not None and _f32(sink_logits, "sink_logits").numel() != heads:
        raise KernelRefused(f"attention_mfma: sink_logits holds one float32 value for each of the {heads} heads")
    if not mfma_attention_takes(q.dtype, head_dim, page):
        raise KernelRefused(f"attention_mfma takes bfloat16, head sizes that are multiples of 16 up to 256 and page sizes that are "
                            f"powers of two from 4; got {q.dtype}, head size {head_dim}, page {page}")
    _gpu(tiles, block_table)
    _i32(tiles, "tiles"), _i32(block_table, "block_table")
    if tiles.dim() != 2 or tiles.shape[1] != TILE_INTS or tiles.data_ptr() % 16:
        raise KernelRefused(f"attention_mfma: tiles must be int32 [n_tiles, {TILE_INTS}], 16-byte aligned")
    if hp not in (1, 2, 4, 8, 16):
        raise KernelRefused("attention_mfma: hp is a power of two up to 16")
    if qt != 1 and not (qt == 2 and hp == 1):
        raise KernelRefused("attention_mfma: 32-token tiles (qt = 2) go with hp = 1")
    n_tiles = tiles.shape[0]
    po = pm = None
    if splits > 1:
        if workspace is None or splits > 64:
            raise KernelRefused("attention_mfma: 2 to 64 key ranges are taken, with a workspace")
        po, pm = workspace
        cols = n_tiles * (qt * 16 // hp) * heads
        if po.dtype != torch.float32 or pm.dtype != torch.float32 or po.numel() < cols * splits * head_dim or pm.numel() < cols * splits * 2:
            raise KernelRefused("attention_mfma: workspace too small")
    lib = build.attn(head_dim, page)
    _check(lib.ns_attn_mfma(_ptr(out), _ptr(po), _ptr(pm), _ptr(q), c_int(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(tiles),
                            _ptr(block_table), c_int(block_table.stride(0)), c_int(n_tiles), c_int(heads), c_int(kv_heads),
                            c_int(page), c_int(hp), c_int(splits), c_int(window), c_float(scale), c_int(qt), c_int(1 if coop else 0),
                            ctypes.c_long(k_cache.shape[0] if short_offsets else 0), c_int(chunk), c_float(cap), c_int(1 if sink else 0),
                            _ptr(sink_logits), _stream()),
           "attention_mfma")
    return out


def wide_attention_takes(dtype, head_dim: int, v_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 1024 and v_dim % 16 == 0 and 16 <= v_dim <= 512
            and page_size >= 4 and page_size & (page_size - 1) == 0)


def attention_wide(q, out, k_cache, v_cache, tiles, block_table, heads: int, kv_heads: int, head_dim: int, v_dim: int, scale: float,
                   window: int = 0, hp: int = 1, splits: int = 1, workspace: tuple[torch.Tensor, torch.Tensor] | None = None, qt: int = 1,
                   slope_exp: float = 0.0, sink_logits: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 attention on the matrix cores for keys of ``head_dim`` and values of ``v_dim`` channels (multiples of 16 up
    to 1,024 and 512), over the tiles of ``tiles`` (as for ``attention_mfma``): ``hp`` heads of a group times 16/hp tokens
    are one wave's columns, ``qt`` such sets of tokens a tile.  ``splits`` > 1 cuts every tile's keys into ranges and needs
    ``workspace`` = (part_o, part_ml) float32 tensors.  ``slope_exp``, ``sink_logits``: as for ``attention_generic``."""
    page = _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim, v_dim)
    if sink_logits is not None and _f32(sink_logits, "sink_logits").numel() != heads:
        raise KernelRefused(f"attention_wide: sink_logits holds one float32 value for each of the {heads} heads")
    if not wide_attention_takes(q.dtype, head_dim, v_dim, page):
        raise KernelRefused(f"attention_wide takes bfloat16, key sizes that are multiples of 16 up to 1024, value sizes up to 512 and page "
                            f"sizes that are powers of two from 4; got {q.dtype}, sizes {head_dim} and {v_dim}, page {page}")
    _gpu(tiles, block_table)
    _i32(tiles, "tiles"), _i32(block_table, "block_table")
    if tiles.dim() != 2 or tiles.shape[1] != TILE_INTS or tiles.data_ptr() % 16:
        raise KernelRefused(f"attention_wide: tiles must be int32 [n_tiles, {TILE_INTS}], 16-byte aligned")
    if hp not in (1, 2, 4, 8, 16) or not 1 <= qt <= 4:
        raise KernelRefused("attention_wide: hp is a power of two up to 16, qt 1 to 4")
    n_tiles = tiles.shape[0]
    po = pm = None
    if splits > 1:
        if workspace is None or splits > 64:
            raise KernelRefused("attention_wide: 2 to 64 key ranges are taken, with a workspace")
        po, pm = workspace
        cols = n_tiles * (qt * 16 // hp) * heads
        if po.dtype != torch.float32 or pm.dtype != torch.float32 or po.numel() < cols * splits * v_dim or pm.numel() < cols * splits * 2:
            raise KernelRefused("attention_wide: workspace too small")
    lib = build.attn_wide(head_dim, v_dim, page)
    _check(lib.ns_attn_wide(_ptr(out), _ptr(po), _ptr(pm), _ptr(q), c_int(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(tiles),
                            _ptr(block_table), c_int(block_table.stride(0)), c_int(n_tiles), c_int(heads), c_int(kv_heads), c_int(page),
                            c_int(hp), c_int(splits), c_int(window), c_float(scale), c_int(qt), c_float(slope_exp), _ptr(sink_logits),
                            _stream()), "attention_wide")
    return out


def attention_prompt_form(head_dim: int, page_size: int) -> int:
    """Which kernel of the library for this head and page size takes prompt portions in tiles of 32 tokens: 32 the one
    on the 32x32 matrix instruction with loads straight into LDS, 16 the one on the 16x16 instruction with keys shared
    through LDS, 0 the one without sharing."""
    return int(build.attn(head_dim, page_size).ns_attn_prompt_form())


# ------------------------------------------------------------------------------------------------ 32-bit streams

MAX_STREAMS = 16
ACTIVATIONS = {"gelu_tanh": 0, "silu": 1}


def _f32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.float32 or not t.is_contiguous() or not t.is_cuda:
        raise KernelRefused(f"{name} must be a contiguous float32 tensor on the GPU")
    return t


def embed_streams(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[i, s, :] = table[ids[i]] * scale for every copy s of the stream; ``out`` float32 [tokens, copies, hidden]."""
    _gpu(table, ids)
    _i32(ids, "ids"), _f32(out, "out")
    n, hidden = ids.numel(), table.shape[1]
    if out.dim() != 3 or out.shape[0] != n or out.shape[2] != hidden or not 1 <= out.shape[1] <= MAX_STREAMS or not table.is_contiguous():
        raise KernelRefused(f"embed_streams: out must be float32 [{n}, copies <= {MAX_STREAMS}, {hidden}]")
    _check(build.core().ns_embed_streams(_ptr(out), _ptr(table), _ptr(ids), c_int(n), c_int(hidden), c_int(out.shape[1]), c_float(scale),
                                         c_int(_dtype_code(table)), _stream()), "embed_streams")
    return out


def stream_read_norm(x: torch.Tensor, coeff: torch.Tensor, weight: torch.Tensor | None, eps: float, rows: torch.Tensor | None = None,
                     out: torch.Tensor | None = None, sum_out: torch.Tensor | None = None, w_offset: float = 0.0,
                     dtype: torch.dtype | None = None) -> torch.Tensor:
    """u = sum_s coeff[s] x[r, s, :] with r = rows[i] (or i); out[i] = (w_offset + weight) * u / sqrt(mean(u^2) + eps) in the weight's dtype.
    ``x`` float32 [tokens, S, W]; ``sum_out`` (float32 [n, W], optional) also receives u.  Without a ``weight`` there is no
    norm: out[i] = u in ``dtype``."""
    _f32(x, "x"), _f32(coeff, "coeff")
    _gpu(weight, rows, out, sum_out)
    if weight is None:
        if dtype is None:
            raise KernelRefused("stream_read_norm: a read without a norm says in which dtype it wants the stream")
        weight_dtype = dtype
    else:
        weight_dtype = weight.dtype
    if x.dim() != 3 or coeff.numel() != x.shape[1] or x.shape[1] > MAX_STREAMS or (weight is not None and (weight.shape != (x.shape[2],) or not weight.is_contiguous())):
        raise KernelRefused("stream_read_norm: x is [tokens, S, W], coeff [S], weight [W]")
    if rows is not None:
        _i32(rows, "rows")
    n = rows.numel() if rows is not None else x.shape[0]
    S, W = x.shape[1], x.shape[2]
    if out is None:
        out = torch.empty((n, W), dtype=weight_dtype, device=x.device)
    if out.shape != (n, W) or out.dtype != weight_dtype or not out.is_contiguous():
        raise KernelRefused("stream_read_norm: out must be contiguous [rows, W] of the weight's dtype")
    if sum_out is not None and (_f32(sum_out, "sum_out").shape != (n, W)):
        raise KernelRefused("stream_read_norm: sum_out must be float32 [rows, W]")
    _check(build.core().ns_stream_read_norm(_ptr(out), _ptr(sum_out), _ptr(x), _ptr(coeff), _ptr(weight), _ptr(rows), c_int(n), c_int(S),
                                            c_int(W), c_float(eps), c_float(w_offset), c_int(_dtype_code(out)), _stream()), "stream_read_norm")
    return out


def _post_args(post: "PostNorm | None", y: torch.Tensor, W: int, what: str):
    """-> (bias, weight, eps, offset) as the kernels take them."""
    if post is None:
        return _ptr(None), _ptr(None), c_float(0.0), c_float(0.0)
    for t in (post.bias, post.weight):
        if t is not None and (not t.is_cuda or t.shape != (W,) or not t.is_contiguous() or t.dtype != y.dtype):
            raise KernelRefused(f"{what}: the bias and the norm weight behind a sublayer are [{W}] in the dtype of its output")
    return _ptr(post.bias), _ptr(post.weight), c_float(post.eps), c_float(post.offset)


def stream_write(x: torch.Tensor, mix: torch.Tensor, gain: torch.Tensor, y: torch.Tensor, post: "PostNorm | None" = None) -> None:
    """In place, all streams at once from the old ones: x[r, t, :] = sum_s mix[s, t] x[r, s, :] + gain[t] * y[r, :]; with
    ``post``, y first passes a bias and an RMS norm of its own (``PostNorm``)."""
    _f32(x, "x"), _f32(mix, "mix"), _f32(gain, "gain")
    _gpu(y)
    if post is not None:
        if x.dim() != 3 or mix.shape != (x.shape[1], x.shape[1]) or gain.shape != (x.shape[1],) or x.shape[1] > MAX_STREAMS:
            raise KernelRefused("stream_write: x is [tokens, S, W], mix [S, S] (from, to), gain [S]")
        if y.dim() != 2 or y.shape != (x.shape[0], x.shape[2]) or y.stride(1) != 1:
            raise KernelRefused("stream_write: y must be [tokens, W]")
        _check(build.core().ns_stream_write_post(_ptr(x), _ptr(mix), _ptr(gain), _ptr(y), c_int(y.stride(0)), c_int(x.shape[0]), c_int(x.shape[1]),
                                                 c_int(x.shape[2]), *_post_args(post, y, x.shape[2], "stream_write"), c_int(_dtype_code(y)),
                                                 _stream()), "stream_write")
        return
    if x.dim() != 3 or mix.shape != (x.shape[1], x.shape[1]) or gain.shape != (x.shape[1],) or x.shape[1] > MAX_STREAMS:
        raise KernelRefused("stream_write: x is [tokens, S, W], mix [S, S] (from, to), gain [S]")
    if y.dim() != 2 or y.shape != (x.shape[0], x.shape[2]) or y.stride(1) != 1:
        raise KernelRefused("stream_write: y must be [tokens, W]")
    _check(build.core().ns_stream_write(_ptr(x), _ptr(mix), _ptr(gain), _ptr(y), c_int(y.stride(0)), c_int(x.shape[0]), c_int(x.shape[1]),
                                        c_int(x.shape[2]), c_int(_dtype_code(y)), _stream()), "stream_write")


STEP_MAX_STREAMS, STEP_MAX_WIDTH = 4, 8192  # what the one-pass kernel of ``stream_step`` takes (rows of a multiple of four columns)


class PostNorm:
    """What a sublayer's output y passes before it is written into a 32-bit stream: a bias (the sublayer's last projection's,
    left to this place), then an RMS norm, (y + bias) / sqrt(mean((y + bias)^2) + eps) * (offset + weight), all in 32-bit.
    Either may be None."""

    def __init__(self, bias: torch.Tensor | None = None, weight: torch.Tensor | None = None, eps: float = 0.0, offset: float = 0.0) -> None:
        self.bias, self.weight, self.eps, self.offset = bias, weight, eps, offset


class PendingWrite:
    """A sublayer's output on its way into a 32-bit stream: x_t <- sum_s mix[s, t] x_s + gain[t] * y, not done yet.
    ``stream_step`` does it in the same pass as the next read.  ``post``: what y passes first (``PostNorm``)."""

    def __init__(self, y: torch.Tensor, mix: torch.Tensor, gain: torch.Tensor, post: "PostNorm | None" = None) -> None:
        self.y, self.mix, self.gain, self.post = y, mix, gain, post


def stream_step(x: torch.Tensor, pending: "PendingWrite | None", coeff: torch.Tensor | None = None, weight: torch.Tensor | None = None,
                eps: float = 0.0, rows: torch.Tensor | None = None, out: torch.Tensor | None = None, sum_out: torch.Tensor | None = None,
                store: bool = True, w_offset: float = 0.0, dtype: torch.dtype | None = None) -> torch.Tensor | None:
    """``stream_write`` of ``pending`` (if any) and then ``stream_read_norm`` with ``coeff`` and ``weight`` (if any), in one
    pass over the rows where the sizes allow it, in two kernels otherwise.  With ``rows`` the read is of those rows only,
    and a pending write is then done on the fly for them and not kept (``store`` must be False): for the last read of a step.
    A read with ``coeff`` but without ``weight`` has no norm: it gives the mix itself in ``dtype``."""
    S, W = x.shape[1], x.shape[2]
    if pending is not None and rows is not None and store:
        raise KernelRefused("stream_step: a write that is kept covers every row")
    one_pass = S <= STEP_MAX_STREAMS and W <= STEP_MAX_WIDTH and W % 4 == 0
    if not one_pass:
        if pending is not None:  # (kept whatever ``store`` says: keeping it harms nobody)
            stream_write(x, pending.mix, pending.gain, pending.y, pending.post)
        return stream_read_norm(x, coeff, weight, eps, rows=rows, out=out, sum_out=sum_out, w_offset=w_offset, dtype=dtype) if coeff is not None else None
    _f32(x, "x")
    y = None
    if pending is not None:
        y = pending.y
        _f32(pending.mix, "mix"), _f32(pending.gain, "gain")
        _gpu(y)
        if pending.mix.shape != (S, S) or pending.gain.shape != (S,) or y.dim() != 2 or y.shape != (x.shape[0], W) or y.stride(1) != 1:
            raise KernelRefused("stream_step: mix [S, S], gain [S], y [tokens, W]")
    if y is None and weight is None and coeff is not None and dtype is None:
        raise KernelRefused("stream_step: a read without a norm says in which dtype it wants the stream")
    dtype = y.dtype if y is not None else (weight.dtype if weight is not None else dtype)
    n = x.shape[0]
    if coeff is not None:
        _f32(coeff, "coeff")
        _gpu(weight, rows, out, sum_out)
        if coeff.numel() != S or (weight is not None and (weight.shape != (W,) or not weight.is_contiguous() or weight.dtype != dtype)):
            raise KernelRefused("stream_step: coeff [S], weight [W] in the dtype of y")
        if rows is not None:
            _i32(rows, "rows")
            n = rows.numel()
        if out is None:
            out = torch.empty((n, W), dtype=dtype, device=x.device)
        if out.shape != (n, W) or out.dtype != dtype or not out.is_contiguous():
            raise KernelRefused("stream_step: out must be contiguous [rows, W] of the weight's dtype")
        if sum_out is not None and _f32(sum_out, "sum_out").shape != (n, W):
            raise KernelRefused("stream_step: sum_out must be float32 [rows, W]")
    elif pending is None:
        return None
    _check(build.core().ns_stream_step(_ptr(x), _ptr(pending.mix if pending else None), _ptr(pending.gain if pending else None), _ptr(y),
                                       c_int(y.stride(0) if y is not None else 0), _ptr(coeff), _ptr(weight), _ptr(rows), _ptr(out),
                                       _ptr(sum_out), c_int(n), c_int(S), c_int(W), c_float(eps), c_int(1 if store else 0), c_float(w_offset),
                                       *_post_args(pending.post if pending else None, y, W, "stream_step"),
                                       c_int(BF16 if dtype == torch.bfloat16 else F32), _stream()), "stream_step")
    return out


def stream_add_rows(x: torch.Tensor, table: torch.Tensor | None, ids: torch.Tensor | None, vec: torch.Tensor | None, scale: float = 1.0) -> None:
    """In place, for every copy s of a 32-bit stream ``x`` [tokens, copies, hidden]: x[r, s] += scale * table[ids[r]] (if
    ``table``) + vec (if ``vec`` [hidden]); ``table`` and ``vec`` in one storage type."""
    _f32(x, "x")
    _gpu(table, ids, vec)
    if table is None and vec is None:
        return
    n, S, W = x.shape
    any_t = table if table is not None else vec
    if ((table is not None and (table.dim() != 2 or table.shape[1] != W or not table.is_contiguous() or ids is None or _i32(ids, "ids").numel() != n))
            or (vec is not None and (vec.shape != (W,) or not vec.is_contiguous() or vec.dtype != any_t.dtype)) or S > MAX_STREAMS):
        raise KernelRefused(f"stream_add_rows: table [rows, {W}] with ids [{n}], vec [{W}], of one dtype")
    _check(build.core().ns_stream_add_rows(_ptr(x), _ptr(table), _ptr(ids), _ptr(vec), c_int(n), c_int(W), c_int(S), c_float(scale),
                                           c_int(_dtype_code(any_t)), _stream()), "stream_add_rows")


def embed_pair_streams(table: torch.Tensor, pair_table: torch.Tensor, ids, positions, token_req, qo_indptr, state_slots, last_token: torch.Tensor,
                       out: torch.Tensor, scale: float, buckets: int, mul_prev: int, mul_cur: int) -> torch.Tensor:
    """``embed_streams`` plus a row of a second table chosen by the token and the one before it in its sequence:
    row (prev * mul_prev + token * mul_cur) mod buckets, and row ``buckets`` for a sequence's first token (position 0).
    ``last_token`` int32 [slots, 1]: every request's last token so far; read for a request's first row of the step and left
    holding its last token of the step."""
    _gpu(table, pair_table, ids, positions, token_req, qo_indptr, state_slots, last_token)
    for name, t in (("ids", ids), ("positions", positions), ("token_req", token_req), ("qo_indptr", qo_indptr), ("state_slots", state_slots),
                    ("last_token", last_token)):
        _i32(t, name)
    _f32(out, "out")
    n, hidden = ids.numel(), table.shape[1]
    if (out.dim() != 3 or out.shape[0] != n or out.shape[2] != hidden or not 1 <= out.shape[1] <= MAX_STREAMS or not table.is_contiguous()
            or pair_table.shape != (buckets + 1, hidden) or not pair_table.is_contiguous() or pair_table.dtype != table.dtype
            or positions.numel() != n or token_req.numel() != n or qo_indptr.numel() != state_slots.numel() + 1):
        raise KernelRefused(f"embed_pair_streams: out float32 [{n}, copies, {hidden}], the second table [{buckets + 1}, {hidden}]")
    _check(build.core().ns_embed_pair_streams(_ptr(out), _ptr(table), _ptr(pair_table), _ptr(ids), _ptr(positions), _ptr(token_req),
                                              _ptr(qo_indptr), _ptr(state_slots), _ptr(last_token), c_int(n), c_int(hidden), c_int(out.shape[1]),
                                              c_float(scale), c_int(buckets), c_int(mul_prev), c_int(mul_cur), c_int(_dtype_code(table)),
                                              _stream()), "embed_pair_streams")
    return out


def whole_norm_kv_write(qkv: torch.Tensor, positions, token_req, block_table, k_cache, v_cache, heads: int, kv_heads: int, head_dim: int,
                        v_dim: int, eps: float, bias: torch.Tensor | None = None, q_weight: torch.Tensor | None = None,
                        k_weight: torch.Tensor | None = None, mix: torch.Tensor | None = None, v_other: torch.Tensor | None = None,
                        v_keep: torch.Tensor | None = None, inv_freq: torch.Tensor | None = None, rotary_dim: int = 0, interleaved: bool = False,
                        factor: float = 1.0) -> None:
    """For attention without rotation whose projections carry biases and whose queries and keys pass an RMS norm over the whole
    projection.  A row of ``qkv`` is q [heads * head_dim], k [kv_heads * head_dim], v [kv_heads * v_dim]; ``bias`` of that
    width is added; q (in place) and k become x / sqrt(mean(x^2 over the whole projection) + eps) * weight; v becomes
    (1 - mix) v + mix v_other where ``v_other`` [tokens, kv_heads * v_dim] is given (``mix``: one value on the device), is
    copied to ``v_keep`` where that is given, and k and v go into the pages of their positions.  ``rotary_dim`` > 0: the first
    so many channels of every head of q and k are rotated by the token's position after the norm (``inv_freq`` float32
    [rotary_dim / 2]; pairing and ``factor`` as in ``rope_kv_write``)."""
    _gpu(qkv, positions, token_req, block_table, k_cache, v_cache, bias, q_weight, k_weight, mix, v_other, v_keep, inv_freq)
    if rotary_dim and (rotary_dim % 2 or rotary_dim > head_dim or inv_freq is None or _f32(inv_freq, "inv_freq").numel() < rotary_dim // 2):
        raise KernelRefused("whole_norm_kv_write: the rotated part is an even number of a head's channels, with a frequency per pair")
    n = positions.numel()
    nq, nk, nv = heads * head_dim, kv_heads * head_dim, kv_heads * v_dim
    if qkv.dim() != 2 or qkv.shape[0] != n or qkv.shape[1] < nq + nk + nv or qkv.stride(1) != 1:
        raise KernelRefused(f"whole_norm_kv_write: qkv must be [{n}, {nq + nk + nv}]")
    _i32(positions, "positions"), _i32(token_req, "token_req"), _i32(block_table, "block_table")
    if token_req.numel() != n or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelRefused("whole_norm_kv_write: token_req is per token, block_table int32 [requests, pages]")
    page = k_cache.shape[2] if k_cache.dim() == 4 else 0
    if (k_cache.dim() != 4 or k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, v_dim, page)
            or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
        raise KernelRefused("whole_norm_kv_write: cache pages do not fit heads, sizes or dtype")
    for t, size, name in ((bias, nq + nk + nv, "bias"), (q_weight, nq, "q_weight"), (k_weight, nk, "k_weight"), (mix, 1, "mix")):
        if t is not None and (t.numel() != size or not t.is_contiguous() or t.dtype != qkv.dtype):
            raise KernelRefused(f"whole_norm_kv_write: {name} holds {size} values of the dtype of qkv")
    for t, name in ((v_other, "v_other"), (v_keep, "v_keep")):
        if t is not None and (t.dim() != 2 or t.shape != (n, nv) or t.stride(1) != 1 or t.dtype != qkv.dtype):
            raise KernelRefused(f"whole_norm_kv_write: {name} must be [{n}, {nv}] of the dtype of qkv")
    if v_other is not None and mix is None:
        raise KernelRefused("whole_norm_kv_write: values of another layer come with the weight they are mixed in with")
    _check(build.core().ns_whole_norm_kv_write(_ptr(qkv), c_int(qkv.stride(0)), _ptr(bias), _ptr(q_weight), _ptr(k_weight), _ptr(mix),
                                               _ptr(v_other), c_int(v_other.stride(0) if v_other is not None else 0), _ptr(v_keep),
                                               c_int(v_keep.stride(0) if v_keep is not None else 0), _ptr(positions), _ptr(token_req),
                                               _ptr(block_table), c_int(block_table.stride(0)), _ptr(k_cache), _ptr(v_cache), c_int(n),
                                               c_int(heads), c_int(kv_heads), c_int(head_dim), c_int(v_dim), c_int(page), c_float(eps),
                                               _ptr(inv_freq if rotary_dim else None), c_int(rotary_dim), c_int(1 if interleaved else 0),
                                               c_float(factor), c_int(_dtype_code(qkv)), _stream()), "whole_norm_kv_write")


def head_norm_rope_kv_write(qkv: torch.Tensor, positions, token_req, block_table, inv_freq, k_cache, v_cache, heads: int, kv_heads: int,
                            head_dim: int, v_dim: int, eps: float, rotary_dim: int, bias: torch.Tensor | None = None,
                            q_weight: torch.Tensor | None = None, k_weight: torch.Tensor | None = None, value_is_key: bool = False,
                            interleaved: bool = False, factor: float = 1.0) -> None:
    """For attention whose queries and keys pass an RMS norm per head and then a rotation.  A row of ``qkv`` is q [heads *
    head_dim], k [kv_heads * head_dim] and, unless ``value_is_key``, v [kv_heads * v_dim]; ``bias`` of that width is added.
    q (in place) and k become x / sqrt(mean(x^2 over the head) + eps) * weight (``q_weight``, ``k_weight`` [head_dim], shared
    by the heads; None: no norm), then their first ``rotary_dim`` channels are rotated by the token's position.  With
    ``value_is_key`` the key projection's raw output (bias added, ahead of norm and rotation) is stored as the values.  k and v go into the
    pages of their positions."""
    _gpu(qkv, positions, token_req, block_table, k_cache, v_cache, bias, q_weight, k_weight, inv_freq)
    n = positions.numel()
    nq, nk, nv = heads * head_dim, kv_heads * head_dim, 0 if value_is_key else kv_heads * v_dim
    if qkv.dim() != 2 or qkv.shape[0] != n or qkv.shape[1] < nq + nk + nv or qkv.stride(1) != 1:
        raise KernelRefused(f"head_norm_rope_kv_write: qkv must be [{n}, {nq + nk + nv}]")
    if value_is_key and v_dim != head_dim:
        raise KernelRefused("head_norm_rope_kv_write: values that are the keys have the keys' size")
    _i32(positions, "positions"), _i32(token_req, "token_req"), _i32(block_table, "block_table")
    if token_req.numel() != n or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelRefused("head_norm_rope_kv_write: token_req is per token, block_table int32 [requests, pages]")
    page = k_cache.shape[2] if k_cache.dim() == 4 else 0
    if (k_cache.dim() != 4 or k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, v_dim, page)
            or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
        raise KernelRefused("head_norm_rope_kv_write: cache pages do not fit heads, sizes or dtype")
    for t, size, name in ((bias, nq + nk + nv, "bias"), (q_weight, head_dim, "q_weight"), (k_weight, head_dim, "k_weight")):
        if t is not None and (t.numel() != size or not t.is_contiguous() or t.dtype != qkv.dtype):
            raise KernelRefused(f"head_norm_rope_kv_write: {name} holds {size} values of the dtype of qkv")
    if rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
        raise KernelRefused("head_norm_rope_kv_write: the rotated channels of a head are an even number, at most the head")
    if rotary_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2 or not inv_freq.is_contiguous()):
        raise KernelRefused("head_norm_rope_kv_write: inv_freq is float32 [rotary_dim / 2]")
    _check(build.core().ns_head_norm_rope_kv_write(_ptr(qkv), c_int(qkv.stride(0)), _ptr(bias), _ptr(q_weight), _ptr(k_weight), _ptr(positions),
                                                   _ptr(token_req), _ptr(block_table), c_int(block_table.stride(0)), _ptr(inv_freq),
                                                   _ptr(k_cache), _ptr(v_cache), c_int(n), c_int(heads), c_int(kv_heads), c_int(head_dim),
                                                   c_int(v_dim), c_int(page), c_float(eps), c_int(rotary_dim), c_int(1 if interleaved else 0),
                                                   c_float(factor), c_int(1 if value_is_key else 0), c_int(_dtype_code(qkv)), _stream()),
           "head_norm_rope_kv_write")


# ------------------------------------------------------------------------------------------------ matrix memory


MEMORY_MAX_KEY_DIM = 512  # key channels of a head that ``memory_scan`` takes (a column's channels are 8 to a lane of one wave)
MOE_MAX_EXPERTS, MOE_MAX_TOP = 1024, 32


def memory_blocks(key_dim: int, value_dim: int) -> int:
    """Workgroups of one head in ``memory_scan`` (those that share its columns, and the one that carries n): the state keeps
    a copy of m, and room for n, for each."""
    b = int(build.core().ns_memory_blocks(c_int(key_dim), c_int(value_dim)))
    if b < 0:
        raise KernelRefused(f"memory_scan takes key sizes up to 512, not {key_dim}")
    return b


def memory_state_floats(heads: int, key_dim: int, value_dim: int) -> int:
    """32-bit words of a request's state: S [heads, value_dim, key_dim], then n [heads, blocks, key_dim] and m [heads, blocks]."""
    return heads * value_dim * key_dim + heads * memory_blocks(key_dim, value_dim) * (key_dim + 1)


def memory_scan(proj: torch.Tensor, offsets: tuple[int, int, int, int, int], gate_bias_i: torch.Tensor | None, gate_bias_f: torch.Tensor | None,
                state: torch.Tensor, qo_indptr, state_slots, heads: int, key_dim: int, value_dim: int, cap: float, q_scale: float,
                out: torch.Tensor, den: torch.Tensor, den_eps: float = 1e-6) -> torch.Tensor:
    """The matrix memory's recurrence over every request's tokens of the step, in order (``csrc/memory.hip``).  A row of
    ``proj`` holds q and k [heads * key_dim], v [heads * value_dim] and the two gate inputs [heads] at the column
    ``offsets`` (q, k, v, input gate, forget gate); ``state`` float32 [slots, >= memory_state_floats].  ``out`` float32
    [tokens, heads * value_dim] receives S^T q and ``den`` float32 [tokens, heads] the denominators max(|n . q|, exp(-m)) +
    den_eps: the read-out is out / den (``gated_rms`` divides as it reads)."""
    _gpu(proj, state, qo_indptr, state_slots, out, den, gate_bias_i, gate_bias_f)
    _f32(out, "out"), _f32(den, "den"), _i32(qo_indptr, "qo_indptr"), _i32(state_slots, "state_slots")
    n = proj.shape[0]
    q_off, k_off, v_off, i_off, f_off = offsets
    if proj.dim() != 2 or proj.stride(1) != 1 or max(q_off, k_off) + heads * key_dim > proj.shape[1] or v_off + heads * value_dim > proj.shape[1] \
            or max(i_off, f_off) + heads > proj.shape[1]:
        raise KernelRefused("memory_scan: the row does not hold q, k, v and the gates at the given columns")
    if out.shape != (n, heads * value_dim) or not out.is_contiguous() or den.shape != (n, heads) or not den.is_contiguous():
        raise KernelRefused(f"memory_scan: out must be float32 [{n}, {heads * value_dim}] and den float32 [{n}, {heads}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < memory_state_floats(heads, key_dim, value_dim):
        raise KernelRefused("memory_scan: state is float32 [slots, words] with room for S, n and m")
    for t in (gate_bias_i, gate_bias_f):
        if t is not None and (_f32(t, "gate bias").numel() != heads):
            raise KernelRefused("memory_scan: a gate's bias is float32 [heads]")
    reqs = qo_indptr.numel() - 1
    if state_slots.numel() < reqs:
        raise KernelRefused("memory_scan: one state slot per request")
    _check(build.core().ns_memory_scan(_ptr(proj), c_int(proj.stride(0)), c_int(q_off), c_int(k_off), c_int(v_off), c_int(i_off), c_int(f_off),
                                       _ptr(gate_bias_i), _ptr(gate_bias_f), _ptr(state), ctypes.c_longlong(state.stride(0)), _ptr(qo_indptr),
                                       _ptr(state_slots), _ptr(out), _ptr(den), c_int(reqs), c_int(heads), c_int(key_dim), c_int(value_dim), c_float(cap),
                                       c_float(q_scale), c_float(den_eps), c_int(_dtype_code(proj)), _stream()), "memory_scan")
    return out


# ------------------------------------------------------------------------------------------------ mixture of experts


def retention_prep(proj: torch.Tensor, offsets: tuple[int, int, int], positions, inv_freq: torch.Tensor | None, heads: int, key_dim: int,
                   value_dim: int, rotary_dim: int, key_scale: float, out: torch.Tensor, interleaved: bool = False, factor: float = 1.0) -> torch.Tensor:
    """Rows [.. q .. k .. v ..] of a stacked product (``offsets``: the columns where q, k and v start) -> ``out`` float32
    [tokens, heads * (2 key_dim + value_dim)] = [q | k | v]: the first ``rotary_dim`` channels of every head of q and k rotated
    by the token's position in 32-bit, k then multiplied by ``key_scale``."""
    _gpu(proj, positions, inv_freq, out)
    _i32(positions, "positions"), _f32(out, "out")
    n = positions.numel()
    q_off, k_off, v_off = offsets
    row = heads * (2 * key_dim + value_dim)
    need = max(q_off + heads * key_dim, k_off + heads * key_dim, v_off + heads * value_dim)
    if (proj.dim() != 2 or proj.shape[0] != n or proj.shape[1] < need or proj.stride(1) != 1 or out.shape != (n, row) or not out.is_contiguous()
            or rotary_dim % 2 or not 0 <= rotary_dim <= key_dim or (rotary_dim and (inv_freq is None or _f32(inv_freq, "inv_freq").numel() < rotary_dim // 2))):
        raise KernelRefused(f"retention_prep: rows of at least {need} columns, out float32 [{n}, {row}], an even rotated part of a head")
    _check(build.core().ns_retention_prep(_ptr(proj), c_int(proj.stride(0)), c_int(q_off), c_int(k_off), c_int(v_off), _ptr(positions),
                                          _ptr(inv_freq if rotary_dim else None), _ptr(out), c_int(n), c_int(heads), c_int(key_dim), c_int(value_dim),
                                          c_int(rotary_dim), c_int(1 if interleaved else 0), c_float(factor), c_float(key_scale),
                                          c_int(_dtype_code(proj)), _stream()), "retention_prep")
    return out


RETENTION_MAX_KEY_DIM = 512  # key channels of a head that ``retention_scan`` takes (a column's channels are 8 to a lane of one wave)


def retention_scan(qkv: torch.Tensor, decay: torch.Tensor, state: torch.Tensor, qo_indptr, state_slots, heads: int, key_dim: int, value_dim: int,
                   out: torch.Tensor) -> torch.Tensor:
    """S <- decay_h S + k v^T and out = S^T q per head over every request's tokens of the step in order.  ``qkv`` float32
    [tokens, heads * (2 key_dim + value_dim)] as ``retention_prep`` leaves it; ``decay`` float32 [heads]; ``state`` float32
    [slots, >= heads * value_dim * key_dim], a request's S as [heads, value_dim, key_dim] in its slot; ``out`` float32 [tokens,
    heads * value_dim]."""
    _f32(qkv, "qkv"), _f32(decay, "decay"), _f32(out, "out"), _i32(qo_indptr, "qo_indptr"), _i32(state_slots, "state_slots")
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or not state.is_cuda:
        raise KernelRefused("retention_scan: the state is float32 [slots, floats per slot] on the GPU")
    stride = state.shape[1]
    n = qkv.shape[0]
    if (key_dim > RETENTION_MAX_KEY_DIM or qkv.shape != (n, heads * (2 * key_dim + value_dim)) or decay.numel() != heads or out.shape != (n, heads * value_dim)
            or stride < heads * key_dim * value_dim or qo_indptr.numel() != state_slots.numel() + 1):
        raise KernelRefused(f"retention_scan: operands do not fit {heads} heads of {key_dim} x {value_dim} (key sizes up to {RETENTION_MAX_KEY_DIM})")
    _check(build.core().ns_retention_scan(_ptr(qkv), _ptr(decay), _ptr(state), ctypes.c_longlong(stride), _ptr(qo_indptr), _ptr(state_slots), _ptr(out),
                                          c_int(state_slots.numel()), c_int(heads), c_int(key_dim), c_int(value_dim), _stream()), "retention_scan")
    return out


def gate_mul(x: torch.Tensor, gate: torch.Tensor, out: torch.Tensor, silu: bool = False) -> torch.Tensor:
    """out = x * sigmoid(gate), or x * gate * sigmoid(gate) with ``silu``, the gate formed in 32-bit; ``gate`` may be a column
    slice of wider rows; ``x`` and ``out`` contiguous [tokens, width] (they may be one tensor)."""
    _gpu(x, gate, out)
    n, width = x.shape
    if (not x.is_contiguous() or out.shape != x.shape or not out.is_contiguous() or out.dtype != x.dtype or gate.dtype != x.dtype or gate.shape != x.shape
            or gate.stride(1) != 1):
        raise KernelRefused("gate_mul: x and out contiguous [tokens, width], gate [tokens, width] of the same dtype")
    _check(build.core().ns_gate_mul(_ptr(out), _ptr(x), _ptr(gate), c_int(gate.stride(0)), c_int(n), c_int(width), c_int(1 if silu else 0),
                                    c_int(_dtype_code(x)), _stream()), "gate_mul")
    return out


def moe_route(h: torch.Tensor, router: torch.Tensor, bias: torch.Tensor | None, top: int, sel: torch.Tensor, weights: torch.Tensor,
              logits: torch.Tensor | None = None, sigmoid: bool = False, correction: torch.Tensor | None = None, groups: int = 1,
              keep: int = 1) -> None:
    """Router logits z = router h + bias in 32-bit (``router`` float32 [experts, W]); ``sel`` int32 [tokens, top] receives the
    experts with the largest logits in falling order, ``weights`` float32 [tokens, top] the soft-max over those logits.
    ``logits``: float32 [tokens, experts], receives z (scratch if the caller has no use for it).
    ``sigmoid``: the scores are s = sigmoid(z), the choice goes by s + ``correction`` (float32 [experts] or None) and the
    weights are the chosen s themselves.  ``groups`` > 1: only experts of the ``keep`` groups (of experts / groups neighbours)
    with the largest sums of their two best choice scores can be chosen."""
    _gpu(h, router, bias, sel, weights, logits, correction)
    if correction is not None and (not sigmoid or _f32(correction, "correction").numel() != router.shape[0]):
        raise KernelRefused("moe_route: a correction [experts] belongs to sigmoid scores")
    if groups < 1 or router.shape[0] % groups or not 1 <= keep <= groups or top > keep * (router.shape[0] // groups):
        raise KernelRefused(f"moe_route: {router.shape[0]} experts in {groups} groups of which {keep} are kept, {top} chosen")
    _f32(router, "router"), _f32(weights, "weights"), _i32(sel, "sel")
    n, W = h.shape
    experts = router.shape[0]
    if logits is None:
        logits = torch.empty((n, experts), dtype=torch.float32, device=h.device)
    if (h.stride(1) != 1 or router.shape != (experts, W) or not router.is_contiguous() or sel.shape != (n, top) or weights.shape != (n, top)
            or (bias is not None and _f32(bias, "bias").numel() != experts) or _f32(logits, "logits").shape != (n, experts) or not logits.is_contiguous()):
        raise KernelRefused("moe_route: h [tokens, W], router [experts, W], bias [experts], sel and weights [tokens, top], logits [tokens, experts]")
    _check(build.core().ns_moe_route(_ptr(h), c_int(h.stride(0)), _ptr(router), _ptr(bias), _ptr(logits), _ptr(sel), _ptr(weights), c_int(n), c_int(W),
                                     c_int(experts), c_int(top), c_int(1 if sigmoid else 0), _ptr(correction), c_int(groups), c_int(keep),
                                     c_int(_dtype_code(h)), _stream()), "moe_route")


def moe_expert_rows(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, sel: torch.Tensor, weights: torch.Tensor,
                    limit: float, alpha: float, act: torch.Tensor, out: torch.Tensor, shift: float = 1.0) -> torch.Tensor:
    """out[t, k] = weights[t, k] * expert sel[t, k] of h[t], for few rows: every (token, chosen expert) streams that expert's
    matrices, cut into slices over many workgroups.  ``gate``, ``up`` [experts, ff, W], ``down`` [experts, W, ff] in the dtype
    of ``h``; ``act`` float32 [tokens, top, ff] (scratch); ``out`` float32 [tokens, top, W]."""
    _gpu(h, gate, up, down, sel, weights, act, out)
    _f32(out, "out"), _f32(act, "act"), _f32(weights, "weights"), _i32(sel, "sel")
    n, W = h.shape
    experts, ff = gate.shape[0], gate.shape[1]
    top = sel.shape[1]
    if (h.stride(1) != 1 or gate.shape != (experts, ff, W) or up.shape != gate.shape or down.shape != (experts, W, ff) or sel.shape != (n, top)
            or weights.shape != (n, top) or out.shape != (n, top, W) or act.shape != (n, top, ff)
            or any(t.dtype != h.dtype or not t.is_contiguous() for t in (gate, up, down))):
        raise KernelRefused("moe_expert_rows: gate and up [experts, ff, W], down [experts, W, ff] in the dtype of h; act [tokens, top, ff] and out [tokens, top, W] float32")
    _check(build.core().ns_moe_expert_rows(_ptr(h), c_int(h.stride(0)), _ptr(gate), _ptr(up), _ptr(down), _ptr(sel), _ptr(weights), _ptr(act),
                                           _ptr(out), c_int(n), c_int(W), c_int(ff), c_int(top), c_float(limit), c_float(alpha), c_float(shift),
                                           c_int(_dtype_code(h)), _stream()), "moe_expert_rows")
    return out


def moe_groups_take(h: torch.Tensor, ff: int) -> bool:
    """Whether the matrix-core kernels for many rows take this input: bfloat16, sizes in multiples of 8."""
    return h.dtype == torch.bfloat16 and h.shape[1] % 8 == 0 and ff % 8 == 0 and h.stride(0) % 8 == 0 and h.data_ptr() % 16 == 0


def moe_expert_groups(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, sel: torch.Tensor, weights: torch.Tensor,
                      limit: float, alpha: float, ints: torch.Tensor, act: torch.Tensor, out: torch.Tensor, shift: float = 1.0) -> torch.Tensor:
    """The same result for many rows in bfloat16: the pairs are sorted by expert on the device and every expert multiplies
    its rows in tiles on the matrix cores.  ``ints`` int32 [tokens * top + 3 * moe_group_tiles] and ``act`` bfloat16
    [tokens * top, ff] are scratch."""
    _gpu(h, gate, up, down, sel, weights, ints, act, out)
    _f32(out, "out"), _f32(weights, "weights"), _i32(sel, "sel"), _i32(ints, "ints")
    n, W = h.shape
    experts, ff = gate.shape[0], gate.shape[1]
    top = sel.shape[1]
    tiles = int(build.core().ns_moe_group_tiles(c_int(n * top), c_int(experts)))
    if (not moe_groups_take(h, ff) or h.stride(1) != 1 or gate.shape != (experts, ff, W) or up.shape != gate.shape or down.shape != (experts, W, ff)
            or sel.shape != (n, top) or weights.shape != (n, top) or out.shape != (n, top, W) or act.shape != (n * top, ff) or act.dtype != h.dtype
            or not act.is_contiguous() or ints.numel() < n * top + 3 * tiles or any(t.dtype != h.dtype or not t.is_contiguous() for t in (gate, up, down))):
        raise KernelRefused("moe_expert_groups: bfloat16 operands with sizes in multiples of 8, act [pairs, ff], ints [pairs + 3 tiles]")
    _check(build.core().ns_moe_expert_groups(_ptr(h), c_int(h.stride(0)), _ptr(gate), _ptr(up), _ptr(down), _ptr(sel), _ptr(weights), _ptr(ints),
                                             _ptr(act), _ptr(out), c_int(n), c_int(W), c_int(ff), c_int(top), c_int(experts), c_float(limit),
                                             c_float(alpha), c_float(shift), _stream()), "moe_expert_groups")
    return out


def moe_experts(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, sel: torch.Tensor, weights: torch.Tensor,
                limit: float, alpha: float, take, shift: float = 1.0) -> torch.Tensor:
    """The chosen experts' weighted outputs, float32 [tokens, top, W], by the kernels that suit the number of rows: with
    fewer (token, expert) pairs than experts every pair streams its expert's matrices; from there on the sorted, tiled
    product reads every matrix at most once.  ``take(shape, dtype)`` gives scratch that lives as long as the result."""
    n, W = h.shape
    experts, ff = gate.shape[0], gate.shape[1]
    top = sel.shape[1]
    out = take((n, top, W), torch.float32)
    if n * top >= max(experts, 16) and moe_groups_take(h, ff):
        tiles = int(build.core().ns_moe_group_tiles(c_int(n * top), c_int(experts)))
        return moe_expert_groups(h, gate, up, down, sel, weights, limit, alpha, take((n * top + 3 * tiles,), torch.int32),
                                 take((n * top, ff), h.dtype), out, shift=shift)
    return moe_expert_rows(h, gate, up, down, sel, weights, limit, alpha, take((n, top, ff), torch.float32), out, shift=shift)


def clipped_glu(gu: torch.Tensor, limit: float, alpha: float, out: torch.Tensor, shift: float = 1.0) -> torch.Tensor:
    """out = g sigmoid(alpha g) (u + shift) with g = min(gu[:, :ff], limit), u = clamp(gu[:, ff:], -limit, limit) (an infinite
    limit clips nothing)."""
    _gpu(gu, out)
    n, ff = out.shape
    if gu.shape != (n, 2 * ff) or gu.stride(1) != 1 or not out.is_contiguous() or out.dtype != gu.dtype:
        raise KernelRefused("clipped_glu: gu [tokens, 2 ff], out [tokens, ff] of the same dtype")
    _check(build.core().ns_clipped_glu(_ptr(out), _ptr(gu), c_int(gu.stride(0)), c_int(n), c_int(ff), c_float(limit), c_float(alpha), c_float(shift),
                                       c_int(_dtype_code(gu)), _stream()), "clipped_glu")
    return out


def moe_combine(parts: torch.Tensor, base: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[t] = base[t] + sum_k parts[t, k] (``parts`` float32 [tokens, top, W]; ``base`` and ``out`` in the model's dtype)."""
    _gpu(parts, base, out)
    _f32(parts, "parts")
    n, top, W = parts.shape
    if out.shape != (n, W) or not out.is_contiguous() or (base is not None and (base.shape != (n, W) or not base.is_contiguous() or base.dtype != out.dtype)):
        raise KernelRefused("moe_combine: base and out are contiguous [tokens, W] of one dtype")
    _check(build.core().ns_moe_combine(_ptr(out), _ptr(base), _ptr(parts), c_int(n), c_int(top), c_int(W), c_int(_dtype_code(out)), _stream()),
           "moe_combine")
    return out


def scaled_sum(a: torch.Tensor, b: torch.Tensor, sa: float, sb: float, out: torch.Tensor, bias: torch.Tensor | None = None,
               bias_b: torch.Tensor | None = None) -> torch.Tensor:
    """out = sa * (a + bias) + sb * (b + bias_b), formed in 32-bit (the biases [W] or None)."""
    _gpu(a, b, out, bias, bias_b)
    n, W = a.shape
    if any(t.shape != (n, W) or not t.is_contiguous() or t.dtype != a.dtype for t in (b, out)) or not a.is_contiguous():
        raise KernelRefused("scaled_sum: a, b and out are contiguous [tokens, W] of one dtype")
    for t in (bias, bias_b):
        if t is not None and (t.numel() != W or t.dtype != a.dtype or not t.is_contiguous()):
            raise KernelRefused("scaled_sum: a bias is [W] of the same dtype")
    _check(build.core().ns_scaled_sum(_ptr(out), _ptr(a), _ptr(b), _ptr(bias), _ptr(bias_b), c_float(sa), c_float(sb), c_int(n), c_int(W),
                                      c_int(_dtype_code(a)), _stream()), "scaled_sum")
    return out


def gelu_gather_mul(g: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = gelu_tanh(g[t]) * table[ids[t]]: ``g`` [tokens, dim] (may be a column slice), ``table`` [vocab, dim]."""
    _gpu(g, ids, table, out)
    _i32(ids, "ids")
    n, dim = out.shape
    if (g.shape != (n, dim) or g.stride(1) != 1 or ids.numel() != n or table.dim() != 2 or table.shape[1] != dim or not table.is_contiguous()
            or not out.is_contiguous() or table.dtype != g.dtype or out.dtype != g.dtype):
        raise KernelRefused("gelu_gather_mul: g and out [tokens, dim], table [vocab, dim], all of one dtype")
    _check(build.core().ns_gelu_gather_mul(_ptr(out), _ptr(g), c_int(g.stride(0)), _ptr(ids), _ptr(table), c_int(n), c_int(dim),
                                           c_int(_dtype_code(g)), _stream()), "gelu_gather_mul")
    return out


def silu_mul_bias(gu: torch.Tensor, bias: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[n, i] = silu(gu[n, i] + bias[i]) * (gu[n, I + i] + bias[I + i]) for gu [N, 2 I]."""
    _gpu(gu, bias)
    n, two_i = gu.shape
    inter = two_i // 2
    if two_i % 2 or not gu.is_contiguous() or bias.shape != (two_i,) or not bias.is_contiguous() or bias.dtype != gu.dtype:
        raise KernelRefused("silu_mul_bias: gu must be contiguous [N, 2 I], bias [2 I] of its dtype")
    if out is None:
        out = torch.empty((n, inter), dtype=gu.dtype, device=gu.device)
    if out.shape != (n, inter) or not out.is_contiguous() or out.dtype != gu.dtype:
        raise KernelRefused("silu_mul_bias: out must be contiguous [N, I]")
    _check(build.core().ns_silu_mul_bias(_ptr(out), _ptr(gu), _ptr(bias), c_int(n), c_int(inter), c_int(_dtype_code(gu)), _stream()), "silu_mul_bias")
    return out


def add_bias(out: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """out[n, :] += bias, in place."""
    _gpu(out, bias)
    if out.dim() != 2 or out.stride(1) != 1 or bias.shape != (out.shape[1],) or not bias.is_contiguous() or bias.dtype != out.dtype:
        raise KernelRefused("add_bias: out [N, W] and bias [W] of one dtype")
    _check(build.core().ns_add_bias(_ptr(out), c_int(out.stride(0)), _ptr(bias), c_int(out.shape[0]), c_int(out.shape[1]), c_int(_dtype_code(out)),
                                    _stream()), "add_bias")
    return out


def latent_prep(proj: torch.Tensor, q_norm: torch.Tensor, c_norm: torch.Tensor, inv_freq: torch.Tensor, factor: float, positions, token_req,
                block_table, k_cache, v_cache, q_rank: int, latent: int, rot: int, heads: int, eps: float, cq: torch.Tensor,
                gate: torch.Tensor | None) -> None:
    """What a latent-attention layer does to a token's row [q_rank | latent | rot | heads] of its first product: the first
    q_rank values RMS-normed with ``q_norm`` into ``cq``; the next ``latent`` RMS-normed with ``c_norm`` and the ``rot`` behind
    them rotated by the position (pair i, i + rot/2; ``factor`` on cosine and sine) into the K page as one key [latent + rot];
    the normed latent also into the V page; sigmoid of the last ``heads`` values into ``gate`` (float32; ``heads`` = 0 and None for a
    layer without gates)."""
    _gpu(proj, q_norm, c_norm, inv_freq, positions, token_req, block_table, k_cache, v_cache, cq, gate)
    n = positions.numel()
    width = q_rank + latent + rot + heads
    _i32(positions, "positions"), _i32(token_req, "token_req"), _i32(block_table, "block_table"), _f32(inv_freq, "inv_freq")
    if (gate is None) != (heads == 0) or (gate is not None and _f32(gate, "gate").shape != (n, heads)):
        raise KernelRefused(f"latent_prep: gate is float32 [{n}, {heads}] (None without gates)")
    if proj.dim() != 2 or proj.shape[0] != n or proj.shape[1] < width or proj.stride(1) != 1:
        raise KernelRefused(f"latent_prep: the projected rows must be [{n}, {width}]")
    page = k_cache.shape[2] if k_cache.dim() == 4 else 0
    if (k_cache.dim() != 4 or k_cache.shape[1:] != (1, page, latent + rot) or v_cache.shape != (k_cache.shape[0], 1, latent, page)
            or k_cache.dtype != proj.dtype or v_cache.dtype != proj.dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
        raise KernelRefused("latent_prep: the pages hold one key of latent + rot channels and one value of latent channels per token")
    if q_rank == 0:
        q_norm = cq = None  # no query latent: the layer's queries are projected from its input
    elif (q_norm.shape != (q_rank,) or q_norm.dtype != proj.dtype or not q_norm.is_contiguous() or cq.shape != (n, q_rank) or cq.dtype != proj.dtype
          or not cq.is_contiguous()):
        raise KernelRefused("latent_prep: the query latent's norm weight or output does not fit its size")
    if (c_norm.shape != (latent,) or c_norm.dtype != proj.dtype
            or not c_norm.is_contiguous()
            or rot % 2 or inv_freq.numel() < max(1, rot // 2) or token_req.numel() != n or block_table.dim() != 2 or block_table.stride(1) != 1):
        raise KernelRefused("latent_prep: norm weights, outputs or frequencies do not fit the sizes")
    _check(build.core().ns_latent_prep(_ptr(proj), c_int(proj.stride(0)), _ptr(q_norm), _ptr(c_norm), _ptr(inv_freq), c_float(factor), _ptr(cq),
                                       _ptr(gate), _ptr(positions), _ptr(token_req), _ptr(block_table), c_int(block_table.stride(0)),
                                       _ptr(k_cache), _ptr(v_cache), c_int(n), c_int(q_rank), c_int(latent), c_int(rot), c_int(heads),
                                       c_int(page), c_float(eps), c_int(_dtype_code(proj)), _stream()), "latent_prep")


def headwise_takes(dtype, n_out: int, k: int, x_head: int, out_head: int) -> bool:
    """Whether ``headwise_product`` takes these sizes: bfloat16, K a multiple of 32, N of 16, heads 16 and 8 bytes apart."""
    return dtype == torch.bfloat16 and k % 32 == 0 and n_out % 16 == 0 and x_head % 8 == 0 and out_head % 4 == 0


def headwise_product(x: torch.Tensor, x_head: int, w: torch.Tensor, out: torch.Tensor, out_head: int, gate: torch.Tensor | None = None) -> torch.Tensor:
    """One product per head on the matrix cores: out[t, h * out_head + n] = gate[t, h] * sum_k x[t, h * x_head + k] w[h, n, k]
    for w [heads, N, K] (bfloat16).  A head's part of a row of ``x`` may be wider than K and of ``out`` wider than N: the
    rest is not read and not written."""
    _gpu(x, w, out, gate)
    H, N, K = w.shape
    n = x.shape[0]
    if (x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or not w.is_contiguous() or x.dim() != 2 or out.dim() != 2
            or x.stride(1) != 1 or out.stride(1) != 1 or out.shape[0] != n or x.shape[1] < (H - 1) * x_head + K or out.shape[1] < (H - 1) * out_head + N
            or K > x_head or N > out_head or not headwise_takes(x.dtype, N, K, x_head, out_head) or x.stride(0) % 8 or out.stride(0) % 4):
        raise KernelRefused("headwise_product: bfloat16 x [tokens, heads * x_head], w [heads, N, K] with K a multiple of 32 and N of 16")
    if gate is not None and _f32(gate, "gate").shape != (n, H):
        raise KernelRefused(f"headwise_product: gate is float32 [{n}, {H}]")
    _check(build.core().ns_headwise_bf16(_ptr(x), ctypes.c_long(x.stride(0)), c_int(x_head), _ptr(w), _ptr(gate), _ptr(out),
                                         ctypes.c_long(out.stride(0)), c_int(out_head), c_int(n), c_int(H), c_int(N), c_int(K), _stream()),
           "headwise_product")
    return out


def latent_q_absorb(q: torch.Tensor, uk: torch.Tensor | None, inv_freq: torch.Tensor, factor: float, positions, heads: int, dim: int, rot: int,
                    latent: int, out: torch.Tensor) -> torch.Tensor:
    """q [tokens, heads * (dim + rot)] -> out [tokens, heads * (latent + rot)]: per head, the first ``dim`` values through
    that head's key matrix, out[c] = sum_d q[d] uk[head * dim + d, c] (``uk`` [heads * dim, latent]), and the ``rot`` values
    behind them rotated by the position.  ``uk`` = None: the rotation alone (the product is the caller's)."""
    _gpu(q, uk, inv_freq, positions, out)
    n = positions.numel()
    _i32(positions, "positions"), _f32(inv_freq, "inv_freq")
    absorb = uk is not None
    if uk is None:
        uk = torch.empty((heads * dim, latent), dtype=q.dtype, device="meta")
    if (q.dim() != 2 or q.shape != (n, heads * (dim + rot)) or q.stride(1) != 1 or uk.shape != (heads * dim, latent) or not uk.is_contiguous()
            or uk.dtype != q.dtype or out.shape != (n, heads * (latent + rot)) or not out.is_contiguous() or out.dtype != q.dtype or rot % 2
            or inv_freq.numel() < max(1, rot // 2) or dim > 2048):
        raise KernelRefused("latent_q_absorb: q [tokens, heads * (dim + rot)], uk [heads * dim, latent], out [tokens, heads * (latent + rot)]")
    _check(build.core().ns_latent_q_absorb(_ptr(q), c_int(q.stride(0)), _ptr(uk if absorb else None), _ptr(inv_freq), c_float(factor),
                                           _ptr(positions), _ptr(out), c_int(n), c_int(heads), c_int(dim), c_int(rot), c_int(latent),
                                           c_int(1 if absorb else 0), c_int(_dtype_code(q)), _stream()),
           "latent_q_absorb")
    return out


def latent_out(o: torch.Tensor, uv_t: torch.Tensor, gate: torch.Tensor | None, heads: int, latent: int, v_dim: int, out: torch.Tensor) -> torch.Tensor:
    """o [tokens, heads * latent] -> out [tokens, heads * v_dim]: out[h, e] = gate[h] * sum_c o[h, c] uv_t[h, c, e]
    (``uv_t`` [heads, latent, v_dim]; ``gate`` float32 [tokens, heads] or None)."""
    _gpu(o, uv_t, gate, out)
    n = o.shape[0]
    if gate is not None:
        _f32(gate, "gate")
    if (o.dim() != 2 or o.shape != (n, heads * latent) or not o.is_contiguous() or uv_t.shape != (heads, latent, v_dim) or not uv_t.is_contiguous()
            or uv_t.dtype != o.dtype or out.shape != (n, heads * v_dim) or not out.is_contiguous() or out.dtype != o.dtype
            or (gate is not None and gate.shape != (n, heads)) or latent > 2048):
        raise KernelRefused("latent_out: o [tokens, heads * latent], uv_t [heads, latent, v_dim], out [tokens, heads * v_dim]")
    _check(build.core().ns_latent_out(_ptr(o), _ptr(uv_t), _ptr(gate), _ptr(out), c_int(n), c_int(heads), c_int(latent), c_int(v_dim),
                                      c_int(_dtype_code(o)), _stream()), "latent_out")
    return out


def activation(x: torch.Tensor, kind: str, out: torch.Tensor | None = None) -> torch.Tensor:
    """out = act(x) element by element (in place by default); ``kind`` one of ``ACTIVATIONS``."""
    _gpu(x, out)
    if kind not in ACTIVATIONS:
        raise KernelRefused(f"activation {kind!r} is not known (known: {sorted(ACTIVATIONS)})")
    out = x if out is None else out
    if not x.is_contiguous() or not out.is_contiguous() or out.shape != x.shape or out.dtype != x.dtype:
        raise KernelRefused("activation: x and out must be contiguous and alike")
    _check(build.core().ns_activation(_ptr(out), _ptr(x), c_size_t(x.numel()), c_int(ACTIVATIONS[kind]), c_int(_dtype_code(x)), _stream()),
           "activation")
    return out


# ------------------------------------------------------------------------------------------------ delta rule

MAX_CONV_TAPS = 16
DELTA_MAX_KEY_DIM = 1024


def _state_args(state: torch.Tensor, what: str):
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or not state.is_cuda:
        raise KernelRefused(f"{what}: the state is float32 [slots, floats per slot] on the GPU")
    return _ptr(state), c_size_t(state.shape[1])


def conv_silu_carry(x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, conv_off: int, token_req, qo_indptr, state_slots,
                    out: torch.Tensor) -> torch.Tensor:
    """A short causal convolution over time per channel, then SiLU, across steps.  ``x`` [tokens, >= C] (its first C columns
    are convolved), ``taps`` float32 [C, K] whose last column multiplies the current token; the K - 1 inputs before a
    request's first token of this step are read from ``state[slot, conv_off:]`` as [K - 1, C] (zeros for a new request)
    and replaced afterwards by the last K - 1 inputs including this step's.  ``out`` float32 [tokens, C]."""
    _gpu(x), _f32(taps, "taps"), _f32(out, "out")
    for name, t in (("token_req", token_req), ("qo_indptr", qo_indptr), ("state_slots", state_slots)):
        _i32(t, name)
    C, K = taps.shape
    n, reqs = token_req.numel(), state_slots.numel()
    if x.dim() != 2 or x.shape[0] != n or x.shape[1] < C or x.stride(1) != 1 or out.shape != (n, C) or qo_indptr.numel() != reqs + 1:
        raise KernelRefused("conv_silu_carry: x is [tokens, >= C], out float32 [tokens, C], qo_indptr [requests + 1]")
    if K > MAX_CONV_TAPS or conv_off + (K - 1) * C > state.shape[1]:
        raise KernelRefused(f"conv_silu_carry: at most {MAX_CONV_TAPS} taps, and the carried inputs must fit the slot")
    sp, stride = _state_args(state, "conv_silu_carry")
    _check(build.core().ns_conv_silu_carry(_ptr(out), _ptr(x), c_int(x.stride(0)), _ptr(taps), sp, stride, c_size_t(conv_off), _ptr(token_req),
                                           _ptr(qo_indptr), _ptr(state_slots), c_int(n), c_int(reqs), c_int(C), c_int(K),
                                           c_int(_dtype_code(x)), _stream()), "conv_silu_carry")
    return out


def delta_prep(qkv: torch.Tensor, a: torch.Tensor, b: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, heads: int, kv_heads: int,
               key_dim: int, g: torch.Tensor, beta: torch.Tensor) -> None:
    """What the delta rule's recurrence reads, in 32-bit.  In place in ``qkv`` (float32 [tokens, C], q [kv_heads, key_dim]
    then k alike then v): q and k of every head become x / sqrt(sum(x^2) + 1e-6), q times key_dim^(-1/2).
    g[t, h, d] = exp(-exp(a_log[h]) * softplus(a[t, h, d] + dt_bias[h, d])); beta[t, h] = sigmoid(b[t, h]).
    ``a`` [tokens, >= heads * key_dim] and ``b`` [tokens, >= heads] may be column slices of wider tensors."""
    _f32(qkv, "qkv"), _f32(g, "g"), _f32(beta, "beta"), _f32(dt_bias, "dt_bias"), _f32(a_log, "a_log")
    _gpu(a, b)
    n = qkv.shape[0]
    if (qkv.dim() != 2 or qkv.shape[1] < 2 * kv_heads * key_dim or a.dtype != b.dtype or a.stride(1) != 1 or b.stride(1) != 1
            or a.shape[0] != n or b.shape[0] != n or a.shape[1] < heads * key_dim or b.shape[1] < heads or g.shape != (n, heads * key_dim)
            or beta.shape != (n, heads) or dt_bias.numel() != heads * key_dim or a_log.numel() != heads or heads % kv_heads):
        raise KernelRefused("delta_prep: operands do not fit heads and key size")
    _check(build.core().ns_delta_prep(_ptr(qkv), c_int(qkv.shape[1]), _ptr(g), _ptr(beta), _ptr(a), c_int(a.stride(0)), _ptr(b),
                                      c_int(b.stride(0)), _ptr(dt_bias), _ptr(a_log), c_int(n), c_int(heads), c_int(kv_heads), c_int(key_dim),
                                      c_int(_dtype_code(a)), _stream()), "delta_prep")


def delta_scan(qkv: torch.Tensor, g: torch.Tensor, beta: torch.Tensor, state: torch.Tensor, qo_indptr, state_slots, heads: int,
               kv_heads: int, key_dim: int, value_dim: int, out: torch.Tensor) -> torch.Tensor:
    """The gated delta rule over every request's tokens of this step, from and into ``state[slot, : heads * key_dim *
    value_dim]`` (S [heads, key_dim, value_dim] per request): S = g_t * S (by key channel); u = beta_t (v_t - S^T k_t);
    S = S + k_t u^T; o_t = S^T q_t.  ``qkv`` as ``delta_prep`` leaves it; ``out`` float32 [tokens, heads * value_dim]."""
    _f32(qkv, "qkv"), _f32(g, "g"), _f32(beta, "beta"), _f32(out, "out")
    _i32(qo_indptr, "qo_indptr"), _i32(state_slots, "state_slots")
    n, reqs = qkv.shape[0], state_slots.numel()
    C = 2 * kv_heads * key_dim + heads * value_dim
    if (qkv.shape != (n, C) or g.shape != (n, heads * key_dim) or beta.shape != (n, heads) or out.shape != (n, heads * value_dim)
            or qo_indptr.numel() != reqs + 1 or heads % kv_heads or key_dim > DELTA_MAX_KEY_DIM
            or state.shape[1] < heads * key_dim * value_dim):
        raise KernelRefused("delta_scan: operands do not fit heads, key size and value size")
    sp, stride = _state_args(state, "delta_scan")
    _check(build.core().ns_delta_scan(_ptr(out), _ptr(qkv), c_int(C), _ptr(g), _ptr(beta), sp, stride, _ptr(qo_indptr), _ptr(state_slots),
                                      c_int(reqs), c_int(heads), c_int(kv_heads), c_int(key_dim), c_int(value_dim), _stream()), "delta_scan")
    return out


def gated_rms(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor | None, eps: float, heads: int, out: torch.Tensor,
              den: torch.Tensor | None = None, silu: bool = False) -> torch.Tensor:
    """out[t, h, :] = x / sqrt(mean(x^2) + eps) * weight * sigmoid(gate[t, h, :]) with x = o[t, h, :], or o[t, h, :] /
    den[t, h] if ``den`` (float32 [tokens, heads]) is given; ``o`` float32 [tokens, heads * E], ``weight`` float32 [E] (all
    heads share it) or [heads * E] or None (no weight), ``gate`` (may be a column slice) and ``out`` in the model's dtype.
    ``silu``: the gate is g sigmoid(g) instead of sigmoid(g)."""
    _f32(o, "o")
    if weight is not None:
        _f32(weight, "weight")
    _gpu(gate, out, den)
    n, width = o.shape
    if (width % heads or (weight is not None and weight.numel() not in (width // heads, width)) or gate.shape[0] != n or gate.shape[1] < width or gate.stride(1) != 1
            or out.shape != (n, width) or not out.is_contiguous() or out.dtype != gate.dtype
            or (den is not None and (_f32(den, "den").shape != (n, heads) or not den.is_contiguous()))):
        raise KernelRefused("gated_rms: operands do not fit heads and value size")
    per_head = width // heads if (weight is not None and weight.numel() == width and heads > 1) else 0
    _check(build.core().ns_gated_rms(_ptr(out), _ptr(o), _ptr(gate), c_int(gate.stride(0)), _ptr(weight), c_int(per_head), _ptr(den), c_int(n),
                                     c_int(heads), c_int(width // heads), c_float(eps), c_int(1 if silu else 0), c_int(_dtype_code(gate)), _stream()),
           "gated_rms")
    return out


# ------------------------------------------------------------------------------------------------ sampling


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor, top_k: torch.Tensor | None = None,
           top_p: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """Per row of float32 ``logits``: arg-max when temperature is 0, else a draw by inverse CDF with the row's uniform
    number.  -> int32 [3, rows]: row 0 the tokens, row 1 the bits of the float32 log-probability of the token under the
    raw logits, row 2 the bits of its float32 log-probability under the processed distribution (0 for arg-max rows)."""
    _gpu(logits, temperature, uniform, top_k, top_p, out)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelRefused("sample: logits must be float32 [rows, vocab]")
    rows, vocab = logits.shape
    for name, t, dt in (("temperature", temperature, torch.float32), ("uniform", uniform, torch.float32),
                        ("top_k", top_k, torch.int32), ("top_p", top_p, torch.float32)):
        if t is not None and (t.dtype != dt or t.numel() != rows or not t.is_contiguous()):
            raise KernelRefused(f"sample: {name} must hold one {dt} per row")
    if out is None:
        out = torch.empty((3, rows), dtype=torch.int32, device=logits.device)
    if out.dtype != torch.int32 or out.shape != (3, rows) or not out.is_contiguous():
        raise KernelRefused("sample: out must be a contiguous int32 [3, rows]")
    _check(build.core().ns_sample(_ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _ptr(logits), c_int(logits.stride(0)), _ptr(temperature),
                                  _ptr(top_k), _ptr(top_p), _ptr(uniform), c_int(rows), c_int(vocab), _stream()), "sample")
    return out


def unpack_sample(packed: torch.Tensor):
    """int32 [3, rows] of ``sample`` -> (tokens int32, log-probabilities float32, processed log-probabilities float32)."""
    return packed[0], packed[1].view(torch.float32), packed[2].view(torch.float32)


# ------------------------------------------------------------------------------------------------ graphs


class Graph:
    """A captured stream of launches.  ``with Graph.capture(stream) as g: ...`` then ``g.launch()``."""

    def __init__(self, stream: torch.cuda.Stream) -> None:
        self.stream, self._exec = stream, None

    def __enter__(self):
        self._ctx = torch.cuda.stream(self.stream)
        self._ctx.__enter__()
        _check(build.core().ns_graph_begin(c_void_p(self.stream.cuda_stream)), "graph capture begin")
        return self

    def __exit__(self, et, ev, tb):
        handle = c_void_p()
        code = build.core().ns_graph_end(c_void_p(self.stream.cuda_stream), ctypes.byref(handle))
        self._ctx.__exit__(et, ev, tb)
        if et is None:
            _check(code, "graph capture end")
            self._exec = handle
        return False

    def launch(self) -> None:
        _check(build.core().ns_graph_launch(self._exec, c_void_p(self.stream.cuda_stream)), "graph launch")

    def __del__(self):
        if getattr(self, "_exec", None):
            try:
                build.core().ns_graph_destroy(self._exec)
            except Exception:
                pass
