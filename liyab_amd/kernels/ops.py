"""The kernels as functions over torch tensors.

Each function checks on the host that shapes, dtypes and layouts are what
its kernel and grid assume, then launches on torch's current stream. Torch
supplies the device memory and the stream; every computation is the
library's own kernel. Nothing here runs without the GPU and the library.
"""

from __future__ import annotations

import ctypes
import struct
from typing import Optional

import torch

from ..errors import KernelError
from . import lib as _lib

F32, BF16 = 0, 1
EPI_NONE, EPI_GELU_TANH, EPI_GELU_ERF, EPI_RESIDUAL = 0, 1, 2, 3
ACTIVATION_EPILOGUE = {"none": EPI_NONE, "gelu_tanh": EPI_GELU_TANH, "gelu_erf": EPI_GELU_ERF}


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"the kernels take float32 or bfloat16, not {dt}")


_pinned_stream: Optional[int] = None


def _stream() -> int:
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class on_current_stream:
    """Within this context every launch goes to the stream that was current on entry, looked
    up once instead of at every call (a model step makes a couple of hundred launches)."""

    def __enter__(self):
        global _pinned_stream
        self._before = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self._before
        return False


_invariant = False


class batch_invariant:
    """Within this context the kernels that serve a row are chosen from the model's sizes and the
    row's own position only, never from what else the step holds: products by the tiled
    matrix-core kernels whose sums run over k in one order whatever the tile (no streaming kernel,
    no cut over K, no norm folded into a product), attention token by token with one split on
    four waves. A row's bfloat16 results then have the same bits alone and in any batch, as the
    reference promises of its passes (include/liyab/engine.h:987-990, src/core/transformer.h:746-751);
    the step-shaped choices outside this context are faster and differ from these by rounding."""

    def __init__(self, on: bool = True):
        self.on = on

    def __enter__(self):
        global _invariant
        self._before = _invariant
        _invariant = self.on
        return self

    def __exit__(self, *exc):
        global _invariant
        _invariant = self._before
        return False


def is_batch_invariant() -> bool:
    return _invariant


def _dev(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise KernelError(f"{what} must be on the GPU")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None, pinned_ok: bool = False) -> None:
    if not (pinned_ok and not t.is_cuda and t.is_pinned()):  # (pinned host memory is mapped into the device's address space)
        _dev(t, what)
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what} must be contiguous int32")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what} holds {t.numel()} values, {n} are needed")


def _f32vec(t: Optional[torch.Tensor], what: str, n: int) -> None:
    if t is None:
        return
    _dev(t, what)
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise KernelError(f"{what} must be {n} contiguous float32 values, got {tuple(t.shape)} {t.dtype}")


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    _dev(t, what)
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what} must be 2-D with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _pages(k_cache: torch.Tensor, num_pages: Optional[int]) -> int:
    """The number of pages a launcher is told the caches hold: all of them unless the caller
    counts fewer (page ids and slots beyond that count are not followed by the kernels)."""
    pages = k_cache.shape[0] if num_pages is None else int(num_pages)
    if not 0 < pages <= k_cache.shape[0]:
        raise KernelError(f"the caches hold {k_cache.shape[0]} pages, not {pages}")
    if pages * k_cache.shape[2] >= 1 << 31:
        raise KernelError(f"{pages} pages of {k_cache.shape[2]} positions: slots must fit 31 bits")
    return pages


def check_device() -> None:
    _lib.call("liyab_check_device")


def fill_(t: torch.Tensor, value: float | int) -> torch.Tensor:
    _dev(t, "fill target")
    if not t.is_contiguous():
        raise KernelError("fill target must be contiguous")
    if t.dtype == torch.float32:
        bits = struct.unpack("<I", struct.pack("<f", float(value)))[0]
        size = 4
    elif t.dtype == torch.int32:
        bits = int(value) & 0xFFFFFFFF
        size = 4
    elif t.dtype == torch.bfloat16:
        bits = struct.unpack("<I", struct.pack("<f", float(value)))[0]
        bits = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF if value == value else 0x7FC0
        size = 2
    else:
        raise KernelError(f"fill: unsupported dtype {t.dtype}")
    _lib.call("liyab_fill", t.data_ptr(), size, bits, t.numel(), _stream())
    return t


def add_into_(residual: torch.Tensor, x: torch.Tensor) -> None:
    """residual (float32) += x, elementwise."""
    _dev(residual, "residual")
    _dev(x, "x")
    if residual.dtype != torch.float32 or not residual.is_contiguous() or not x.is_contiguous():
        raise KernelError("add_into: residual must be contiguous float32 and x contiguous")
    if residual.numel() != x.numel():
        raise KernelError(f"add_into: {residual.numel()} vs {x.numel()} values")
    _lib.call("liyab_add_into", residual.data_ptr(), x.data_ptr(), dtype_code(x.dtype), x.numel(), _stream())


def embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0,
          pos_table: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
          last_tokens: Optional[torch.Tensor] = None) -> None:
    """out[t] = scale * table[ids[t]] (+ pos_table[positions[t]]); out is float32 [n, d].
    An id below zero stands for last_tokens[-1 - id]. The caller has checked ids against the
    table's rows (and positions against pos_table's)."""
    _dev(out, "out")
    n, d = out.shape
    if out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embed: out must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != d or not table.is_contiguous():
        raise KernelError(f"embed: table {tuple(table.shape)} does not have rows of {d}")
    _i32(ids, "ids", n)
    if pos_table is not None:
        if pos_table.dtype != table.dtype or pos_table.dim() != 2 or pos_table.shape[1] != d or not pos_table.is_contiguous():
            raise KernelError("embed: the position table must match the token table's dtype and width")
        if positions is None:
            raise KernelError("embed: a position table needs positions")
        _i32(positions, "positions", n)
    if last_tokens is not None:
        _i32(last_tokens, "last_tokens")
    _lib.call("liyab_embed", out.data_ptr(), table.data_ptr(), _ptr(pos_table), dtype_code(table.dtype),
              ids.data_ptr(), _ptr(positions), n, d, float(scale), _ptr(last_tokens), _stream())


def add_rows_(x: torch.Tensor, table: torch.Tensor, rows: torch.Tensor) -> None:
    """x[t] += table[rows[t]]; x is float32 [n, d]."""
    _dev(x, "x")
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("add_rows: x must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != d or not table.is_contiguous():
        raise KernelError(f"add_rows: table {tuple(table.shape)} does not have rows of {d}")
    _i32(rows, "rows", n)
    _lib.call("liyab_add_rows", x.data_ptr(), table.data_ptr(), dtype_code(table.dtype), rows.data_ptr(), n, d, _stream())


def gather_rows(out: torch.Tensor, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = x[rows[r]] (x[r] without rows) in out's dtype; x float32 [*, d], out [n, d]."""
    _dev(out, "out")
    _dev(x, "x")
    n, d = out.shape
    if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != d or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"gather_rows: x must be contiguous float32 [*, {d}] and out contiguous, got {tuple(x.shape)} {x.dtype}")
    if rows is not None:
        _i32(rows, "rows", n)
    elif x.shape[0] < n:
        raise KernelError("gather_rows: fewer input rows than output rows")
    _lib.call("liyab_gather_rows", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), _ptr(rows), n, d, _stream())


def scale_(t: torch.Tensor, scale: float) -> torch.Tensor:
    """t *= scale; t contiguous float32."""
    _dev(t, "scale target")
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise KernelError("scale: the target must be contiguous float32")
    _lib.call("liyab_scale", t.data_ptr(), float(scale), t.numel(), _stream())
    return t


def _planes(x: torch.Tensor, what: str):
    """Rows given as they are, float32 [rows, d], or as a sum of planes, float32 [parts, rows, d]
    (row r is x[0][r] + x[1][r] + ..., added in that order). Returns (pointer, parts, floats
    between planes, rows, d)."""
    _dev(x, what)
    if x.dtype != torch.float32 or x.dim() not in (2, 3) or not x.is_contiguous():
        raise KernelError(f"{what}: rows must be contiguous float32 [rows, d] or [parts, rows, d], got {tuple(x.shape)} {x.dtype}")
    if x.dim() == 2:
        return x.data_ptr(), 1, 0, x.shape[0], x.shape[1]
    if not 1 <= x.shape[0] <= 16:
        raise KernelError(f"{what}: {x.shape[0]} planes (1 to 16)")
    return x.data_ptr(), x.shape[0], x.stride(0), x.shape[1], x.shape[2]


def norm_takes_planes(d: int) -> bool:
    """Whether the norm kernel adds planes up as it loads a row of this width (sum_parts first otherwise)."""
    return d % 4 == 0 and d <= 16384


def layernorm(out: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
              eps: float, rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = LayerNorm(x[rows[r]] or x[r]); x float32 [*, d], out [n, d] float32 or bfloat16.
    x may be a sum of planes [parts, *, d] (widths that `norm_takes_planes`): the planes are
    added up, in their order, as a row is loaded."""
    _dev(out, "out")
    ptr, n_parts, stride, x_rows, xd = _planes(x, "layernorm")
    n, d = out.shape
    if xd != d or not out.is_contiguous():
        raise KernelError("layernorm: x must have rows of d and out must be contiguous [n, d]")
    _f32vec(weight, "norm weight", d)
    _f32vec(bias, "norm bias", d)
    if rows is not None:
        _i32(rows, "rows", n)
    elif x_rows < n:
        raise KernelError("layernorm: fewer input rows than output rows")
    if n_parts == 1:
        _lib.call("liyab_layernorm", out.data_ptr(), dtype_code(out.dtype), ptr, _ptr(weight), _ptr(bias),
                  _ptr(rows), n, d, float(eps), _stream())
        return
    _lib.call("liyab_layernorm_parts", out.data_ptr(), dtype_code(out.dtype), ptr, n_parts, stride, x_rows, _ptr(weight),
              _ptr(bias), _ptr(rows), n, d, float(eps), _stream())


def sum_parts(out: torch.Tensor, planes: torch.Tensor) -> None:
    """out = planes[0] + planes[1] + ..., in the order the norm kernels add them; out float32
    [rows, d] (it may be planes[0])."""
    _dev(out, "out")
    ptr, n_parts, stride, x_rows, d = _planes(planes, "sum_parts")
    if out.dtype != torch.float32 or tuple(out.shape) != (x_rows, d) or not out.is_contiguous():
        raise KernelError(f"sum_parts: out must be contiguous float32 [{x_rows}, {d}]")
    _lib.call("liyab_sum_parts", out.data_ptr(), x_rows, d, ptr, n_parts, stride, _stream())


def gemm_simple(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out: Optional[torch.Tensor] = None,
                residual: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE) -> None:
    """out = epilogue(a . w^T + bias), or residual += a . w^T + bias.
    a [M, K] and w [N, K] share a dtype; rows of a and out may be strided."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous() or w.dtype != a.dtype:
        raise KernelError(f"gemm: w {tuple(w.shape)} {w.dtype} does not fit a {tuple(a.shape)} {a.dtype}")
    N = w.shape[0]
    _f32vec(bias, "bias", N)
    ldo = ldr = 0
    out_code = F32
    if epilogue == EPI_RESIDUAL:
        if residual is None or residual.dtype != torch.float32 or tuple(residual.shape) != (M, N):
            raise KernelError("gemm: the residual epilogue needs a float32 residual [M, N]")
        ldr = _rows(residual, "residual")
    else:
        if out is None or tuple(out.shape) != (M, N):
            raise KernelError("gemm: out must be [M, N]")
        ldo = _rows(out, "out")
        out_code = dtype_code(out.dtype)
    _lib.call("liyab_gemm_simple", _ptr(out), out_code, ldo, a.data_ptr(), lda, w.data_ptr(), dtype_code(a.dtype),
              _ptr(bias), _ptr(residual), ldr, M, N, K, epilogue, _stream())


def kv_write(k_cache: torch.Tensor, v_cache: torch.Tensor, src: torch.Tensor, k_off: int, v_off: int,
             slots: torch.Tensor, num_pages: Optional[int] = None) -> None:
    """Writes token t's keys src[t, k_off:k_off+Hkv*hd] and values to slot slots[t] of caches
    laid out [pages, kv_heads, page_size, head_dim]. Slots are page * page_size + offset; a
    slot outside the caches' `num_pages` (all of them by default) pages is not written."""
    _dev(k_cache, "k_cache")
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("kv_write: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    if src.dtype != k_cache.dtype or v_cache.dtype != k_cache.dtype:
        raise KernelError("kv_write: source and caches must share a dtype")
    stride = _rows(src, "src")
    n = src.shape[0]
    _i32(slots, "slots", n)
    _, hkv, page, hd = k_cache.shape
    if k_off + hkv * hd > src.shape[1] or v_off + hkv * hd > src.shape[1]:
        raise KernelError("kv_write: column offsets pass the source's width")
    _lib.call("liyab_kv_write", k_cache.data_ptr(), v_cache.data_ptr(), src.data_ptr(), dtype_code(src.dtype), stride,
              k_off, v_off, slots.data_ptr(), n, hkv, hd, page, _pages(k_cache, num_pages), _stream())


def attention_generic(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, *, n_head: int,
                      scale: float, window: int = 0, num_pages: Optional[int] = None) -> None:
    """out[t, h*hd:(h+1)*hd] = softmax(scale * q_th . K[:pos_t+1]) V for the request tok_seq[t].
    q is [n, >= n_head*hd] (a view into a wider projection output is fine)."""
    n = out.shape[0]
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    _, hkv, page, hd = k_cache.shape
    os_ = _rows(out, "out")
    qs = _rows(q, "q")
    if q.shape[0] != n or q.shape[1] < n_head * hd or out.shape[1] != n_head * hd:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {n_head} heads of {hd}")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention: q, out and the caches must share a dtype")
    _dev(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("attention: block_tables must be contiguous int32 [requests, max_blocks]")
    _i32(tok_seq, "tok_seq", n)
    _i32(tok_pos, "tok_pos", n)
    _lib.call("liyab_attention_generic", out.data_ptr(), os_, q.data_ptr(), qs, k_cache.data_ptr(), v_cache.data_ptr(),
              dtype_code(q.dtype), block_tables.data_ptr(), block_tables.shape[1], tok_seq.data_ptr(),
              tok_pos.data_ptr(), n, float(scale), int(window), n_head, hkv, hd, page, _pages(k_cache, num_pages), _stream())


_argmax_scratch = {}


def _scatter(scatter, rows):
    if scatter is None:
        return None, None
    index, target = scatter
    _i32(index, "scatter index", rows)
    _i32(target, "scatter target")
    return index.data_ptr(), target.data_ptr()


def argmax(out: torch.Tensor, logits: torch.Tensor, scatter=None) -> None:
    """out[r] = the first maximal element of logits[r] (ties go to the lowest id). With
    scatter = (index, target), target[index[r]] = out[r] too; the caller has checked the
    indices against the target. `out` may be pinned host memory: the kernel then writes the
    tokens where the host reads them, and no copy follows."""
    ld = _rows(logits, "logits")
    rows, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("argmax: logits must be float32")
    _i32(out, "out", rows, pinned_ok=True)
    key = logits.device
    sc = _argmax_scratch.get(key)
    if sc is None or sc[0].numel() < rows * 64:
        cap = max(rows, 64) * 64
        sc = (torch.empty(cap, dtype=torch.float32, device=key), torch.empty(cap, dtype=torch.int32, device=key))
        _argmax_scratch[key] = sc
    si, so = _scatter(scatter, rows)
    _lib.call("liyab_argmax", out.data_ptr(), logits.data_ptr(), ld, rows, V, sc[0].data_ptr(), sc[1].data_ptr(), si, so,
              _stream())


def sample(out: torch.Tensor, logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, uniform: torch.Tensor, scatter=None) -> None:
    """Per-row sampling; temperature/top_p float32 [rows], top_k int32 [rows], uniform float64 [rows] in [0, 1).
    top_k and top_p may both be None when no row cuts its candidates: a shorter kernel runs then.
    `out` may be pinned host memory, as for `argmax`."""
    ld = _rows(logits, "logits")
    rows, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    _i32(out, "out", rows, pinned_ok=True)
    _f32vec(temperature, "temperature", rows)
    if (top_k is None) != (top_p is None):
        raise KernelError("sample: top_k and top_p are given together or not at all")
    if top_k is not None:
        _f32vec(top_p, "top_p", rows)
        _i32(top_k, "top_k", rows)
    _dev(uniform, "uniform")
    if uniform.dtype != torch.float64 or uniform.numel() != rows or not uniform.is_contiguous():
        raise KernelError("sample: uniform must be contiguous float64 [rows]")
    si, so = _scatter(scatter, rows)
    _lib.call("liyab_sample", out.data_ptr(), logits.data_ptr(), ld, rows, V, temperature.data_ptr(),
              0 if top_k is None else top_k.data_ptr(), 0 if top_p is None else top_p.data_ptr(),
              uniform.data_ptr(), si, so, _stream())


EPI_QKV_PAGED = 4


class _Rows:
    """What `_epilogue` reads of a first operand that is no tensor: its rows and its dtype."""

    def __init__(self, rows: int, dtype: torch.dtype):
        self.shape, self.dtype = (rows, 0), dtype


def _epilogue(a, w, bias, out, residual, epilogue, kv):
    """Checks the epilogue's operands against [M, N] and fills the launchers' struct."""
    M, N = a.shape[0], w.shape[0]
    _f32vec(bias, "bias", N)
    e = _lib.EpiParams()
    e.mode = epilogue
    e.bias = _ptr(bias)
    e.exact = 1 if a.dtype == torch.float32 else 0
    e.out_dtype = F32
    if epilogue == EPI_RESIDUAL:
        if residual is None or residual.dtype != torch.float32 or tuple(residual.shape) != (M, N):
            raise KernelError("gemm: the residual epilogue needs a float32 residual [M, N]")
        e.residual, e.ldr = residual.data_ptr(), _rows(residual, "residual")
    elif epilogue == EPI_QKV_PAGED:
        k_cache, v_cache, slots, q_dim = kv[:4]
        e.num_slots = _pages(k_cache, kv[4] if len(kv) > 4 else None) * k_cache.shape[2]
        if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
            raise KernelError("gemm: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
        _, hkv, page, hd = k_cache.shape
        if out is None or tuple(out.shape) != (M, q_dim) or q_dim + 2 * hkv * hd != N:
            raise KernelError(f"gemm: the paged QKV epilogue needs out [M, {q_dim}] and N = q_dim + 2 * kv_dim")
        if not (out.dtype == k_cache.dtype == v_cache.dtype):
            raise KernelError("gemm: queries and caches must share a dtype")
        _i32(slots, "slots", M)
        e.out, e.ldo, e.out_dtype = out.data_ptr(), _rows(out, "out"), dtype_code(out.dtype)
        e.kc, e.vc, e.slots = k_cache.data_ptr(), v_cache.data_ptr(), slots.data_ptr()
        e.q_dim, e.kv_dim, e.hd, e.n_kv_head, e.page_size = q_dim, hkv * hd, hd, hkv, page
    else:
        if out is None or tuple(out.shape) != (M, N):
            raise KernelError("gemm: out must be [M, N]")
        e.out, e.ldo, e.out_dtype = out.data_ptr(), _rows(out, "out"), dtype_code(out.dtype)
    return e


def gemm_mfma(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, residual=None,
              epilogue: int = EPI_NONE, kv=None, tile: int = 0) -> None:
    """The matrix-core product for bfloat16 operands with K a multiple of 8."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_mfma: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    e = _epilogue(a, w, bias, out, residual, epilogue, kv)
    _lib.call("liyab_gemm_mfma", a.data_ptr(), lda, w.data_ptr(), M, w.shape[0], K, tile, ctypes.byref(e), _stream())


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, residual=None,
                epilogue: int = EPI_NONE, kv=None, ksplit: int = 0, wide: int = -1, mtile: int = 0) -> None:
    """The weight-streaming product for at most 64 bfloat16 rows, K a multiple of 8. ksplit
    (waves sharing K), wide (64 output features a workgroup) and mtile (tiles of 16 rows a
    workgroup) are chosen from the shape unless given."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    if M > 64:
        raise KernelError(f"gemm_skinny: {M} rows; it takes at most 64")
    e = _epilogue(a, w, bias, out, residual, epilogue, kv)
    _lib.call("liyab_gemm_skinny", a.data_ptr(), lda, w.data_ptr(), M, w.shape[0], K, ksplit, wide, mtile, ctypes.byref(e), _stream())


def gemm_skinny_parts(a: torch.Tensor, w: torch.Tensor, planes: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                      base: Optional[torch.Tensor] = None, ksplit: int = 0) -> None:
    """planes[p] = a . w^T summed over the p-th of planes.shape[0] parts of K: the
    weight-streaming product cut over K, for few output features and a long K. a [M <= 64, K]
    and w [N, K] bfloat16, planes float32 [parts, M, N]. With `base` (float32 [M, N] or a sum
    of planes [*, M, N], not overlapping `planes`) the first plane also takes `bias` and the
    rows of `base`, so that the planes add up to base + a . w^T + bias."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    _dev(planes, "planes")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny_parts: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    N = w.shape[0]
    if planes.dtype != torch.float32 or planes.dim() != 3 or tuple(planes.shape[1:]) != (M, N) or not planes.is_contiguous():
        raise KernelError(f"gemm_skinny_parts: planes must be contiguous float32 [parts, {M}, {N}], got {tuple(planes.shape)}")
    bptr, n_base, bstride = None, 0, 0
    if base is not None:
        bptr, n_base, bstride, b_rows, b_d = _planes(base, "gemm_skinny_parts: base")
        if (b_rows, b_d) != (M, N):
            raise KernelError(f"gemm_skinny_parts: base must have rows [{M}, {N}], got {tuple(base.shape)}")
        _f32vec(bias, "bias", N)
    elif bias is not None:
        raise KernelError("gemm_skinny_parts: a bias needs the rows it is added to (base)")
    _lib.call("liyab_gemm_skinny_parts", a.data_ptr(), lda, w.data_ptr(), M, N, K, planes.shape[0], ksplit,
              planes.data_ptr(), planes.stride(0), _ptr(bias), bptr, n_base, bstride, _stream())


def gemm_mfma_dl_parts(a: torch.Tensor, w: torch.Tensor, planes: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                       base: Optional[torch.Tensor] = None, tile: int = 6) -> None:
    """The tiled matrix-core product cut over K (K a multiple of 64), as `gemm_skinny_parts` for
    any number of rows: planes float32 [parts, M, N]; with `base` the first plane also takes
    `bias` and the rows of `base`. tile: 6 = 64 x 64 tiles, 16 = 64 x 32, 17 = 32 x 32."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    _dev(planes, "planes")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_mfma_dl_parts: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    N = w.shape[0]
    if planes.dtype != torch.float32 or planes.dim() != 3 or tuple(planes.shape[1:]) != (M, N) or not planes.is_contiguous():
        raise KernelError(f"gemm_mfma_dl_parts: planes must be contiguous float32 [parts, {M}, {N}], got {tuple(planes.shape)}")
    bptr, n_base, bstride = None, 0, 0
    if base is not None:
        bptr, n_base, bstride, b_rows, b_d = _planes(base, "gemm_mfma_dl_parts: base")
        if (b_rows, b_d) != (M, N):
            raise KernelError(f"gemm_mfma_dl_parts: base must have rows [{M}, {N}], got {tuple(base.shape)}")
        _f32vec(bias, "bias", N)
    elif bias is not None:
        raise KernelError("gemm_mfma_dl_parts: a bias needs the rows it is added to (base)")
    _lib.call("liyab_gemm_mfma_dl_parts", a.data_ptr(), lda, w.data_ptr(), M, N, K, planes.shape[0], tile,
              planes.data_ptr(), planes.stride(0), _ptr(bias), bptr, n_base, bstride, _stream())


def gemm_att_parts(partials: torch.Tensor, w: torch.Tensor, planes: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                   base: Optional[torch.Tensor] = None) -> None:
    """The product cut over K (as `gemm_skinny_parts`) whose first operand is attention's output
    still in splits: partials float32 [M <= 32, heads, splits <= 8, head size + 4] as
    `attention_decode(..., leave_splits=True)` leaves them, merged as they are loaded.
    w [N, heads * head size] bfloat16, planes float32 [parts, M, N]."""
    _dev(partials, "partials")
    _dev(w, "w")
    _dev(planes, "planes")
    if partials.dtype != torch.float32 or partials.dim() != 4 or not partials.is_contiguous():
        raise KernelError(f"gemm_att_parts: partials must be contiguous float32 [M, heads, splits, head size + 4], got {tuple(partials.shape)}")
    M, H, S, hd4 = partials.shape
    K = H * (hd4 - 4)
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_att_parts: needs contiguous bfloat16 w [N, {K}], got {tuple(w.shape)} {w.dtype}")
    N = w.shape[0]
    if not att_parts_takes(M, S, hd4 - 4):
        raise KernelError(f"gemm_att_parts: {M} rows in {S} splits of heads of {hd4 - 4} are outside what it takes")
    if planes.dtype != torch.float32 or planes.dim() != 3 or tuple(planes.shape[1:]) != (M, N) or not planes.is_contiguous():
        raise KernelError(f"gemm_att_parts: planes must be contiguous float32 [parts, {M}, {N}], got {tuple(planes.shape)}")
    bptr, n_base, bstride = None, 0, 0
    if base is not None:
        bptr, n_base, bstride, b_rows, b_d = _planes(base, "gemm_att_parts: base")
        if (b_rows, b_d) != (M, N):
            raise KernelError(f"gemm_att_parts: base must have rows [{M}, {N}], got {tuple(base.shape)}")
        _f32vec(bias, "bias", N)
    elif bias is not None:
        raise KernelError("gemm_att_parts: a bias needs the rows it is added to (base)")
    _lib.call("liyab_gemm_att_parts", partials.data_ptr(), S, H, hd4 - 4, w.data_ptr(), M, N, planes.shape[0],
              planes.data_ptr(), planes.stride(0), _ptr(bias), bptr, n_base, bstride, _stream())


def att_parts_takes(M: int, splits: int, hd: int) -> bool:
    return 0 < M <= 32 and 1 <= splits <= 8 and hd % 8 == 0 and 8 <= hd <= 256


def k_parts(M: int, N: int, K: int) -> int:
    """Into how many parts of K the weight-streaming product is best cut (1: not at all). With
    few output features a product fills a fraction of the chip's compute units, and a long K
    then streams through those few; cut over K it covers the chip. Measured at 8 rows, whole
    and in parts (us): 3,072 -> 768 7.2 and 4.5 (four parts), 768 -> 768 4.6 and 3.4 (four),
    6,400 -> 1,600 13.4 and 8.5 (two), 1,600 -> 1,600 5.4 and 4.6 (two)."""
    if M > 32 or K % 8 != 0 or _invariant:
        return 1
    groups, units = (N + 15) // 16 * ((M + 15) // 16), (K + 63) // 64  # workgroups uncut; units of 64 k
    parts = 1
    while parts < 4 and groups * parts * 2 <= 256 and units // (parts * 2) >= 3:
        parts *= 2
    return parts


def skinny_parts_takes(M: int, N: int, K: int) -> bool:
    """Whether `gemm_skinny_parts` takes this shape and is the kernel `gemm` would choose for it."""
    return 0 < M <= 64 and K % 8 == 0 and N <= 8192 and not (M > 32 and K % 64 == 0 and N >= 2048)


def tiled_k_parts(M: int, N: int, K: int) -> int:
    """Into how many parts of K the tiled product of more than 32 rows (of more than 16, with many
    output features) is best cut when it is added to the residual stream (1: not at all).
    Several tiles of rows, few output features and a long K (a prompt's portion through the feed-forward's second product: 128 x 768 x 3,072 is
    24 tiles of 64 x 64, each walking the whole of K in 18.7 us): cut until the tiles cover the
    chip. One tile of rows (33 to 64): the 64 x 32 tiles are few and each walks the whole of K;
    cut over K they cover the chip: alone, at 64 rows, 3,072 -> 768 takes 8.2 us whole (the streaming kernel) and 4.9 in 8 parts, 6,400 ->
    1,600 19.8 and 8.2. In a decode step the next readers pay for the planes, though: inner
    dimensions from 3,072 gain, in 4 parts (ms a step at 64 rows, whole and cut: GPT-2 small's
    sizes 0.806 and 0.797, medium's 1.767 and 1.715; XL's 5.19 and 4.90)."""
    if K % 64 != 0 or M <= 16 or _invariant:
        return 1
    if M <= 64:
        if N <= 2048:
            return 4 if K >= 3072 and M > 32 else 1
        # more output features: the largest tiles that take the rows in one, 32 x 32 up to 32 rows and
        # 64 x 64 beyond (every tile reads all the rows: at 64 rows, 32 x 32 tiles read them twice as
        # often as the weights), cut while tiles x parts stay within the chip (us alone, whole as it
        # was and cut: 64 rows, 16,384 -> 4,096 42.2 and 32.3 in 4 parts, 4,096 -> 4,096 13.5 and 9.7,
        # 8,192 -> 8,192 34.8 and 31.6 in 2 parts; 32 rows, 16,384 -> 4,096 39.7 and 27.8 in 2 parts,
        # 4,096 -> 4,096 12.3 and 9.6, 8,192 -> 8,192 27.3 whole)
        side = 32 if M <= 32 else 64
        tiles, parts = (N + side - 1) // side, 1
        while parts < 4 and tiles * parts * 2 <= 256 and K // 64 // (parts * 2) >= 8:  # (256: the compute units of the part this was measured on)
            parts *= 2
        return parts
    # several tiles of rows (a prompt's portion): 64 x 64 tiles, cut until they cover the chip,
    # a part keeping 256 of K or more; in two parts while two workgroups a compute unit hold them
    # (ms a step of 768 / 1,024 tokens whole and in two parts: GPT-2 small's sizes 1.00 and 0.99 /
    # 1.13 and 1.12, medium's 2.32 and 2.16 / 2.54 and 2.47; XL's at 512 tokens 6.11 and 5.88)
    tiles = (M + 63) // 64 * ((N + 63) // 64)
    nk = K // 64
    parts = 1
    while parts < TILED_MAX_PARTS and tiles * parts * 2 <= (512 if parts == 1 else 256) and nk // (parts * 2) >= 4:
        parts *= 2
    return parts


TILED_MAX_PARTS = 4  # (us a step of 128 / 256 / 512 tokens of one prompt with at most 1, 2, 4, 8 parts: 765 665 637 668 / 809 720 694 679 / 922 843 842 846)


def gemm_skinny_ln(x: torch.Tensor, ln_weight: Optional[torch.Tensor], ln_bias: Optional[torch.Tensor], eps: float,
                   w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, epilogue: int = EPI_NONE, kv=None,
                   wide: int = -1) -> None:
    """The weight-streaming product over LayerNorm(x) of the float32 rows x [M, K], or of a sum
    of planes [parts, M, K], the norm computed inside the product kernel (`skinny_ln_takes`).
    wide: 32 instead of 16 output features a workgroup (-1: chosen from the shape)."""
    ptr, n_parts, stride, M, K = _planes(x, "gemm_skinny_ln")
    _dev(w, "w")
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny_ln: needs contiguous bfloat16 w [N, {K}], got {tuple(w.shape)} {w.dtype}")
    if not skinny_ln_takes(M, K):
        raise KernelError(f"gemm_skinny_ln: {M} rows of {K} are outside what it takes")
    if epilogue == EPI_RESIDUAL:
        raise KernelError("gemm_skinny_ln: the residual epilogue is not taken")
    _f32vec(ln_weight, "norm weight", K)
    _f32vec(ln_bias, "norm bias", K)
    e = _epilogue(_Rows(M, torch.bfloat16), w, bias, out, None, epilogue, kv)
    e.exact = 0
    _lib.call("liyab_gemm_skinny_ln", ptr, n_parts, stride, _ptr(ln_weight), _ptr(ln_bias), float(eps),
              w.data_ptr(), M, w.shape[0], K, wide, ctypes.byref(e), _stream())


def gemm_skinny_dyt(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], alpha: torch.Tensor, w: torch.Tensor,
                    out_bias: Optional[torch.Tensor], *, out=None, epilogue: int = EPI_NONE, kv=None, wide: int = -1) -> None:
    """`gemm_skinny_ln` with the Dynamic Tanh norm in the norm's place: the product over tanh(alpha x) * weight + bias of the
    float32 rows x [M, K] (alpha: one float32 value on the device)."""
    ptr, n_parts, stride, M, K = _planes(x, "gemm_skinny_dyt")
    _dev(w, "w")
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny_dyt: needs contiguous bfloat16 w [N, {K}], got {tuple(w.shape)} {w.dtype}")
    if not skinny_ln_takes(M, K) or epilogue == EPI_RESIDUAL:
        raise KernelError(f"gemm_skinny_dyt: {M} rows of {K}, or the residual epilogue, are outside what it takes")
    _f32vec(weight, "norm weight", K)
    _f32vec(bias, "norm bias", K)
    _f32vec(alpha, "norm alpha", 1)
    e = _epilogue(_Rows(M, torch.bfloat16), w, out_bias, out, None, epilogue, kv)
    e.exact = 0
    _lib.call("liyab_gemm_skinny_dyt", ptr, n_parts, stride, _ptr(weight), _ptr(bias), alpha.data_ptr(), w.data_ptr(), M, w.shape[0], K, wide,
              ctypes.byref(e), _stream())


def skinny_ln_takes(M: int, K: int) -> bool:
    """What the product kernel with the norm inside takes: one or two tiles of 16 rows, a row in
    a wave's registers."""
    return 0 < M <= 32 and K % 8 == 0 and K <= 2048


_compute_units = 0


def compute_units() -> int:
    global _compute_units
    if not _compute_units:
        _compute_units = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return _compute_units


def skinny_ln_pays(M: int, N: int, K: int) -> bool:
    """Whether folding the norm into the product beats the norm kernel followed by the plain
    product. The folded kernel keeps a row in registers, so one workgroup fills a compute unit:
    with more workgroups (16 or 32 output features each) than compute units they run in two
    rounds, which costs more than the norm's kernel (GPT-2 XL's 1,600 -> 4,800 at 8 rows in
    strips of 16: 15.2 us folded against 9 + 4.5)."""
    return not _invariant and skinny_ln_takes(M, K) and (N + (31 if M <= 16 else 15)) // (32 if M <= 16 else 16) <= compute_units()


def gemm_mfma_dl(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, residual=None,
                 epilogue: int = EPI_NONE, kv=None, tile: int = 0) -> None:
    """The matrix-core product with tiles loaded straight into LDS, three stages deep; bfloat16
    operands, K a multiple of 64."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_mfma_dl: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    if K % 64 != 0 or M == 0:
        raise KernelError(f"gemm_mfma_dl: K = {K} must be a multiple of 64 and M positive")
    e = _epilogue(a, w, bias, out, residual, epilogue, kv)
    _lib.call("liyab_gemm_mfma_dl", a.data_ptr(), lda, w.data_ptr(), M, w.shape[0], K, tile, ctypes.byref(e), _stream())


def mfma_takes(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out: Optional[torch.Tensor] = None,
         residual: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE, kv=None) -> None:
    """The product kernel for these operands: matrix cores for bfloat16 shapes they take,
    the plain tiled kernel for float32 and everything else. `kv` = (k_cache, v_cache, slots,
    q_dim[, num_pages]) with the paged QKV epilogue (a slot outside the caches' pages is not written)."""
    if _invariant and mfma_takes(a, w):
        # one family of kernels whatever the number of rows: their sum over k has one order for
        # every tile shape, so a row's bits do not depend on the rows beside it. K a multiple of 64:
        # four sums, unit u of 64 k going to sum u % 4 (16 k an instruction), added in their order;
        # up to 64 rows four groups of waves walk K side by side, a sum each, in small tiles that
        # cover the chip; more rows take the large tiles, whose one group keeps the four sums.
        M, N, K = a.shape[0], w.shape[0], a.shape[1]
        if K % 64 == 0:
            if M <= 64:
                tile = 17 if M <= 32 or 2 * ((N + 31) // 32) <= compute_units() else 16
            else:
                tile = 108 if M * N >= 2048 * 2048 else (106 if K >= 2048 else 102)
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=tile)
        else:
            gemm_mfma(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=2)
        return
    if mfma_takes(a, w):
        M, N = a.shape[0], w.shape[0]
        if 12 < M <= 128 and N >= 16384 and a.shape[1] % 64 == 0 and (N + 127) // 128 >= compute_units():
            # a vocabulary's worth of output features: large tiles re-read the tokens least
            # (16 rows: 22.5 against 25.1 us for 768 -> 50,257; 64 rows: 27.9 against 32.9); with fewer such tiles
            # than compute units they stream too slowly (4,096 -> 16,384 at 64 rows: 128 tiles, 65 us)
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=8)
        elif ((M > 32 or (M > 16 and N * a.shape[1] >= 6 << 20)) and a.shape[1] % 64 == 0 and N >= 2048
              and (M + 63) // 64 * ((N + 31) // 32) <= compute_units()):
            # one tile of 33 to 64 rows and many output features: 64 x 32 tiles share the tokens'
            # rows through LDS where the streaming kernel's workgroups each read them again (40
            # rows: 5.2 against 6.4 us for 768 -> 2,304, 8.0 against 10.4 for 1,600 -> 4,800; the
            # products back to the model's width, with fewer tiles, stay with the streaming kernel);
            # the largest matrices already from 17 rows (32 rows, weights cold from HBM: 8.9
            # against 12.5 us for 1,600 -> 4,800, but 6.6 against 6.1 for 1,024 -> 3,072); more
            # tiles of rows as long as every tile has a compute unit of its own (the stages fill
            # a unit's LDS; 128 rows: 6.1 against 7.7 us for 768 -> 2,304 in 64 x 64 tiles; with
            # more tiles than units, 400 rows: 10.7 against 8.0)
            # tiles of 32 x 32 while each has a compute unit of its own: a workgroup brings in a third
            # less of the operands and twice as many pull (64 rows, cold weights: 5.05 against 5.53 us
            # for 768 -> 2,304, 5.97 against 6.85 for 1,024 -> 3,072; 13.9 against 9.7 for 1,600 -> 4,800)
            small = (M + 31) // 32 * ((N + 31) // 32) <= compute_units()
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=17 if small else 16)
        elif M <= 16 or (M <= 64 and N <= 8192):
            # few tokens: stream the weights (for a huge N and more than 16 tokens the tiled
            # kernel's shared loads beat every workgroup re-reading the tokens); 11 to 16 tokens and
            # very many output features in strips of 64, which read the tokens a quarter as often (16
            # rows, alone: 4,096 -> 16,384 31.6 against 36.4 us, -> 12,288 25.3 against 28.5; at 8 rows
            # and at 6,400 features strips of 16 win)
            gemm_skinny(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, wide=1 if 10 < M <= 16 and N >= 12288 else 0)
        elif a.shape[1] % 64 == 0:
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv)
        else:
            gemm_mfma(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv)
        return
    if epilogue == EPI_QKV_PAGED:
        # the plain kernel writes the whole projection; a second kernel moves keys and values
        raise KernelError("gemm: the paged QKV epilogue is for the matrix-core kernels; use gemm + kv_write")
    gemm_simple(a, w, bias, out=out, residual=residual, epilogue=epilogue)


def attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_tables: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, *, n_head: int,
                     scale: float, window: int = 0, n_splits: int = 1, partials: Optional[torch.Tensor] = None,
                     tok_list: Optional[torch.Tensor] = None, n_tokens: Optional[int] = None, waves: int = 4,
                     rows_are_requests: bool = False, leave_splits: bool = False, chunk: int = 0,
                     num_pages: Optional[int] = None, softcap: float = 0.0, bias_table: Optional[torch.Tensor] = None,
                     sinks: Optional[torch.Tensor] = None) -> None:
    """Each token on its own over its request's cache (bfloat16, or float32 throughout), its keys cut into `n_splits`.
    With `tok_list` (int32) only those rows are computed. `rows_are_requests`: row t belongs to
    request t (every request brings one token), which saves the kernel a lookup. With
    `leave_splits` (several splits) `out` is not written: `partials`, viewed as [tokens, heads,
    splits, head size + 4], keeps each split's weighted values, maximum and sum for a reader
    that merges them (`gemm_att_parts`). `chunk` > 0: split z takes keys [z * chunk, (z + 1) * chunk) of a
    token's keys instead of an equal share (`n_splits * chunk` must cover the longest context): a token's
    sums then follow from its position alone. `softcap` > 0: scores become cap * tanh(score / cap); `bias_table` (float32
    [distances, heads]): + table[min(position - key, distances - 1), head]; `sinks` (float32 [heads]): exp(sinks[head]) joins
    the softmax's denominator (a learned logit with no key and no value)."""
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    _, hkv, page, hd = k_cache.shape
    os_, qs = _rows(out, "out"), _rows(q, "q")
    rows = out.shape[0]
    n = rows if n_tokens is None else n_tokens
    if q.shape[0] != rows or q.shape[1] < n_head * hd or out.shape[1] != n_head * hd:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {n_head} heads of {hd}")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype) or q.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("attention_decode: q, out and the caches must all be bfloat16 or all float32")
    _dev(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("attention: block_tables must be contiguous int32 [requests, max_blocks]")
    _i32(tok_seq, "tok_seq", rows)
    _i32(tok_pos, "tok_pos", rows)
    if tok_list is not None:
        _i32(tok_list, "tok_list", n)
    elif n != rows:
        raise KernelError("attention_decode: n_tokens needs tok_list")
    if leave_splits and n_splits <= 1:
        raise KernelError("attention_decode: splits are left only when there are several")
    if n_splits > 1:
        need = n * n_head * n_splits * (hd + 4)
        if partials is None or partials.dtype != torch.float32 or partials.numel() < need or not partials.is_contiguous():
            raise KernelError(f"attention_decode: {n_splits} splits need {need} float32 of partials")
    args = (out.data_ptr(), os_, q.data_ptr(), qs, k_cache.data_ptr(), v_cache.data_ptr(),
            dtype_code(q.dtype), block_tables.data_ptr(), block_tables.shape[1], _ptr(tok_list), tok_seq.data_ptr(), tok_pos.data_ptr(),
            n, float(scale), int(window), n_head, hkv, hd, page, n_splits, int(chunk), waves, 1 if rows_are_requests else 0,
            _ptr(partials), 1 if leave_splits else 0, _pages(k_cache, num_pages))
    _f32vec(sinks, "sinks", n_head)
    if softcap > 0 or bias_table is not None or sinks is not None:
        if sinks is not None and leave_splits:
            raise KernelError("attention_decode: splits left unmerged take no sink")
        _lib.call("liyab_attention_decode_scored", *args, float(softcap), _ptr(bias_table), _bias_rows(bias_table, n_head) - 1, _ptr(sinks), _stream())
    else:
        _lib.call("liyab_attention_decode", *args, _stream())


def _bias_rows(bias_table: Optional[torch.Tensor], n_head: int) -> int:
    """The rows of a bias-by-distance table, float32 [distances, heads] on the device (1 for none)."""
    if bias_table is None:
        return 1
    _dev(bias_table, "bias_table")
    if bias_table.dtype != torch.float32 or bias_table.dim() != 2 or bias_table.shape[1] != n_head or bias_table.shape[0] < 1 or not bias_table.is_contiguous():
        raise KernelError(f"attention: the bias table must be contiguous float32 [distances, {n_head}], got {tuple(bias_table.shape)} {bias_table.dtype}")
    return bias_table.shape[0]


def attention_merge(out: torch.Tensor, partials: torch.Tensor) -> None:
    """out [tokens, heads * head size] (bfloat16 or float32) = the splits that `attention_decode(...,
    leave_splits=True)` left in partials [tokens, heads, splits, head size + 4], merged in split order."""
    _dev(partials, "partials")
    os_ = _rows(out, "out")
    if partials.dtype != torch.float32 or partials.dim() != 4 or not partials.is_contiguous():
        raise KernelError("attention_merge: partials must be contiguous float32 [tokens, heads, splits, head size + 4]")
    n, H, S, hd4 = partials.shape
    if out.dtype not in (torch.bfloat16, torch.float32) or tuple(out.shape) != (n, H * (hd4 - 4)):
        raise KernelError(f"attention_merge: out must be bfloat16 or float32 [{n}, {H * (hd4 - 4)}]")
    _lib.call("liyab_attention_merge", out.data_ptr(), dtype_code(out.dtype), os_, partials.data_ptr(), n, H, hd4 - 4, S, _stream())


def attention_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, work: torch.Tensor, n_tiles: int, *, n_head: int, scale: float,
                      window: int = 0, tile: int = 128, ksplit: int = 1, num_pages: Optional[int] = None, softcap: float = 0.0,
                      bias_table: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None) -> None:
    """Tiles of up to `tile` (64 or 128) consecutive queries of one request over its bfloat16
    cache, on the matrix cores; `ksplit` waves (1, 2, or 4 with tiles of 64) share the keys of
    32 queries. work: int32 [n_tiles, 4] = (request index, first row, first
    position, queries); the caller has checked rows and positions against out and the block tables."""
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    _, hkv, page, hd = k_cache.shape
    os_, qs = _rows(out, "out"), _rows(q, "q")
    if q.shape[0] != out.shape[0] or q.shape[1] < n_head * hd or out.shape[1] != n_head * hd:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {n_head} heads of {hd}")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16):
        raise KernelError("attention_prefill: q, out and the caches must be bfloat16")
    if not prefill_takes(hd):
        raise KernelError(f"attention_prefill: head size {hd} is not a multiple of 16 in 16..128")
    _dev(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("attention: block_tables must be contiguous int32 [requests, max_blocks]")
    _i32(work, "work", 4 * n_tiles)
    args = (out.data_ptr(), os_, q.data_ptr(), qs, k_cache.data_ptr(), v_cache.data_ptr(),
            block_tables.data_ptr(), block_tables.shape[1], work.data_ptr(), n_tiles, int(tile), int(ksplit), float(scale), int(window),
            n_head, hkv, hd, page, _pages(k_cache, num_pages))
    _f32vec(sinks, "sinks", n_head)
    if softcap > 0 or bias_table is not None or sinks is not None:  # (see attention_decode)
        _lib.call("liyab_attention_prefill_scored", *args, float(softcap), _ptr(bias_table), _bias_rows(bias_table, n_head) - 1, _ptr(sinks), _stream())
    else:
        _lib.call("liyab_attention_prefill", *args, _stream())


PREFILL_KSPLIT4_WORK = 256  # tiles x heads up to which four waves share a tile of 64 queries' keys


def prefill_takes(hd: int) -> bool:
    return hd % 16 == 0 and 16 <= hd <= 128


def decode_plan(n_tokens: int, n_head: int, context_bucket: int):
    """(splits of the keys, waves per workgroup) for tokens whose attention the kernel finishes
    itself (several splits: plus the merge kernel). `context_bucket`: the most keys a token has,
    rounded up. From measurements at 12 to 32 heads of 64 and 128, 1 to 8 tokens and 300 to
    4,000 keys (us, attention and merge): with many (token, head) pairs a workgroup of 4 waves
    a pair is fastest, with a few hundred one of 8 (a decode step at batch 24 / 32 / 40 with 4,
    8 and 16 waves: 610 595 654 / 648 633 692 / 706 698 755; 200 pairs at 544 / 2,000 keys: 7.1
    / 19.7 with 8 waves, 8.9 / 20.0 with 16). With fewer pairs than would fill the chip the keys
    are cut across workgroups of 4 waves, into 4, 8 or 16 splits of 128 keys or more, while
    pairs x splits stay within the chip's 256 compute units (32 pairs of 128 dimensions at
    1,000 / 2,000 / 4,000 keys: 7.5 / 10.6 / 18.4 in 8 splits against 11.8 / 19.1 / 33.1 uncut
    on 16 waves; 12 pairs of 64: 6.9 / 7.8 / 9.7 against 8.7 / 11.8 / 18.6). Two splits never
    beat 8 waves uncut. Uncut, 16 waves a pair pay from 4,000 keys on only."""
    pairs = max(1, n_tokens * n_head)
    if pairs >= 512 or context_bucket <= 256:
        return 1, 4
    splits = 1
    while splits < 16 and pairs * splits * 2 <= 256 and context_bucket // (splits * 2) >= 128:
        splits *= 2
    if splits >= 4:
        # (splits of 1,024 keys and more on 8 waves: 12 pairs at 30,000 keys in 16 splits 26.7 us on
        # 4 waves, 22.4 on 8; 32 pairs of 128 dimensions 92.6 and 89.1)
        return splits, (8 if context_bucket // splits >= 1024 else 4)
    return 1, (16 if context_bucket >= 4096 and pairs < 256 else 8)


def decode_split_plan(n_tokens: int, n_head: int, context_bucket: int):
    """(splits, waves per workgroup) for a step whose attention output is read by somebody who
    merges a (token, head) pair's splits himself (1 split: not cut). Measured at 12 heads of 64
    and contexts of 512 to 1,024 (us a decode step at batch 1 / 8 / 16, uncut: 376 / 430 / 499):
    8 splits of 4 waves 347 / 418 / 505, 4 of 4 360 / 425 / 496, 4 of 8 353 / 426 / 503, 2 of
    16 390 / 444 / 588. So: workgroups of 4 waves, 8 splits (4 from a hundred pairs on), a
    split keeping 128 keys or more of the longest context."""
    pairs = max(1, n_tokens * n_head)
    most = 8 if pairs <= 96 else (4 if pairs <= SPLIT4_PAIRS else (2 if pairs <= SPLIT2_PAIRS else 1))
    splits = 1
    while splits < most and context_bucket // (2 * splits) >= 128:
        splits *= 2
    # very long contexts of one or two requests: 8 splits of 4 waves leave most of the chip idle and
    # each walks thousands of keys; 16 waves a split walk them four times as fast (us, 12 pairs of 64
    # at 8,000 / 16,000 / 30,000 keys: 14.5 / 25.1 / 41.2 on 4 waves, 11.7 / 17.0 / 23.6 on 16; from
    # 48 pairs on 4 waves win)
    return splits, (16 if pairs <= 32 and context_bucket // splits >= 1024 else 4)


# pairs up to which 4 and 2 splits are taken (beyond 16 tokens splits lost: us a step at batch 17 / 24 / 32
# uncut 529 / 594 / 633, in 4 splits 568 / 630 / 708, in 2 splits 573 / 635 / 704)
SPLIT4_PAIRS, SPLIT2_PAIRS = 192, 192


ATTENTION_MAX_HEAD_DIM = 256  # what the attention kernels take (attention_generic.hip, attention_decode.hip)


INVARIANT_CHUNK = 256  # keys a split where splits go by position alone
INVARIANT_SPLIT_WORK = 1024  # (token, head, split) workgroups up to which such splits are launched side by side
INVARIANT_MAX_SPLITS = 16  # what one workgroup walks in turn (attention_decode.hip: AD_LOOP_CHUNKS)


def invariant_chunk(reach: int) -> int:
    """Keys a split where splits go by position alone, for requests that reach at most `reach` keys:
    INVARIANT_CHUNK, doubled until INVARIANT_MAX_SPLITS splits cover the reach."""
    chunk = INVARIANT_CHUNK
    while chunk * INVARIANT_MAX_SPLITS < reach:
        chunk *= 2
    return chunk


def attention_takes(head_dim: int) -> bool:
    """Whether some attention kernel of the library takes this head size, in either precision."""
    return 0 < head_dim <= ATTENTION_MAX_HEAD_DIM


def attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              block_tables: torch.Tensor, ctx, *, n_head: int, scale: float, window: int = 0,
              splits_ok: bool = False, softcap: float = 0.0, bias_table: Optional[torch.Tensor] = None,
              sinks: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """Attention of the step's tokens over their requests' cached keys and values; the kernel
    is chosen from the step's shape (`ctx` is the step's StepContext; `ctx.plans["attention"]`
    says how the step's tokens are cut, see parts/attention.py; without it every token goes to
    the plain kernel). With `splits_ok`, a step of few tokens may leave `out` unwritten and
    return the splits of each (token, head) pair instead, float32 [tokens, heads, splits, head
    size + 4], for `gemm_att_parts`. `softcap`, `bias_table`: what is done to the scores before the softmax, `sinks`: a learned
    logit a head in its denominator (see `attention_decode`); every kernel below does the same."""
    hd = k_cache.shape[3]
    host = ctx.host
    scored = dict(softcap=softcap, bias_table=bias_table, sinks=sinks) if softcap > 0 or bias_table is not None or sinks is not None else {}
    if sinks is not None and splits_ok:
        raise KernelError("attention: splits left to the caller take no sink")
    plan = ctx.plans.get("attention")
    fast = (plan is not None and q.dtype == torch.bfloat16 and hd % 8 == 0 and q.stride(0) % 8 == 0
            and out.stride(0) % 8 == 0)

    def decode(tok_list, n):
        splits, waves = decode_plan(n, n_head, min(plan.context_bucket, window) if window > 0 else plan.context_bucket)
        partials = None
        if splits > 1:
            partials = ctx.workspace.get("attn_partials", (n * n_head * splits * (hd + 4),), torch.float32)
        attention_decode(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head,
                         scale=scale, window=window, n_splits=splits, partials=partials, waves=waves,
                         tok_list=tok_list, n_tokens=n if tok_list is not None else None,
                         rows_are_requests=tok_list is None and host.max_q_len == 1, **scored)

    if (plan is not None and block_tables.shape[1] <= 2048
            and (fast and _invariant or q.dtype == torch.float32 and hd % 8 == 0 and q.stride(0) % 4 == 0 and out.stride(0) % 4 == 0)):
        # the 32-bit path and the batch-invariant mode: every token on its own on four waves, its keys
        # in splits of INVARIANT_CHUNK from its first key on, merged in their order: the order of a
        # token's sums follows from its position alone, so its bits do not depend on the batch
        n = out.shape[0]
        # a split's keys follow from what a request can reach at most (the table's width, the window): a
        # constant of the engine, never of the step; at most 16 splits, so that one workgroup can walk them
        # all and the merge's arrays hold them (contexts past 4,096 keys take longer splits)
        reach = block_tables.shape[1] * k_cache.shape[2] if window <= 0 else min(window, block_tables.shape[1] * k_cache.shape[2])
        chunk = invariant_chunk(reach)
        splits = max(1, -(-min(plan.context_bucket, reach) // chunk))
        # many tokens: a workgroup walks its token's splits in turn (the same bits: the kernel merges them
        # as the merge kernel does), which saves the splits' traffic and leaves the chip as full
        if n * n_head * splits > INVARIANT_SPLIT_WORK:
            splits = 1
        partials = ctx.workspace.get("attn_partials", (n * n_head * splits * (hd + 4),), torch.float32) if splits > 1 else None
        attention_decode(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head, scale=scale,
                         window=window, n_splits=splits, partials=partials, waves=4, chunk=chunk,
                         rows_are_requests=host.max_q_len == 1, **scored)
        return None
    if fast and plan.mode == "decode" and block_tables.shape[1] <= 2048:
        n = out.shape[0]
        splits, waves = decode_split_plan(n, n_head, plan.context_bucket) if splits_ok else (1, 4)
        if splits > 1 and att_parts_takes(n, splits, hd):
            partials = ctx.workspace.get("attn_partials", (n, n_head, splits, hd + 4), torch.float32)
            attention_decode(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head,
                             scale=scale, window=window, n_splits=splits, partials=partials, waves=waves,
                             rows_are_requests=host.max_q_len == 1, leave_splits=True, **scored)
            return partials
        decode(None, n)
        return None
    if fast and plan.mode == "prefill" and prefill_takes(hd) and scale > 0 and block_tables.shape[1] <= 2048:
        # long portions in tiles on the matrix cores, the short ones token by token
        if plan.n_tiles:
            # with fewer workgroups than compute units, two waves share each query group's keys:
            # the longest tile's walk over its keys is then the kernel's critical path, and halves
            work = plan.n_tiles * n_head
            # (heads past 96: two waves a query group at every size, 185 against 217 us for 16 x 1,024 tokens of 12 heads of 128)
            ksplit = (4 if plan.tile == 64 and hd <= 64 and work <= PREFILL_KSPLIT4_WORK else 2) if work <= 256 or hd > 96 else 1
            attention_prefill(out, q, k_cache, v_cache, block_tables, plan.work, plan.n_tiles, n_head=n_head,
                              scale=scale, window=window, tile=plan.tile, ksplit=ksplit, **scored)
        if plan.n_single:
            decode(plan.single_rows, plan.n_single)
        return
    if scored:
        attention_scored(out, q, k_cache, v_cache, block_tables, ctx, n_head=n_head, scale=scale, window=window, **scored)
        return None
    attention_generic(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head, scale=scale,
                      window=window)


# -- root-mean-square norms, the gated residual update, the input convolution --------------------
def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = x[rows[r]] (or x[r]) / sqrt(mean(.^2) + eps) * weight; x float32 [*, d], out [n, d]
    float32 or bfloat16."""
    _dev(out, "out")
    _dev(x, "x")
    n, d = out.shape
    if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != d or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"rmsnorm: x must be contiguous float32 [*, {d}] and out contiguous, got {tuple(x.shape)} {x.dtype}")
    _f32vec(weight, "norm weight", d)
    if rows is not None:
        _i32(rows, "rows", n)
    elif x.shape[0] < n:
        raise KernelError("rmsnorm: fewer input rows than output rows")
    _lib.call("liyab_rmsnorm", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), _ptr(weight), _ptr(rows), n, d, float(eps), _stream())


def _keep_args(keep, d: int):
    """The arguments that say which rows of a step are kept as a convolution's input history: keep =
    (state float32 [slots, ring, d], ctx) or None."""
    if keep is None:
        return (None, 0, 0, None, None, None, None, None)
    state, ctx = keep
    _dev(state, "state")
    if state.dtype != torch.float32 or state.dim() != 3 or state.shape[2] != d or state.shape[1] < 1 or not state.is_contiguous():
        raise KernelError(f"kept rows: the state must be contiguous float32 [slots, ring, {d}], got {tuple(state.shape)} {state.dtype}")
    n = ctx.n_tokens
    _i32(ctx.tok_seq, "tok_seq", n)
    _i32(ctx.positions, "positions", n)
    _i32(ctx.context_lens, "context_lens", ctx.n_seqs)
    _i32(ctx.state_slots, "state_slots", ctx.n_seqs)
    _i32(ctx.seq_starts, "seq_starts", ctx.n_seqs + 1)
    return (state.data_ptr(), state.shape[1], state.shape[0], ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(),
            ctx.context_lens.data_ptr(), ctx.state_slots.data_ptr(), ctx.seq_starts.data_ptr() + 4 * ctx.n_seqs)


def gated_norm_add(x: torch.Tensor, y: torch.Tensor, weight: Optional[torch.Tensor], eps: float, *, n_sum: int = 1,
                   gate: Optional[torch.Tensor] = None, cast_out: Optional[torch.Tensor] = None, keep=None,
                   normalize: bool = True, next_norm=None) -> None:
    """x[t] += weight * s / sqrt(mean(s^2) + eps) with s = (y[t * n_sum] + ... + y[t * n_sum + n_sum - 1]) *
    sigmoid(gate[t]); x float32 [n, d] in place, y float32 [n * n_sum, d], gate float32 [n, d] (rows may
    be strided: columns of a wider product) or None. `cast_out` [n, d] (float32 or bfloat16) gets the new
    rows rounded. `keep` = (state, ctx): before the update, the last rows of each request go to its input
    history, state[slot, position % ring] (the rows behind the step's tokens are left out). Without
    `normalize`: x[t] += s. `next_norm` = (weight float32 [d], eps): `cast_out` gets the new row's root-mean-square norm under
    that weight instead of the row itself (what the next sublayer reads)."""
    _dev(x, "x")
    _dev(y, "y")
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("gated_norm_add: x must be contiguous float32 [n, d]")
    if y.dtype != torch.float32 or not y.is_contiguous() or y.numel() != n * n_sum * d or n_sum < 1:
        raise KernelError(f"gated_norm_add: y must be contiguous float32 with {n_sum} rows of {d} a token, got {tuple(y.shape)} {y.dtype}")
    _f32vec(weight, "norm weight", d)
    gs = 0
    if gate is not None:
        gs = _rows(gate, "gate")
        if gate.dtype != torch.float32 or tuple(gate.shape) != (n, d):
            raise KernelError(f"gated_norm_add: the gate must be float32 [{n}, {d}], got {tuple(gate.shape)} {gate.dtype}")
    code = F32
    if cast_out is not None:
        _dev(cast_out, "cast_out")
        if tuple(cast_out.shape) != (n, d) or not cast_out.is_contiguous():
            raise KernelError(f"gated_norm_add: cast_out must be contiguous [{n}, {d}]")
        code = dtype_code(cast_out.dtype)
    if keep is not None and keep[1].n_tokens != n:
        raise KernelError("gated_norm_add: rows are kept for a step of as many rows as x has")
    next_w, next_eps = (None, 0.0) if next_norm is None else next_norm
    _f32vec(next_w, "the next norm's weight", d)
    if next_w is not None and cast_out is None:
        raise KernelError("gated_norm_add: the next norm's rows need a place (cast_out)")
    _lib.call("liyab_gated_norm_add", x.data_ptr(), _ptr(cast_out), code, y.data_ptr(), n_sum, _ptr(gate), gs, _ptr(weight), float(eps),
              1 if normalize else 0, n, d, *_keep_args(keep, d), _ptr(next_w), float(next_eps), _stream())


def keep_rows(x: torch.Tensor, state: torch.Tensor, ctx) -> None:
    """The last rows of each request in the step go to its input history (see `gated_norm_add`'s `keep`)."""
    _dev(x, "x")
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or ctx.n_tokens != n:
        raise KernelError("keep_rows: x must be the step's contiguous float32 rows")
    a = _keep_args((state, ctx), d)
    _lib.call("liyab_keep_rows", a[0], a[1], a[2], x.data_ptr(), *a[3:], n, d, _stream())


CONV_MAX_TAPS = 16


def causal_conv(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], ctx,
                cast_out: Optional[torch.Tensor] = None) -> None:
    """out[t] = x[t] + sum_j weight[:, j] * x[t - taps + 1 + j] over each request's own tokens in time, zeros
    before its start; x float32 [n, d] (the step's rows), weight float32 [d, taps], state float32 [slots,
    taps - 1, d] (position p of a request at ring place p % (taps - 1)) for what lies before the step's
    portion. out (and cast_out = x rounded) [n, d] float32 or bfloat16."""
    _dev(out, "out")
    _dev(x, "x")
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or ctx.n_tokens != n:
        raise KernelError("causal_conv: x must be the step's contiguous float32 rows")
    if tuple(out.shape) != (n, d) or not out.is_contiguous():
        raise KernelError(f"causal_conv: out must be contiguous [{n}, {d}]")
    if cast_out is not None and (tuple(cast_out.shape) != (n, d) or not cast_out.is_contiguous() or cast_out.dtype != out.dtype):
        raise KernelError("causal_conv: cast_out must match out")
    _dev(weight, "weight")
    if weight.dtype != torch.float32 or weight.dim() != 2 or weight.shape[0] != d or not weight.is_contiguous():
        raise KernelError(f"causal_conv: the weight must be contiguous float32 [{d}, taps], got {tuple(weight.shape)} {weight.dtype}")
    taps = weight.shape[1]
    if not 1 <= taps <= CONV_MAX_TAPS:
        raise KernelError(f"causal_conv: {taps} taps; 1 to {CONV_MAX_TAPS} are taken")
    n_slots = 0
    if taps > 1:
        if state is None or state.dtype != torch.float32 or tuple(state.shape[1:]) != (taps - 1, d) or not state.is_contiguous():
            raise KernelError(f"causal_conv: the state must be contiguous float32 [slots, {taps - 1}, {d}]")
        _dev(state, "state")
        n_slots = state.shape[0]
    _i32(ctx.tok_seq, "tok_seq", n)
    _i32(ctx.positions, "positions", n)
    _i32(ctx.seq_starts, "seq_starts", ctx.n_seqs + 1)
    _i32(ctx.state_slots, "state_slots", ctx.n_seqs)
    _lib.call("liyab_causal_conv", out.data_ptr(), _ptr(cast_out), dtype_code(out.dtype), x.data_ptr(), weight.data_ptr(), taps,
              _ptr(state) if taps > 1 else None, n_slots, ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), ctx.seq_starts.data_ptr(),
              ctx.state_slots.data_ptr(), n, d, _stream())


# -- latent attention's cached row, products a head, routed experts -------------------------------
def latent_store(cache: torch.Tensor, src: torch.Tensor, col_off: int, weight: Optional[torch.Tensor], eps: float,
                 slots: torch.Tensor, num_pages: Optional[int] = None) -> None:
    """cache[slot of t] = rmsnorm(src[t, col_off : col_off + rank]) * weight for each row t of the step; cache
    [pages, 1, page_size, rank] in src's dtype; slots int32 [n] = page * page_size + offset (a slot outside
    the pages is not written)."""
    _dev(cache, "cache")
    if cache.dim() != 4 or cache.shape[1] != 1 or not cache.is_contiguous() or cache.dtype != src.dtype:
        raise KernelError(f"latent_store: the cache must be contiguous [pages, 1, page_size, rank] in the rows' dtype, got {tuple(cache.shape)}")
    stride = _rows(src, "src")
    n, rank = src.shape[0], cache.shape[3]
    if col_off < 0 or col_off + rank > src.shape[1]:
        raise KernelError("latent_store: the columns pass the source's width")
    _f32vec(weight, "norm weight", rank)
    _i32(slots, "slots", n)
    _lib.call("liyab_latent_store", cache.data_ptr(), dtype_code(src.dtype), src.data_ptr(), stride, col_off, _ptr(weight), float(eps),
              slots.data_ptr(), n, rank, cache.shape[2], _pages(cache, num_pages), _stream())


GROUPED_ROWS = 64  # rows a tile of the grouped product (csrc/grouped_product.hip: kGroupedRows)
SKINNY_ROWS = 16  # or as few as this, for steps in which a group gets few rows (kSkinnyRows)


def heads_product(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, gate: Optional[torch.Tensor] = None) -> None:
    """out[t, h * N + j] = sum_k a[t, h * K + k] * w[h, j, k] (* sigmoid(gate[t, h * N + j])): a product of
    its own for every head. a [n, >= H * K] and out [n, >= H * N] may be column ranges of wider rows; w
    [H, N, K] contiguous in a's dtype; gate float32 or bfloat16 logits, or None."""
    _dev(w, "w")
    if w.dim() != 3 or not w.is_contiguous() or w.dtype != a.dtype:
        raise KernelError(f"heads_product: w must be contiguous [heads, N, K] in a's dtype, got {tuple(w.shape)} {w.dtype}")
    H, N, K = w.shape
    lda, ldo = _rows(a, "a"), _rows(out, "out")
    n = a.shape[0]
    if a.shape[1] != H * K or tuple(out.shape) != (n, H * N):
        raise KernelError(f"heads_product: a {tuple(a.shape)} / out {tuple(out.shape)} do not fit {H} heads of {K} -> {N}")
    gs = 0
    if gate is not None:
        gs = _rows(gate, "gate")
        if tuple(gate.shape) != (n, H * N):
            raise KernelError(f"heads_product: the gate must be [{n}, {H * N}]")
    # few rows: tiles of 16 rows x 16 features, so that some hundred workgroups share the heads' matrices (64 rows of 12
    # heads, 128 -> 64: 10 us in 12 tiles of 64 x 64)
    block = SKINNY_ROWS if (n <= 128 and a.dtype == torch.bfloat16 and K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0
                            and w.data_ptr() % 16 == 0) else GROUPED_ROWS
    _lib.call("liyab_grouped_product", a.data_ptr(), lda, 1, K, w.data_ptr(), None, dtype_code(a.dtype), out.data_ptr(),
              dtype_code(out.dtype), ldo, N, None, None, (n + block - 1) // block, block, H, None, _ptr(gate),
              dtype_code(gate.dtype) if gate is not None else F32, gs, n, N, K, 0, 1, 0, _stream())


MOE_MAX_TOP = 64


def moe_tiles(n_entries: int, n_experts: int, block: int = GROUPED_ROWS) -> int:
    """The tiles of `block` places that hold `n_entries` entries listed by expert, whatever their
    experts: a bound that follows from the sizes alone."""
    return -(-(n_entries + min(n_entries, n_experts) * (block - 1)) // block)


def moe_block(n_entries: int, n_experts: int, dtype: torch.dtype, *inner_sizes: int) -> int:
    """The row places a tile for a step of `n_entries` (token, choice) entries: 16 while an expert gets 32
    rows or fewer on average (the products are then streams of the chosen experts' weights, and tiles of 16
    rows x 16 features make some hundred workgroups pull on them where tiles of 64 x 64 make a few dozen:
    one token of 2 x 1,536 features over 768, 16.4 -> 6 us), 64 beyond; the small tiles are for bfloat16
    operands whose inner sizes are multiples of 8."""
    few = n_entries <= 32 * n_experts and dtype == torch.bfloat16 and all(k % 8 == 0 for k in inner_sizes)
    return SKINNY_ROWS if few else GROUPED_ROWS


MOE_MAX_GROUPS = 64


def moe_route(logits: torch.Tensor, top: int, ids: torch.Tensor, weights: torch.Tensor, rows_list: torch.Tensor,
              tile_group: torch.Tensor, block: int = GROUPED_ROWS, groups: Optional[tuple] = None) -> None:
    """From float32 router logits [n, experts] (rows may be strided): ids int32 and weights float32 [n,
    top] (the experts with the largest logits, softmax over those alone), and the entries t * top + k
    listed by expert in tiles of `block` places: rows_list int32 [tiles * block] (-1: empty), tile_group
    int32 [tiles] (-1: unused), tiles = moe_tiles(n * top, experts, block). `groups` = (count, keep): the choice among groups
    of experts instead: softmax over all experts, the experts in `count` equal groups of neighbours, only those of the `keep`
    groups with the largest member can be chosen, the weights the chosen scores divided by their sum."""
    ld = _rows(logits, "logits")
    n, E = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("moe_route: the logits must be float32")
    if not 1 <= top <= min(E, MOE_MAX_TOP):
        raise KernelError(f"moe_route: {top} of {E} experts a token (at most {MOE_MAX_TOP})")
    if block not in (GROUPED_ROWS, SKINNY_ROWS):
        raise KernelError(f"moe_route: tiles of {block} places ({GROUPED_ROWS} or {SKINNY_ROWS})")
    tiles = moe_tiles(n * top, E, block)
    _i32(ids, "ids", n * top)
    _i32(rows_list, "rows_list", tiles * block)
    _i32(tile_group, "tile_group", tiles)
    _dev(weights, "weights")
    if weights.dtype != torch.float32 or weights.numel() < n * top or not weights.is_contiguous():
        raise KernelError("moe_route: weights must be contiguous float32 [n, top]")
    mode, count, keep = 0, 1, 1
    if groups is not None:
        mode, count, keep = 1, int(groups[0]), int(groups[1])
        if not (1 <= count <= MOE_MAX_GROUPS and E % count == 0 and 1 <= keep <= count and top <= keep * (E // count)):
            raise KernelError(f"moe_route: {keep} of {count} groups of {E} experts do not hold {top} choices (at most {MOE_MAX_GROUPS} groups)")
    if n <= 1024:  # one launch: a thread routes a token, then the workgroup lists the entries
        _lib.call("liyab_moe_route_align", logits.data_ptr(), ld, n, E, top, ids.data_ptr(), weights.data_ptr(), block,
                  rows_list.data_ptr(), tile_group.data_ptr(), tiles, mode, count, keep, _stream())
        return
    _lib.call("liyab_moe_route", logits.data_ptr(), ld, n, E, top, ids.data_ptr(), weights.data_ptr(), mode, count, keep, _stream())
    _lib.call("liyab_moe_align", ids.data_ptr(), n * top, E, block, rows_list.data_ptr(), tile_group.data_ptr(), tiles, _stream())


def moe_product(out: torch.Tensor, a: torch.Tensor, w0: torch.Tensor, w1: Optional[torch.Tensor], rows_list: torch.Tensor,
                tile_group: torch.Tensor, *, a_div: int = 1, row_scale: Optional[torch.Tensor] = None, block: int = GROUPED_ROWS,
                act: str = "none", out_div: int = 1, out_extra: int = 0) -> None:
    """For every listed entry e of expert g: out[e] = f(a[e // a_div] . w0[g]^T, a[e // a_div] . w1[g]^T) *
    row_scale[e], f(u, v) = silu(u) * v with two matrices and u with one. a [*, K] and out [entries, N]
    contiguous, w0 / w1 [experts, N, K] in a's dtype; rows_list and tile_group as `moe_route` leaves them for
    tiles of `block` places. `act` = "relu2" (one matrix): f(u) = relu(u)^2. `out_extra`: rows of `out` left free behind each
    `out_div` rows (a token's entries), which another product fills: entry e then lies at row e + (e // out_div) * out_extra."""
    _dev(w0, "w0")
    if w0.dim() != 3 or not w0.is_contiguous() or w0.dtype != a.dtype:
        raise KernelError(f"moe_product: w0 must be contiguous [experts, N, K] in a's dtype, got {tuple(w0.shape)} {w0.dtype}")
    E, N, K = w0.shape
    if w1 is not None and (tuple(w1.shape) != (E, N, K) or not w1.is_contiguous() or w1.dtype != a.dtype):
        raise KernelError("moe_product: w1 must match w0")
    lda, ldo = _rows(a, "a"), _rows(out, "out")
    if act not in ("none", "relu2") or (act != "none" and w1 is not None) or out_extra < 0 or out_div < 1 or (out_extra and out.shape[0] % (out_div + out_extra)):
        raise KernelError(f"moe_product: activation '{act}' / {out_extra} free rows a token are not taken here")
    entries = out.shape[0] // (out_div + out_extra) * out_div if out_extra else out.shape[0]
    if a.shape[1] != K or out.shape[1] != N or a_div < 1 or a.shape[0] * a_div < entries:
        raise KernelError(f"moe_product: a {tuple(a.shape)} / out {tuple(out.shape)} do not fit [{E}, {N}, {K}] with {a_div} entries a row")
    tiles = tile_group.numel()
    if block not in (GROUPED_ROWS, SKINNY_ROWS) or (block == SKINNY_ROWS and (a.dtype != torch.bfloat16 or K % 8 != 0 or lda % 8 != 0)):
        raise KernelError(f"moe_product: tiles of {block} places do not go with these operands")
    if tiles < moe_tiles(entries, E, block):
        raise KernelError(f"moe_product: {tiles} tiles do not hold {entries} entries of {E} experts")
    _i32(rows_list, "rows_list", tiles * block)
    _i32(tile_group, "tile_group", tiles)
    if row_scale is not None:
        _dev(row_scale, "row_scale")
        if row_scale.dtype != torch.float32 or row_scale.numel() < entries or not row_scale.is_contiguous():
            raise KernelError("moe_product: row_scale must be contiguous float32 [entries]")
    _lib.call("liyab_grouped_product", a.data_ptr(), lda, a_div, 0, w0.data_ptr(), _ptr(w1), dtype_code(a.dtype), out.data_ptr(),
              dtype_code(out.dtype), ldo, 0, rows_list.data_ptr(), tile_group.data_ptr(), tiles, block, E, _ptr(row_scale), None, F32, 0,
              entries, N, K, 1 if act == "relu2" else 0, int(out_div), int(out_extra), _stream())


# -- norms without statistics, clamped gated activations, two sublayers' results joined ------------
def dyt(out: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], alpha: torch.Tensor,
        rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = tanh(alpha * x[rows[r]] (or x[r])) * weight + bias; x float32 [*, d], alpha one float32 value on the
    device, out [n, d] float32 or bfloat16."""
    _dev(out, "out")
    _dev(x, "x")
    n, d = out.shape
    if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != d or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"dyt: x must be contiguous float32 [*, {d}] and out contiguous, got {tuple(x.shape)} {x.dtype}")
    _f32vec(weight, "norm weight", d)
    _f32vec(bias, "norm bias", d)
    _f32vec(alpha, "norm alpha", 1)
    if rows is not None:
        _i32(rows, "rows", n)
    elif x.shape[0] < n:
        raise KernelError("dyt: fewer input rows than output rows")
    _lib.call("liyab_dyt", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), _ptr(weight), _ptr(bias), alpha.data_ptr(), _ptr(rows), n, d, _stream())


def glu_clamped(out: torch.Tensor, gu: torch.Tensor, limit: float, slope: float, shift: float) -> None:
    """out = g * sigmoid(slope * g) * (u + shift) with g = min(G, limit), u = clamp(U, -limit, limit); gu float32
    [n, 2 * ff] = [G | U], out contiguous [n, ff] float32 or bfloat16."""
    _dev(out, "out")
    ld = _rows(gu, "gu")
    n, ff = out.shape
    if gu.dtype != torch.float32 or tuple(gu.shape) != (n, 2 * ff) or not out.is_contiguous():
        raise KernelError(f"glu_clamped: needs float32 [n, {2 * ff}] and a contiguous out [n, {ff}], got {tuple(gu.shape)} {gu.dtype}")
    _lib.call("liyab_glu_clamped", out.data_ptr(), dtype_code(out.dtype), gu.data_ptr(), ld, n, ff, float(limit), float(slope), float(shift), _stream())


ACTIVATE = {"tanh": 0, "silu": 1, "sigmoid": 2, "relu2": 3}


def activate(out: torch.Tensor, x: torch.Tensor, op: str) -> None:
    """out = op(x), x float32 rows, out rows of the same shape in float32 or bfloat16."""
    ldo, ldi = _rows(out, "out"), _rows(x, "x")
    if x.dtype != torch.float32 or out.shape != x.shape:
        raise KernelError("activate: x must be float32 and out of its shape")
    _lib.call("liyab_activate", out.data_ptr(), dtype_code(out.dtype), ldo, x.data_ptr(), ldi, ACTIVATE[op], x.shape[0], x.shape[1], _stream())


def mean_norm_add(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float, weight: float = 0.5) -> None:
    """x += weight * (a / rms(a) * wa + b / rms(b) * wb), all float32 [n, d] contiguous, rms over a row with eps inside the root."""
    n, d = x.shape
    for t, what in ((x, "x"), (a, "a"), (b, "b")):
        _dev(t, what)
        if t.dtype != torch.float32 or tuple(t.shape) != (n, d) or not t.is_contiguous():
            raise KernelError(f"mean_norm_add: {what} must be contiguous float32 [{n}, {d}]")
    _f32vec(wa, "weight a", d)
    _f32vec(wb, "weight b", d)
    _lib.call("liyab_mean_norm_add", x.data_ptr(), a.data_ptr(), b.data_ptr(), wa.data_ptr(), wb.data_ptr(), float(eps), float(weight), n, d, _stream())


# -- mixers with a matrix of state a head ---------------------------------------------------------------
def scan_takes(rows: int, cols: int) -> bool:
    """Whether the recurrence kernel takes a state of rows x cols a head (csrc/recurrent.hip: scan_shape): a column a
    thread of 512, up to 64 rows of it in registers (a multiple of 4), sixteen tokens' vectors staged in at most 128 KiB of LDS."""
    threads = 512
    if rows <= 0 or not 0 < cols <= threads:
        return False
    lanes = 1
    while lanes < cols:
        lanes *= 2
    while threads // lanes > 1 and (threads // lanes) * 4 > -(-rows // 4) * 4:
        lanes *= 2
    blocks = threads // lanes
    per = -(-(-(-rows // blocks)) // 4) * 4
    staged = blocks * per
    return per <= 64 and 4 * (3 * 16 * staged + 2 * 16 * lanes + 16 * threads) <= 128 * 1024


SCAN_SEGMENT = 64  # tokens a segment where a long portion's recurrence runs in segments side by side
SCAN_SEGMENT_FROM = 192  # the longest portion of a step from which it does


def _scan_segments(ctx, n: int, n_head: int, rows: int, cols: int):
    """(tokens a segment, the most segments, scratch for the segments' states, for their decays) for a step's recurrence: in
    segments side by side when some request brings a long portion, else (0, 0, None, None). The grids follow from the step's
    rows and requests, never from the portions' lengths."""
    if ctx.host.max_q_len < SCAN_SEGMENT_FROM:
        return 0, 0, None, None
    most = -(-n // SCAN_SEGMENT) + ctx.n_seqs
    state = ctx.workspace.get("scan_seg_state", (most, n_head, rows, cols), torch.float32)
    decay = ctx.workspace.get("scan_seg_decay", (most, n_head, rows), torch.float32)
    return SCAN_SEGMENT, most, state.data_ptr(), decay.data_ptr()


def _step_lists(ctx, n: int) -> None:
    _i32(ctx.tok_seq, "tok_seq", n)
    _i32(ctx.positions, "positions", n)
    _i32(ctx.seq_starts, "seq_starts", ctx.n_seqs + 1)
    _i32(ctx.state_slots, "state_slots", ctx.n_seqs)


def _state(state: torch.Tensor, what: str) -> int:
    _dev(state, "state")
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous():
        raise KernelError(f"{what}: the state must be contiguous float32 [slots, floats a slot], got {tuple(state.shape)} {state.dtype}")
    return state.shape[1]


def token_shift(out: torch.Tensor, h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, prev_off: int, ctx) -> None:
    """out[t, c] = h[t] + (h[t - 1] - h[t]) * mu[c]; h [n, d] in the compute dtype, mu float32 [n_mix, d], out [n, n_mix, d];
    the row before a request's first row of the step is state[slot, prev_off : prev_off + d], zeros at position 0."""
    _dev(out, "out")
    _dev(h, "h")
    n, d = h.shape
    stride = _state(state, "token_shift")
    if not h.is_contiguous() or not out.is_contiguous() or out.dtype != h.dtype or mu.dim() != 2 or tuple(out.shape) != (n, mu.shape[0], d):
        raise KernelError("token_shift: h [n, d] and out [n, n_mix, d] must be contiguous and of one dtype")
    _f32vec(mu, "mu", mu.shape[0] * d)
    if prev_off < 0 or prev_off + d > stride or ctx.n_tokens != n:
        raise KernelError("token_shift: the previous row does not lie in the slot, or h is not the step's rows")
    _step_lists(ctx, n)
    _lib.call("liyab_token_shift", out.data_ptr(), dtype_code(h.dtype), h.data_ptr(), mu.data_ptr(), mu.shape[0], state.data_ptr() + 4 * prev_off,
              stride, state.shape[0], ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), ctx.seq_starts.data_ptr(), ctx.state_slots.data_ptr(),
              n, d, _stream())


def wkv_scan(out: torch.Tensor, proj: torch.Tensor, w0: torch.Tensor, u: torch.Tensor, norm_w: torch.Tensor, eps: float, state: torch.Tensor,
             h: torch.Tensor, ctx, *, n_head: int, head_dim: int) -> None:
    """The decayed outer-product recurrence with a bonus over each request's rows of the step. proj float32 [n, 5 * H * D] =
    [r | k | v | gate logits | raw decay]; decay = exp(-exp(raw + w0)); per head o = (S + diag(u) k v^T)^T r, S <- diag(decay) S
    + k v^T; out [n, H * D] (compute dtype) = o / rms(o over the head) * norm_w * silu(gate). state float32 [slots, H * D * D + width]:
    the heads' matrices, then the request's last row of h [n, width], which is kept here for the next step's token shift."""
    _dev(out, "out")
    n, HD = out.shape
    H, D = n_head, head_dim
    stride = _state(state, "wkv_scan")
    ld = _rows(proj, "proj")
    if HD != H * D or proj.dtype != torch.float32 or tuple(proj.shape) != (n, 5 * HD) or not out.is_contiguous():
        raise KernelError(f"wkv_scan: needs float32 proj [n, {5 * H * D}] and a contiguous out [n, {H * D}], got {tuple(proj.shape)} {proj.dtype}")
    for t, what in ((w0, "w0"), (u, "u"), (norm_w, "norm weight")):
        _f32vec(t, what, HD)
    _dev(h, "h")
    if h.dim() != 2 or h.shape[0] != n or not h.is_contiguous() or stride != H * D * D + h.shape[1] or ctx.n_tokens != n:
        raise KernelError("wkv_scan: the state must hold the heads' matrices and one row of h")
    if not scan_takes(D, D):
        raise KernelError(f"wkv_scan: heads of {D} are not taken")
    _step_lists(ctx, n)
    p = proj.data_ptr()
    _lib.call("liyab_wkv_scan", out.data_ptr(), dtype_code(out.dtype), p, p + 4 * HD, p + 8 * HD, p + 16 * HD, p + 12 * HD, ld, w0.data_ptr(),
              u.data_ptr(), norm_w.data_ptr(), float(eps), state.data_ptr(), stride, state.shape[0], h.data_ptr(), dtype_code(h.dtype),
              h.shape[1], h.shape[1], H * D * D, ctx.seq_starts.data_ptr(), ctx.positions.data_ptr(), ctx.state_slots.data_ptr(), ctx.n_seqs,
              H, D, *_scan_segments(ctx, n, H, D, D), _stream())


def conv_act(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
             ring_off: int, ctx, act: bool = True) -> None:
    """(`act` False: without the silu.) out[t, c] = silu(bias[c] + sum_j weight[c, j] * x[t - taps + 1 + j, c]) over each request's own rows in time; x, out float32
    rows (columns of wider rows are fine), weight float32 [C, taps]; the rows before a request's first row of the step come from
    state[slot, ring_off + (position % (taps - 1)) * C + c], zeros before position 0."""
    ldo, ldi = _rows(out, "out"), _rows(x, "x")
    n, C = x.shape
    if x.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (n, C) or ctx.n_tokens != n:
        raise KernelError("conv_act: x and out must be the step's float32 rows of one shape")
    _dev(weight, "weight")
    if weight.dtype != torch.float32 or weight.dim() != 2 or weight.shape[0] != C or not weight.is_contiguous():
        raise KernelError(f"conv_act: the weight must be contiguous float32 [{C}, taps]")
    taps = weight.shape[1]
    _f32vec(bias, "bias", C)
    stride, slots, base = 0, 0, None
    if taps > 1:
        stride = _state(state, "conv_act")
        if ring_off < 0 or ring_off + (taps - 1) * C > stride:
            raise KernelError("conv_act: the ring does not lie in the slot")
        slots, base = state.shape[0], state.data_ptr() + 4 * ring_off
    _step_lists(ctx, n)
    _lib.call("liyab_conv_act", out.data_ptr(), ldo, x.data_ptr(), ldi, weight.data_ptr(), _ptr(bias), taps, base, stride, slots,
              ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), ctx.seq_starts.data_ptr(), ctx.state_slots.data_ptr(), n, C, 1 if act else 0,
              _stream())


def ssd_scan(y: torch.Tensor, xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
             state: torch.Tensor, keep_src: Optional[torch.Tensor], keep_ring: int, ctx, *, n_head: int, head_dim: int, n_state: int,
             n_groups: int) -> None:
    """The selective state-space recurrence over each request's rows of the step: dt = softplus(dt_raw + dt_bias), per head
    S <- exp(-exp(a_log) dt) S + dt B x^T, y = S^T C + d_skip x. xbc float32 [n, inner + 2 * groups * state] = [x | B | C],
    dt_raw float32 [n, heads] (columns of wider rows are fine), y float32 [n, inner]. state float32 [slots, inner * state +
    keep_ring * channels]: the heads' matrices, then the last `keep_ring` rows of keep_src [n, channels] at ring place position %
    keep_ring, which are kept here for the next step's convolution."""
    H, P, N, G = n_head, head_dim, n_state, n_groups
    inner = H * P
    n = y.shape[0]
    ldy, ldx, ldp = _rows(y, "y"), _rows(xbc, "xbc"), _rows(dt_raw, "dt_raw")
    stride = _state(state, "ssd_scan")
    if (y.dtype != torch.float32 or xbc.dtype != torch.float32 or dt_raw.dtype != torch.float32 or tuple(y.shape) != (n, inner)
            or tuple(xbc.shape) != (n, inner + 2 * G * N) or tuple(dt_raw.shape) != (n, H) or ctx.n_tokens != n):
        raise KernelError("ssd_scan: y [n, inner], xbc [n, inner + 2 groups x state] and dt_raw [n, heads] must be the step's float32 rows")
    for t, what in ((dt_bias, "dt_bias"), (a_log, "A_log"), (d_skip, "D")):
        _f32vec(t, what, H)
    kptr, kld, kw = None, 0, 0
    if keep_src is not None and keep_ring > 0:
        kld = _rows(keep_src, "keep_src")
        kw = keep_src.shape[1]
        if keep_src.dtype != torch.float32 or keep_src.shape[0] != n:
            raise KernelError("ssd_scan: the kept rows must be the step's float32 rows")
        kptr = keep_src.data_ptr()
    if stride != inner * N + (keep_ring * kw if kptr is not None else 0):
        raise KernelError("ssd_scan: the state must hold the heads' matrices and the kept rows")
    if not scan_takes(N, P):
        raise KernelError(f"ssd_scan: a state of {N} x {P} a head is not taken")
    _step_lists(ctx, n)
    _lib.call("liyab_ssd_scan", y.data_ptr(), ldy, xbc.data_ptr(), ldx, dt_raw.data_ptr(), ldp, dt_bias.data_ptr(), a_log.data_ptr(),
              d_skip.data_ptr(), state.data_ptr(), stride, state.shape[0], kptr, kld, kw, keep_ring if kptr is not None else 0, inner * N,
              ctx.seq_starts.data_ptr(), ctx.positions.data_ptr(), ctx.state_slots.data_ptr(), ctx.n_seqs, H, P, N, G,
              *_scan_segments(ctx, n, H, N, P), _stream())


def gated_group_norm(out: torch.Tensor, y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float, groups: int) -> None:
    """out = (y * silu(z)) / rms(.) * weight, the root mean square over each of `groups` equal parts of a row; y, z float32 rows
    [n, inner] (columns of wider rows are fine), out contiguous [n, inner] float32 or bfloat16."""
    _dev(out, "out")
    ldy, ldz = _rows(y, "y"), _rows(z, "z")
    n, inner = out.shape
    if y.dtype != torch.float32 or z.dtype != torch.float32 or tuple(y.shape) != (n, inner) or tuple(z.shape) != (n, inner) or not out.is_contiguous():
        raise KernelError("gated_group_norm: y and z must be float32 [n, inner], out contiguous [n, inner]")
    if groups < 1 or inner % groups != 0:
        raise KernelError(f"gated_group_norm: {inner} channels in {groups} parts")
    _f32vec(weight, "norm weight", inner)
    _lib.call("liyab_gated_group_norm", out.data_ptr(), dtype_code(out.dtype), y.data_ptr(), ldy, z.data_ptr(), ldz, weight.data_ptr(), float(eps),
              n, inner, groups, _stream())


# -- attention whose scores are more than scale * q . k ---------------------------------------------------
def qk_prepare(src: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, slots: torch.Tensor, positions: torch.Tensor,
               *, q_off: int, k_off: int, v_off: int, n_head: int, q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
               eps: float = 0.0, freqs: Optional[torch.Tensor] = None, rot_dims: int = 0, temp_coef: float = 0.0, temp_every: int = 0,
               num_pages: Optional[int] = None, head_dim: Optional[int] = None, value_dim: Optional[int] = None, rot_halves: bool = False,
               rot_mag: float = 1.0, v_keep: Optional[torch.Tensor] = None, v_first: Optional[torch.Tensor] = None,
               v_lam: Optional[torch.Tensor] = None) -> None:
    """From a projection's float32 rows `src` (queries at column q_off, keys at k_off, values at v_off, which may be k_off) to
    queries in `q_out` [n, heads * dk] and keys and values in their slots of the pages (k_cache [pages, kv_heads, page, dk],
    v_cache [.., dv]), all in the compute dtype. Per head, each optional: a root-mean-square norm with a weight [dk] (queries,
    keys), pairs (2i, 2i + 1) of the first rot_dims entries turned by position * freqs[i] (queries, keys; freqs float64), the query times
    1 + temp_coef * ln(floor((position + 1) / temp_every) + 1). A slot outside the pages is not written. `head_dim`,
    `value_dim`: the heads' own widths where the caches' rows (and the queries') are wider, zeros behind the heads. `rot_halves`:
    the turned pairs are (i, i + rot_dims / 2) instead; `rot_mag` multiplies cosine and sine. `v_keep` (float32 [n, kv_heads * dv]) gets
    the values as projected, for later layers of the step; `v_first` (such rows) and `v_lam` (one float32 on the device): the values
    cached are (1 - lam) v + lam v_first."""
    ld = _rows(src, "src")
    n = src.shape[0]
    _dev(q_out, "q_out")
    _dev(k_cache, "k_cache")
    _dev(v_cache, "v_cache")
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.shape[:3] != v_cache.shape[:3] or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("qk_prepare: caches must be contiguous [pages, kv_heads, page_size, width] with the same pages")
    _, G, page, dk_out = k_cache.shape
    dv_out = v_cache.shape[3]
    dk, dv = head_dim or dk_out, value_dim or dv_out
    if not (0 < dk <= dk_out and 0 < dv <= dv_out):
        raise KernelError(f"qk_prepare: heads of {dk} / {dv} in rows of {dk_out} / {dv_out}")
    if src.dtype != torch.float32 or tuple(q_out.shape) != (n, n_head * dk_out) or not q_out.is_contiguous() or not (q_out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("qk_prepare: src must be float32 rows, q_out contiguous [n, heads * dk], queries and caches of one dtype")
    if min(q_off, k_off, v_off) < 0 or q_off + n_head * dk > src.shape[1] or k_off + G * dk > src.shape[1] or v_off + G * dv > src.shape[1]:
        raise KernelError("qk_prepare: the heads' columns pass the source's rows")
    _f32vec(q_norm, "query norm weight", dk)
    _f32vec(k_norm, "key norm weight", dk)
    if rot_dims:
        if rot_dims % 2 or rot_dims > dk or freqs is None:
            raise KernelError(f"qk_prepare: {rot_dims} turned entries of heads of {dk}")
        _dev(freqs, "freqs")
        if freqs.dtype != torch.float64 or not freqs.is_contiguous() or freqs.numel() != rot_dims // 2:
            raise KernelError(f"qk_prepare: the frequencies must be {rot_dims // 2} contiguous float64 values")
    _i32(slots, "slots", n)
    _i32(positions, "positions", n)
    for kept, what in ((v_keep, "v_keep"), (v_first, "v_first")):
        _f32vec(kept, what, n * G * dv)
    _f32vec(v_lam, "v_lam", 1)
    if (v_first is None) != (v_lam is None) or (v_keep is not None and v_first is not None):
        raise KernelError("qk_prepare: values are kept, or mixed with kept ones at a rate")
    _lib.call("liyab_qk_prepare", src.data_ptr(), ld, q_off, k_off, v_off, n_head, G, dk, dv, dk_out, dv_out, q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
              dtype_code(q_out.dtype), slots.data_ptr(), page, _pages(k_cache, num_pages), _ptr(q_norm), _ptr(k_norm), float(eps),
              _ptr(freqs) if rot_dims else None, rot_dims, float(temp_coef), int(temp_every), positions.data_ptr(), n,
              1 if rot_halves else 0, float(rot_mag), _ptr(v_keep), _ptr(v_first), _ptr(v_lam), _stream())


def attention_scored(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor, ctx, *,
                     n_head: int, scale: float, softcap: float = 0.0, window: int = 0, bias_table: Optional[torch.Tensor] = None,
                     gate: Optional[torch.Tensor] = None, num_pages: Optional[int] = None, sinks: Optional[torch.Tensor] = None) -> None:
    """Causal attention of the step's rows over their requests' pages with score = scale * q . k, then cap * tanh(score / cap)
    (softcap > 0), then + bias_table[min(distance, rows - 1), head] (float32 [rows, heads]); softmax in 32-bit; values `dv` wide.
    out [n, heads * dv] = result * sigmoid(gate) (gate: float32 rows [n, heads * dv], or None). `sinks` (float32 [heads]):
    exp(sinks[head]) joins the softmax's denominator."""
    _dev(out, "out")
    _dev(q, "q")
    n = out.shape[0]
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.shape[:3] != v_cache.shape[:3] or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention_scored: caches must be contiguous [pages, kv_heads, page_size, width] with the same pages")
    _, G, page, dk = k_cache.shape
    dv = v_cache.shape[3]
    so, sq = _rows(out, "out"), _rows(q, "q")
    if tuple(q.shape) != (n, n_head * dk) or tuple(out.shape) != (n, n_head * dv) or not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention_scored: q [n, heads * dk], out [n, heads * dv] and the caches must share a dtype")
    if n_head % G or dv > 256 or dk > 512:
        raise KernelError(f"attention_scored: {n_head} heads over {G}, keys of {dk}, values of {dv} are not taken")
    if block_tables.dim() != 2 or block_tables.shape[0] < ctx.n_seqs:
        raise KernelError("attention_scored: block_tables must be [requests, max_blocks]")
    _i32(block_tables, "block_tables")
    _i32(ctx.tok_seq, "tok_seq", n)
    _i32(ctx.positions, "positions", n)
    max_dist = 0
    if bias_table is not None:
        _dev(bias_table, "bias_table")
        if bias_table.dtype != torch.float32 or bias_table.dim() != 2 or bias_table.shape[1] != n_head or not bias_table.is_contiguous():
            raise KernelError(f"attention_scored: the bias table must be contiguous float32 [distances, {n_head}]")
        max_dist = bias_table.shape[0] - 1
    gs = 0
    if gate is not None:
        gs = _rows(gate, "gate")
        if gate.dtype != torch.float32 or tuple(gate.shape) != (n, n_head * dv):
            raise KernelError("attention_scored: the gate must be float32 rows [n, heads * dv]")
    _f32vec(sinks, "sinks", n_head)
    _lib.call("liyab_attention_scored", out.data_ptr(), so, q.data_ptr(), sq, k_cache.data_ptr(), v_cache.data_ptr(), dtype_code(q.dtype),
              block_tables.data_ptr(), block_tables.shape[1], ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), n, float(scale), float(softcap),
              int(window), _ptr(bias_table), max_dist, _ptr(gate), gs, n_head, G, dk, dv, page, _pages(k_cache, num_pages), _ptr(sinks), _stream())


def gate_rows(x: torch.Tensor, gate: torch.Tensor, scale: float = 1.0) -> None:
    """x *= scale * sigmoid(gate) in place; x rows in float32 or bfloat16, gate float32 rows of the same shape (columns of wider
    rows are fine)."""
    ldx, ldg = _rows(x, "x"), _rows(gate, "gate")
    if gate.dtype != torch.float32 or gate.shape != x.shape:
        raise KernelError("gate_rows: the gate must be float32 and of x's shape")
    _lib.call("liyab_gate_rows", x.data_ptr(), dtype_code(x.dtype), ldx, gate.data_ptr(), ldg, x.shape[0], x.shape[1], float(scale), _stream())


# -- two norms of one stream with a convolution over time each; rings of kept rows; small row kernels ---------
SHIFT_MAX_TAPS = 16


class StateSlice:
    """A stretch of a layer's per-request state [slots, floats a slot] float32 that one part owns: `offset` floats from a
    slot's start, `size` floats long. Kernels get the stretch's address in slot 0 and the slots' stride."""

    def __init__(self, state: torch.Tensor, offset: int, size: int):
        stride = _state(state, "a part's state")
        if offset < 0 or size < 0 or offset + size > stride:
            raise KernelError(f"a stretch of {size} floats at {offset} does not lie in a slot of {stride}")
        self.state, self.offset, self.size = state, int(offset), int(size)

    @property
    def stride(self) -> int:
        return self.state.shape[1]

    @property
    def n_slots(self) -> int:
        return self.state.shape[0]

    def data_ptr(self) -> int:
        return self.state.data_ptr() + 4 * self.offset

    def sub(self, offset: int, size: int) -> "StateSlice":
        if offset < 0 or offset + size > self.size:
            raise KernelError("a stretch past its owner's")
        return StateSlice(self.state, self.offset + offset, size)


def norm_shift(out: torch.Tensor, x: torch.Tensor, weights: torch.Tensor, offset: float, eps: float, conv: Optional[torch.Tensor],
               ring: Optional[StateSlice], ctx, hbuf: Optional[torch.Tensor] = None, keep_single: bool = False) -> None:
    """out[s, t] = h_s[t] + sum_j conv[s, :, j] * h_s[t - taps + 1 + j] with h_s = x / sqrt(mean(x^2) + eps) * (weights[s] + offset)
    over each request's own rows in time (conv None: out = h). x float32 [n, d] (the step's rows), weights float32 [S, d],
    conv float32 [S, taps, d] (a tap's channels side by side), out [S, n, d] float32 or bfloat16; rows before the step's portion come from `ring` ((taps - 1) x
    [S, d] floats, position p at place p % (taps - 1)); `hbuf` float32 [n, S * d] gets h itself, for `ring_keep`. `keep_single`: a
    request that brings one token keeps its row in the ring here; a step of single tokens (`single_token_step`) then needs neither
    `hbuf` nor `ring_keep`."""
    _dev(out, "out")
    _dev(x, "x")
    n, d = x.shape
    S = weights.shape[0] if weights.dim() == 2 else 0
    if x.dtype != torch.float32 or not x.is_contiguous() or ctx.n_tokens != n:
        raise KernelError("norm_shift: x must be the step's contiguous float32 rows")
    if not 1 <= S <= 2 or tuple(out.shape) != (S, n, d) or not out.is_contiguous():
        raise KernelError(f"norm_shift: out must be contiguous [{S}, {n}, {d}] for one or two sublayers")
    _f32vec(weights, "norm weights", S * d)
    taps = 0
    if conv is not None:
        _dev(conv, "conv")
        if conv.dtype != torch.float32 or conv.dim() != 3 or (conv.shape[0], conv.shape[2]) != (S, d) or not conv.is_contiguous():
            raise KernelError(f"norm_shift: the convolution's weights must be contiguous float32 [{S}, taps, {d}]")
        taps = conv.shape[1]
        if not 1 <= taps <= SHIFT_MAX_TAPS:
            raise KernelError(f"norm_shift: {taps} taps; 1 to {SHIFT_MAX_TAPS} are taken")
    if taps > 1 and (ring is None or ring.size != (taps - 1) * S * d):
        raise KernelError(f"norm_shift: {taps} taps need a ring of {(taps - 1) * S * d} floats a slot")
    if hbuf is not None and (hbuf.dtype != torch.float32 or tuple(hbuf.shape) != (n, S * d) or not hbuf.is_contiguous()):
        raise KernelError(f"norm_shift: hbuf must be contiguous float32 [{n}, {S * d}]")
    _step_lists(ctx, n)
    _lib.call("liyab_norm_shift", out.data_ptr(), dtype_code(out.dtype), _ptr(hbuf), x.data_ptr(), weights.data_ptr(), float(offset), float(eps),
              _ptr(conv), taps, ring.data_ptr() if taps > 1 else None, ring.stride if taps > 1 else 0, ring.n_slots if taps > 1 else 0,
              ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), ctx.seq_starts.data_ptr(), ctx.state_slots.data_ptr(), n, d, S,
              1 if keep_single and taps > 1 else 0, _stream())


def single_token_step(ctx) -> bool:
    """Whether every request of the step brings one token (as many rows as requests: it follows from the step's shape, as a
    captured graph's launches must)."""
    return ctx.n_tokens == ctx.n_seqs


def ring_keep(ring: StateSlice, places: int, src: torch.Tensor, ctx) -> None:
    """The last `places` rows of each request in the step go to its history: position p to place p % places of `ring` (places x
    [width] floats); src float32 [n, width] (columns of wider rows are fine). Rows behind the step's tokens are left out. It
    runs after every kernel of the step that reads the ring."""
    ld = _rows(src, "src")
    n, width = src.shape
    if src.dtype != torch.float32 or ctx.n_tokens != n or places < 1 or ring.size != places * width:
        raise KernelError(f"ring_keep: the step's float32 rows of {width} and a ring of {places} places of them are needed")
    _step_lists(ctx, n)
    _i32(ctx.context_lens, "context_lens", ctx.n_seqs)
    _lib.call("liyab_ring_keep", ring.data_ptr(), ring.stride, places, ring.n_slots, src.data_ptr(), ld, width, ctx.tok_seq.data_ptr(),
              ctx.positions.data_ptr(), ctx.context_lens.data_ptr(), ctx.state_slots.data_ptr(), ctx.seq_starts.data_ptr() + 4 * ctx.n_seqs, n, _stream())


def normed_powers(out: torch.Tensor, z: torch.Tensor, coef: torch.Tensor, eps: float) -> None:
    """out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with N(v) = v / sqrt(mean(v^2) + eps) over a row; z float32 rows [n, ff] (columns
    of wider rows are fine), coef float32 [4] on the device, out contiguous [n, ff] float32 or bfloat16."""
    _dev(out, "out")
    ld = _rows(z, "z")
    n, ff = z.shape
    if z.dtype != torch.float32 or tuple(out.shape) != (n, ff) or not out.is_contiguous():
        raise KernelError("normed_powers: z must be float32 rows and out contiguous of its shape")
    _f32vec(coef, "the powers' weights", 4)
    _lib.call("liyab_normed_powers", out.data_ptr(), dtype_code(out.dtype), z.data_ptr(), ld, n, ff, coef.data_ptr(), float(eps), _stream())


def softcap_(t: torch.Tensor, cap: float) -> torch.Tensor:
    """t <- cap * tanh(t / cap) in place; t contiguous float32."""
    _dev(t, "t")
    if t.dtype != torch.float32 or not t.is_contiguous() or not cap > 0:
        raise KernelError("softcap_: a contiguous float32 tensor and a positive cap are needed")
    _lib.call("liyab_softcap", t.data_ptr(), float(cap), t.numel(), _stream())
    return t


# -- the delta-rule recurrence -------------------------------------------------------------------------------
def delta_takes(head_dim: int) -> bool:
    """Whether the delta-rule kernel takes heads of this size (a quarter of a column's rows in a lane's registers)."""
    return 1 <= head_dim <= 256


DELTA_SINGLE_MAX = 64  # the widest heads the one-kernel form for steps of single tokens takes (csrc/delta_rule.hip)


def delta_segments_from(n: int, n_seqs: int) -> bool:
    """Whether a step of n rows of n_seqs requests walks its delta-rule recurrences in segments side by side: when some request
    may bring SCAN_SEGMENT_FROM rows or more. It follows from the step's rows and requests alone (as the grids do), so that a
    captured graph of such a step holds for every step of its shape; a step of short portions only that walks in segments
    all the same computes the same recurrence in three launches."""
    return n - n_seqs + 1 >= SCAN_SEGMENT_FROM


def _delta_segments(ctx, n: int, n_head: int, head_dim: int):
    """(tokens a segment, the most segments, scratch for the segments' ends, transitions and starts), or (0, 0, None, None, None)."""
    if not delta_segments_from(n, ctx.n_seqs):
        return 0, 0, None, None, None
    most = -(-n // SCAN_SEGMENT) + ctx.n_seqs
    state = ctx.workspace.get("delta_seg_state", (most, n_head, head_dim, head_dim), torch.float32)
    trans = ctx.workspace.get("delta_seg_trans", (most, n_head, head_dim, head_dim), torch.float32)
    start = ctx.workspace.get("delta_seg_start", (most, n_head, head_dim, head_dim), torch.float32)
    return SCAN_SEGMENT, most, state.data_ptr(), trans.data_ptr(), start.data_ptr()


def delta_rule(out: torch.Tensor, proj: torch.Tensor, wraw: torch.Tensor, w0: torch.Tensor, a_bias: torch.Tensor, norm_w: Optional[torch.Tensor],
               eps: float, state: StateSlice, ctx, *, n_head: int, head_dim: int, decay_scale: float, key_eps: float) -> None:
    """The decayed delta rule over each request's rows of the step. proj float32 [n, >= 5 * H * D] = [r | k | v | removal logits |
    gate logits | ...], wraw float32 [n, H * D] the decay's logits before w0; with u = k / sqrt(sum(k^2) + key_eps), w = exp(-decay_scale
    * sigmoid(wraw + w0)), a = sigmoid(removal + a_bias): S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r a head; out [n, H * D]
    (compute dtype) = o / rms(o over the head) * norm_w * sigmoid(gate). `state`: the heads' matrices [H, D, D] of a slot."""
    _dev(out, "out")
    n, HD = out.shape
    H, D = n_head, head_dim
    ld, ldw = _rows(proj, "proj"), _rows(wraw, "wraw")
    if HD != H * D or proj.dtype != torch.float32 or proj.shape[0] != n or proj.shape[1] < 5 * HD or not out.is_contiguous() or ctx.n_tokens != n:
        raise KernelError(f"delta_rule: needs the step's float32 proj [n, >= {5 * H * D}] and a contiguous out [n, {H * D}]")
    if wraw.dtype != torch.float32 or tuple(wraw.shape) != (n, HD):
        raise KernelError(f"delta_rule: the decay's logits must be float32 [{n}, {HD}]")
    for t, what in ((w0, "w0"), (a_bias, "a_bias"), (norm_w, "norm weight")):
        _f32vec(t, what, HD)
    if not delta_takes(D) or state.size != H * D * D:
        raise KernelError(f"delta_rule: heads of {D} with {state.size} floats of state a slot")
    _step_lists(ctx, n)
    p = proj.data_ptr()
    if single_token_step(ctx) and D <= DELTA_SINGLE_MAX:
        # every request brings one token: the three kernels' work in one (the same arithmetic in the same order)
        _lib.call("liyab_delta_single", out.data_ptr(), dtype_code(out.dtype), p, p + 4 * HD, p + 8 * HD, p + 12 * HD, p + 16 * HD, ld,
                  wraw.data_ptr(), ldw, w0.data_ptr(), a_bias.data_ptr(), _ptr(norm_w), float(eps), float(decay_scale), float(key_eps),
                  state.data_ptr(), state.stride, state.n_slots, ctx.seq_starts.data_ptr(), ctx.positions.data_ptr(), ctx.state_slots.data_ptr(),
                  ctx.n_seqs, H, D, _stream())
        return
    ws = ctx.workspace
    prep = ws.get("delta_prep", (n, 3, HD), torch.float32)
    o = ws.get("delta_o", (n, HD), torch.float32)
    _lib.call("liyab_delta_prepare", prep.data_ptr(), p + 4 * HD, wraw.data_ptr(), p + 12 * HD, ld, ldw, w0.data_ptr(), a_bias.data_ptr(),
              float(decay_scale), float(key_eps), n, H, D, _stream())
    _lib.call("liyab_delta_scan", o.data_ptr(), p, p + 4 * HD, p + 8 * HD, ld, prep.data_ptr(), state.data_ptr(), state.stride, state.n_slots,
              ctx.seq_starts.data_ptr(), ctx.positions.data_ptr(), ctx.state_slots.data_ptr(), ctx.n_seqs, H, D, *_delta_segments(ctx, n, H, D),
              _stream())
    _lib.call("liyab_head_norm_gate", out.data_ptr(), dtype_code(out.dtype), o.data_ptr(), p + 16 * HD, ld, _ptr(norm_w), float(eps), n, H, D, _stream())


# -- attention in two maps a head --------------------------------------------------------------------------------
def maps_store(proj: torch.Tensor, q_out: torch.Tensor, k1: torch.Tensor, k2: torch.Tensor, v_cache: torch.Tensor, slots: torch.Tensor,
               conv: Optional[torch.Tensor], ring: Optional[StateSlice], ctx, *, n_head: int, n_kv_head: int, head_dim: int, value_dim: int,
               num_pages: Optional[int] = None, keep_single: bool = False) -> None:
    """From a projection's float32 rows [q | k | v] (a query or key head = [map 1 | map 2]) through a causal convolution over time on
    each channel (conv float32 [taps, C], a tap's channels side by side, or None; rows before the step's portion from `ring`, (taps - 1) x [C] floats) to queries
    q_out [n, 2, H * P] and keys and values in their slots of the pages (k1, k2, v_cache [pages, G, page_size, P]), zeros behind a
    head's own entries."""
    H, G, D, V = n_head, n_kv_head, head_dim, value_dim
    n = proj.shape[0]
    ld = _rows(proj, "proj")
    C = 2 * H * D + 2 * G * D + G * V
    if proj.dtype != torch.float32 or proj.shape[1] != C or ctx.n_tokens != n:
        raise KernelError(f"maps_store: the step's float32 rows of {C} channels are needed, got {tuple(proj.shape)} {proj.dtype}")
    for c in (k1, k2, v_cache):
        _dev(c, "cache")
        if c.dim() != 4 or tuple(c.shape) != tuple(k1.shape) or c.shape[1] != G or not c.is_contiguous() or c.dtype != q_out.dtype:
            raise KernelError("maps_store: the three planes must be contiguous [pages, kv heads, page_size, P] in the queries' dtype")
    P = k1.shape[3]
    _dev(q_out, "q_out")
    if P < max(D, V) or tuple(q_out.shape) != (n, 2, H * P) or not q_out.is_contiguous():
        raise KernelError(f"maps_store: q_out must be contiguous [{n}, 2, {H * P}]")
    taps = 0
    if conv is not None:
        _dev(conv, "conv")
        if conv.dtype != torch.float32 or conv.dim() != 2 or conv.shape[1] != C or not conv.is_contiguous():
            raise KernelError(f"maps_store: the convolution's weights must be contiguous float32 [taps, {C}]")
        taps = conv.shape[0]
        if not 1 <= taps <= SHIFT_MAX_TAPS:
            raise KernelError(f"maps_store: {taps} taps; 1 to {SHIFT_MAX_TAPS} are taken")
    if taps > 1 and (ring is None or ring.size != (taps - 1) * C):
        raise KernelError(f"maps_store: {taps} taps need a ring of {(taps - 1) * C} floats a slot")
    _i32(slots, "slots", n)
    _step_lists(ctx, n)
    _lib.call("liyab_maps_store", proj.data_ptr(), ld, _ptr(conv), taps, ring.data_ptr() if taps > 1 else None, ring.stride if taps > 1 else 0,
              ring.n_slots if taps > 1 else 0, q_out.data_ptr(), k1.data_ptr(), k2.data_ptr(), v_cache.data_ptr(), dtype_code(q_out.dtype),
              slots.data_ptr(), k1.shape[2], _pages(k1, num_pages), ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), ctx.seq_starts.data_ptr(),
              ctx.state_slots.data_ptr(), n, H, G, D, V, P, 1 if keep_single and taps > 1 else 0, _stream())


def maps_join(out: torch.Tensor, a1: torch.Tensor, a2: torch.Tensor, lam: float, eps: float, out_scale: float, *, n_head: int, value_dim: int) -> None:
    """out[t, h] = unit_rms(a1[t, h] - lam * a2[t, h]) * out_scale over a head's first `value_dim` entries; a1, a2 [n, H * P] rows of
    one stride (two maps of one buffer), out contiguous [n, H * value_dim], all of one dtype."""
    _dev(out, "out")
    lda, ldb = _rows(a1, "a1"), _rows(a2, "a2")
    n, H, V = out.shape[0], n_head, value_dim
    if a1.shape != a2.shape or lda != ldb or a1.shape[0] != n or a1.shape[1] % H or a1.dtype != out.dtype or a2.dtype != out.dtype:
        raise KernelError("maps_join: two maps of one shape, stride and dtype are needed")
    P = a1.shape[1] // H
    if P < V or tuple(out.shape) != (n, H * V) or not out.is_contiguous():
        raise KernelError(f"maps_join: out must be contiguous [{n}, {H * V}]")
    _lib.call("liyab_maps_join", out.data_ptr(), a1.data_ptr(), a2.data_ptr(), lda, dtype_code(out.dtype), float(lam), float(eps), float(out_scale),
              n, H, V, P, _stream())


# -- a linear recurrence a channel with real gates; two results joined with constant weights ---------------------
def weighted_sum(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor, wa: float, wb: float) -> None:
    """out = wa * a + wb * b; contiguous float32 tensors of one shape (out may be a or b)."""
    for t, what in ((out, "out"), (a, "a"), (b, "b")):
        _dev(t, what)
        if t.dtype != torch.float32 or not t.is_contiguous() or t.shape != out.shape:
            raise KernelError("weighted_sum: out, a and b must be contiguous float32 of one shape")
    _lib.call("liyab_weighted_sum", out.data_ptr(), a.data_ptr(), b.data_ptr(), float(wa), float(wb), out.numel(), _stream())


def lru_conv(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor], ring_off: int,
             ctx, blocks: int = 1, split: Optional[torch.Tensor] = None) -> None:
    """out[t, c] = bias[c] + sum_j weight[c, j] * x[t - taps + 1 + j, c] over each request's own rows in time; x float32 rows (columns of
    wider rows are fine), out contiguous float32 [n, C], weight float32 [C, taps]; the rows before a request's first row of the step come
    from state[slot, ring_off + (position % (taps - 1)) * C + c], zeros before position 0. `split` (bfloat16 [n, 2 C]): out once more as
    two bfloat16 numbers a value, out = hi + lo, each of the `blocks` equal parts of the channels as [hi | lo]."""
    ldi = _rows(x, "x")
    n, C = x.shape
    _dev(out, "out")
    if x.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (n, C) or not out.is_contiguous() or ctx.n_tokens != n:
        raise KernelError("lru_conv: x must be the step's float32 rows and out contiguous float32 of the same shape")
    _dev(weight, "weight")
    if weight.dtype != torch.float32 or weight.dim() != 2 or weight.shape[0] != C or not weight.is_contiguous():
        raise KernelError(f"lru_conv: the weight must be contiguous float32 [{C}, taps]")
    taps = weight.shape[1]
    if not 1 <= taps <= CONV_MAX_TAPS or blocks < 1 or C % blocks:
        raise KernelError(f"lru_conv: {taps} taps (1 to {CONV_MAX_TAPS}), {C} channels in {blocks} parts")
    _f32vec(bias, "bias", C)
    if split is not None:
        _dev(split, "split")
        if split.dtype != torch.bfloat16 or tuple(split.shape) != (n, 2 * C) or not split.is_contiguous():
            raise KernelError(f"lru_conv: the split rows must be contiguous bfloat16 [{n}, {2 * C}]")
    stride, slots, base = 0, 0, None
    if taps > 1:
        stride = _state(state, "lru_conv")
        if ring_off < 0 or ring_off + (taps - 1) * C > stride:
            raise KernelError("lru_conv: the ring does not lie in the slot")
        slots, base = state.shape[0], state.data_ptr() + 4 * ring_off
    _step_lists(ctx, n)
    _lib.call("liyab_lru_conv", out.data_ptr(), _ptr(split), x.data_ptr(), ldi, weight.data_ptr(), _ptr(bias), taps, base, stride, slots,
              ctx.tok_seq.data_ptr(), ctx.positions.data_ptr(), ctx.seq_starts.data_ptr(), ctx.state_slots.data_ptr(), n, C, int(blocks), _stream())


LRU_STRETCHES_FROM = 48  # the longest portion a step may hold from which its recurrence runs in stretches side by side


def lru_stretches(ctx, n: int) -> bool:
    """Whether a step's recurrence a channel runs in stretches side by side (sixteen waves a request, each a stretch of its rows) rather
    than one wave a request: from the step's rows and requests alone, as its grids, so that a captured graph holds for every step of
    its shape."""
    return n - ctx.n_seqs + 1 >= LRU_STRETCHES_FROM


def lru_scan(out: torch.Tensor, z: torch.Tensor, u: torch.Tensor, y: torch.Tensor, x: torch.Tensor, br: torch.Tensor, bi: torch.Tensor,
             lam: torch.Tensor, rate: float, state: torch.Tensor, taps: int, ctx, blocks: int, out_scale: float = 1.0) -> None:
    """S_t = a_t * S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t along each request's rows of the step, with r = sigmoid(zr + br), i = sigmoid(zi +
    bi), a = exp(-rate * r * softplus(lam)); z float32 rows [n, 2 C], each of the `blocks` parts of the channels as [zr | zi]; u contiguous
    float32 [n, C]. S starts from state[slot, :C] (zero at position 0), which gets the last S; out[t] = out_scale * S_t * gelu_tanh(y_t) in
    out's dtype (y float32 rows, out contiguous [n, C]). The last taps - 1 rows of x (float32 rows) go to the slot's ring behind S,
    position p at place p % (taps - 1). Steps that may hold a long portion walk in stretches (`lru_stretches`)."""
    ldz, ldy, ldx = _rows(z, "z"), _rows(y, "y"), _rows(x, "x")
    n, C = y.shape
    stride = _state(state, "lru_scan")
    _dev(out, "out")
    if y.dtype != torch.float32 or x.dtype != torch.float32 or tuple(x.shape) != (n, C) or tuple(out.shape) != (n, C) or not out.is_contiguous() or ctx.n_tokens != n:
        raise KernelError("lru_scan: y and x must be the step's float32 rows and out contiguous of the same shape")
    if z.dtype != torch.float32 or tuple(z.shape) != (n, 2 * C) or u.dtype != torch.float32 or tuple(u.shape) != (n, C) or not u.is_contiguous():
        raise KernelError(f"lru_scan: z must be float32 rows [{n}, {2 * C}] and u contiguous float32 [{n}, {C}]")
    if blocks < 1 or C % blocks or taps < 1 or stride < taps * C:
        raise KernelError(f"lru_scan: {C} channels in {blocks} parts, {taps} taps, a slot of {stride} floats")
    _f32vec(br, "br", C)
    _f32vec(bi, "bi", C)
    _f32vec(lam, "lam", C)
    _step_lists(ctx, n)
    decay = gated = None
    stretches = lru_stretches(ctx, n)
    if stretches:
        decay = ctx.workspace.get("lru_decay", (n, C), torch.float32)
        gated = ctx.workspace.get("lru_gated", (n, C), torch.float32)
        _lib.call("liyab_lru_coeffs", decay.data_ptr(), gated.data_ptr(), z.data_ptr(), ldz, u.data_ptr(), br.data_ptr(), bi.data_ptr(), lam.data_ptr(),
                  float(rate), n, C, int(blocks), _stream())
    _lib.call("liyab_lru_scan", out.data_ptr(), dtype_code(out.dtype), z.data_ptr(), ldz, u.data_ptr(), _ptr(decay), _ptr(gated), br.data_ptr(), bi.data_ptr(),
              lam.data_ptr(), float(rate), float(out_scale), y.data_ptr(), ldy, state.data_ptr(), stride, state.shape[0], x.data_ptr(), ldx, int(taps),
              ctx.seq_starts.data_ptr(), ctx.positions.data_ptr(), ctx.state_slots.data_ptr(), ctx.n_seqs, C, int(blocks), 1 if stretches else 0, _stream())
