"""Python faces of the HIP kernels: each checks on the host that the operands
match what the kernel and its grid assume (device, dtype, shape, strides) and
then launches on torch's current stream. There is no CPU path and no library
fallback: an operand that is not on the GPU, or a size a kernel does not take,
raises.
"""
from __future__ import annotations

import contextlib
import ctypes
import functools
from typing import Optional

import torch

from . import library

_F32, _BF16 = 0, 1


class KernelError(RuntimeError):
    pass


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _F32
    if t.dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("HIP kernels need tensors on the GPU (there is no CPU path); "
                              f"got a tensor on {t.device}")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    # torch's current stream as a raw handle (the two calls below take a fraction of a
    # microsecond; torch.cuda.current_stream() builds a Stream object and takes ten)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def to_device(values, dtype: torch.dtype, device) -> torch.Tensor:
    """A short list of numbers as a device tensor, through pinned memory and without a wait
    (torch.tensor(..., device=...) copies from pageable memory and blocks the host until the
    stream has come that far, which undoes any step launched ahead)."""
    t = torch.tensor(values, dtype=dtype)
    if torch.device(device).type == "cpu":
        return t
    return t.pin_memory().to(device, non_blocking=True)


def _check(code: int, what: str) -> None:
    if code == 0:
        return
    if code == -1:
        raise KernelError(f"{what}: the kernel refused these sizes or arguments")
    raise KernelError(f"{what}: kernel launch failed (code {code})")


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor")


# ---------------------------------------------------------------------------
def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 [T]."""
    _need_gpu(table, ids)
    _i32(ids, "ids")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [V, H] matrix")
    V, H = table.shape
    T = ids.numel()
    out = torch.empty((T, H), dtype=table.dtype, device=table.device)
    lib = library.load("embedding")
    _check(lib.ptl_embedding(_ptr(out), _ptr(table), _ptr(ids), T, H, V, _dtype_code(table),
                             _stream()), "embedding")
    return out


def stage_step(dst: torch.Tensor, src: torch.Tensor, tokens: Optional[torch.Tensor] = None,
               tok_at: int = 0, n_tok: int = 0) -> None:
    """dst (int32, device) <- src (int32, pinned host memory of the same length), read by a
    kernel over the bus; dst[tok_at : tok_at + n_tok] <- tokens (int32, device) when given."""
    _need_gpu(dst)
    if src.is_cuda or not src.is_pinned():
        raise KernelError("stage_step: the source must be pinned host memory")
    if (dst.dtype != torch.int32 or src.dtype != torch.int32 or dst.numel() != src.numel()
            or not dst.is_contiguous() or not src.is_contiguous()):
        raise KernelError("stage_step: two contiguous int32 buffers of one length")
    if tokens is not None:
        _need_gpu(tokens)
        _i32(tokens, "tokens")
        if not (0 <= tok_at and 0 <= n_tok <= tokens.numel() and tok_at + n_tok <= dst.numel()):
            raise KernelError("stage_step: the tokens do not fit where they are to go")
    lib = library.load("embedding")
    _check(lib.ptl_stage_step(_ptr(dst), ctypes.c_void_p(src.data_ptr()), dst.numel(),
                              _ptr(tokens) if tokens is not None else None, int(tok_at),
                              int(n_tok) if tokens is not None else 0, _stream()), "stage_step")


def add_rmsnorm(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = rmsnorm(x + residual) * weight; ``residual`` (if given) is replaced
    by the sum in place. weight is float32 [H]. Returns y."""
    _need_gpu(x, residual, weight)
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("add_rmsnorm: x must be a contiguous [T, H] matrix")
    T, H = x.shape
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"add_rmsnorm: weight must be float32 [{H}]")
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype
                                 or not residual.is_contiguous()):
        raise KernelError("add_rmsnorm: residual must match x in shape and dtype")
    y = out if out is not None else torch.empty_like(x)
    lib = library.load("norm")
    _check(lib.ptl_add_rmsnorm(_ptr(y), _ptr(x), _ptr(residual), _ptr(weight), T, H,
                               ctypes.c_float(eps), _dtype_code(x), _stream()), "add_rmsnorm")
    return y


def rmsnorm_cols(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """rmsnorm(x) * weight for x [T, H] whose rows may be strided (a range of columns of a fused
    projection); the result is contiguous, in x's dtype. weight is float32 [H]."""
    _need_gpu(x, weight)
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("rmsnorm_cols: x must be a [T, H] matrix with dense rows")
    T, H = x.shape
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"rmsnorm_cols: weight must be float32 [{H}]")
    y = torch.empty((T, H), dtype=x.dtype, device=x.device)
    _check(library.load("norm").ptl_rmsnorm_cols(_ptr(y), ctypes.c_long(H), _ptr(x),
                                                 ctypes.c_long(x.stride(0) if T > 1 else H), _ptr(weight), T, H,
                                                 ctypes.c_float(eps), _dtype_code(x), _stream()), "rmsnorm_cols")
    return y


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """out[:, i] = silu(gate_up[:, i]) * gate_up[:, I + i] for a [T, 2I] input."""
    _need_gpu(gate_up)
    if gate_up.dim() != 2 or not gate_up.is_contiguous() or gate_up.shape[1] % 2:
        raise KernelError("silu_mul: input must be a contiguous [T, 2I] matrix")
    T, I2 = gate_up.shape
    out = torch.empty((T, I2 // 2), dtype=gate_up.dtype, device=gate_up.device)
    lib = library.load("activation")
    _check(lib.ptl_silu_mul(_ptr(out), _ptr(gate_up), T, I2 // 2, _dtype_code(gate_up), _stream()),
           "silu_mul")
    return out


def rope_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
               inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
               k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
               page_size: int = 1, k_in_place: bool = False) -> None:
    """Rotate q in place (and k, when ``k_in_place``) by the angles
    positions * inv_freq and write the rotated k and v into the caches
    [num_pages, Hkv, page_size, D] at ``slots`` (int32, page*page_size+offset).
    q, k, v are [T, heads, D] views that share one row stride (slices of one
    projection output). inv_freq None: no rotation. slots None: no store."""
    _need_gpu(q, k, v, positions, inv_freq, slots, k_cache, v_cache)
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    if k.shape != (T, Hkv, D) or v.shape != (T, Hkv, D):
        raise KernelError("rope_store: k and v must be [T, Hkv, D]")
    rs = q.stride(0)
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.stride(2) != 1 or (t.shape[1] > 1 and t.stride(1) != D) or (T > 1 and t.stride(0) != rs) \
                or t.dtype != q.dtype:
            raise KernelError(f"rope_store: {name} must be a [T, heads, D] view with dense heads "
                              "and the common row stride")
    _i32(positions, "positions")
    if positions.numel() != T:
        raise KernelError("rope_store: one position per token")
    if D % 2:
        raise KernelError(f"rope_store: head size {D} must be even")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != D // 2
                                 or not inv_freq.is_contiguous()):
        raise KernelError(f"rope_store: inv_freq must be float32 [{D // 2}]")
    if slots is not None:
        if slots.dtype != torch.int32 or slots.numel() != T or not slots.is_contiguous():
            raise KernelError("rope_store: slots must be contiguous int32 [T]")
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c is None or c.dim() != 4 or c.shape[1:] != (Hkv, page_size, D) \
                    or c.dtype != q.dtype or not c.is_contiguous():
                raise KernelError(f"rope_store: {name} must be contiguous "
                                  f"[pages, {Hkv}, {page_size}, {D}] of {q.dtype}")
    lib = library.load("rope")
    _check(lib.ptl_rope_store(_ptr(q), _ptr(k), _ptr(v), ctypes.c_long(rs), _ptr(positions),
                              _ptr(inv_freq), _ptr(slots), _ptr(k_cache), _ptr(v_cache),
                              T, Hq, Hkv, D, page_size, int(k_in_place), _dtype_code(q),
                              _stream()), "rope_store")


def gemm_nt(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w.T with float32 accumulation through the vector-FMA kernel.
    x [M, K] (rows may be strided), w [N, K] contiguous, same dtype."""
    _need_gpu(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"gemm_nt: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    if x.dtype != w.dtype:
        raise KernelError(f"gemm_nt: x is {x.dtype} but w is {w.dtype}")
    if x.stride(1) != 1 or not w.is_contiguous():
        raise KernelError("gemm_nt: x rows and w must be dense")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32 and out_dtype != torch.float32:
        raise KernelError("gemm_nt: float32 inputs give float32 outputs")
    y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return y
    lib = library.load("gemm")
    _check(lib.ptl_gemm_nt(_ptr(y), _ptr(x), _ptr(w), M, N, K, ctypes.c_long(x.stride(0)),
                           ctypes.c_long(y.stride(0)), _dtype_code(x),
                           _F32 if out_dtype == torch.float32 else _BF16, _stream()), "gemm_nt")
    return y


SKINNY_MAX_ROWS = 64
BLOCKED_MAX_ROWS = 64      # rows of x up to which the kernels take the blocked copy of a weight


def blocked_weight(w: torch.Tensor) -> Optional[torch.Tensor]:
    """A second copy of the bfloat16 matrix w [N, K] for the decode kernels: tiles of 16 rows x
    32 columns, each tile row-major in 1 KB, the tiles of a row block one after the other along
    K (shape [ceil(N / 16), K / 32, 16, 32]; rows beyond N are zero). A wave's load instruction
    then reads 1 KB in one piece instead of 16 pieces of 64 bytes that lie a row apart (see
    gs_row_ptr in csrc/gemm.hip). None when w cannot be cut so (K no multiple of 32)."""
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] % 32 or not w.is_contiguous():
        return None
    N, K = w.shape
    rows = -(-N // 16) * 16
    if rows != N:
        w = torch.cat([w, w.new_zeros((rows - N, K))], dim=0)
    return w.view(rows // 16, 16, K // 32, 32).permute(0, 2, 1, 3).contiguous()


def _weight_arg(w: torch.Tensor, blocked: Optional[torch.Tensor], M: int, what: str):
    """(pointer, flag) of the weight a decode kernel is to read: the blocked copy when one is
    given and the rows of x are few enough, else w."""
    if blocked is None or M > BLOCKED_MAX_ROWS:
        return _ptr(w), 0
    N, K = w.shape
    if (blocked.dtype != torch.bfloat16 or not blocked.is_cuda or not blocked.is_contiguous()
            or tuple(blocked.shape) != (-(-N // 16), K // 32, 16, 32) or K % 32
            or blocked.data_ptr() % 16):
        raise KernelError(f"{what}: the blocked copy does not belong to a [{N}, {K}] bfloat16 matrix")
    return _ptr(blocked), 1


def gemm_skinny_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming matrix-core kernel takes this product."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and 0 < x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(1) == 1
            and (x.shape[0] == 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0)


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w.T for at most 64 rows of bfloat16 x, streaming w once
    (see csrc/gemm.hip). Output bfloat16 or float32. ``blocked``: ``blocked_weight(w)``, read
    instead of w when x has at most 16 rows."""
    _need_gpu(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"gemm_skinny: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    if not gemm_skinny_fits(x, w):
        raise KernelError("gemm_skinny: needs bfloat16, at most 64 rows, K a multiple of 8 and "
                          "16-byte aligned rows")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("gemm_skinny: output is bfloat16 or float32")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    ldx = x.stride(0) if M > 1 else max(K, 8)
    lib = library.load("gemm")
    wp, wb = _weight_arg(w, blocked, M, "gemm_skinny")
    _check(lib.ptl_gemm_skinny_bf16(_ptr(y), _ptr(x), wp, wb, M, N, K, ctypes.c_long(ldx),
                                    ctypes.c_long(N), _F32 if out_dtype == torch.float32 else _BF16,
                                    _stream()), "gemm_skinny")
    return y


def gemm_library_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_library`` takes x [M, K] and w [N, K]: bfloat16, dense rows of w,
    16-byte aligned rows of both."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2
            and x.shape[1] == w.shape[1] and x.stride(1) == 1 and w.is_contiguous()
            and x.shape[1] % 8 == 0 and (x.shape[0] == 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


_timed_products = False        # inside ``timed_library_products``


def gemm_library(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                 checked: bool = False) -> torch.Tensor:
    """y = x @ w.T by hipBLASLt, called directly with the descriptors and the algorithm of
    the shape kept from its first call (see csrc/blaslt.hip). Output bfloat16 or float32.
    ``checked``: the caller has just asked ``gemm_library_fits``. The library's first proposal
    runs, except inside ``timed_library_products``."""
    _need_gpu(x, w)
    if not checked and not gemm_library_fits(x, w):
        raise KernelError("gemm_library: needs bfloat16 x [M, K] and w [N, K] with K a multiple of 8 "
                          "and 16-byte aligned rows")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("gemm_library: output is bfloat16 or float32")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    ldx = x.stride(0) if M > 1 else max(K, 8)
    lib = library.load("blaslt")
    _check(lib.ptl_blaslt_gemm_bf16(_ptr(y), _ptr(x), _ptr(w), M, N, K, ctypes.c_long(ldx),
                                    ctypes.c_long(N), _F32 if out_dtype == torch.float32 else _BF16,
                                    1 if _timed_products else 0, _stream()), "gemm_library")
    return y


@contextlib.contextmanager
def timed_library_products(on: bool = True):
    """Inside, ``gemm_library`` runs the proposal of the library that a timing of the shape
    kept: the first such call of a shape times the library's proposals on its own operands
    (it waits for the stream; not while the stream is captured) and keeps the fastest whose
    result agrees with the first proposal's (csrc/blaslt.hip). For the warm-up pass and the
    recording of a step that is replayed as a graph: such shapes come back with every replay.
    Outside, every call runs the library's first proposal, whatever was timed. ``on=False``:
    no effect (for callers that pass a switch on)."""
    global _timed_products
    before = _timed_products
    _timed_products = bool(on) or before
    try:
        yield
    finally:
        _timed_products = before


def library_product_choice(M: int, N: int, K: int, ldx: int, out_dtype: torch.dtype = torch.bfloat16) -> int:
    """The proposal kept for a shape by its timing (0 = the library's first), -1 if the shape
    has not been timed."""
    lib = library.load("blaslt")
    return int(lib.ptl_blaslt_timed_choice(int(M), int(N), int(K), ctypes.c_long(int(ldx)), ctypes.c_long(int(N)),
                                           _F32 if out_dtype == torch.float32 else _BF16))


FUSED_MAX_ROWS = 16


class RowScale:
    """The normalisation factor that rows of a tensor still lack: row m is to be multiplied by
    rsqrt(sum(partials[m]) / size + eps). ``partials`` [M, count] float32 are the sums of squares
    of the un-normalised row over column blocks (written by ``gemm_skinny_add_norm``)."""
    __slots__ = ("partials", "size", "eps")

    def __init__(self, partials: torch.Tensor, size: int, eps: float):
        self.partials, self.size, self.eps = partials, int(size), float(eps)

    def args(self, M: int, K: int, what: str):
        p = self.partials
        if (p.dtype != torch.float32 or p.dim() != 2 or p.shape[0] != M or not p.is_contiguous()
                or not p.is_cuda):
            raise KernelError(f"{what}: partial sums must be contiguous float32 [{M}, count] on the GPU")
        if self.size != K:
            raise KernelError(f"{what}: rows of {K} elements, but the partial sums are of rows of "
                              f"{self.size}")
        return _ptr(p), int(p.shape[1]), ctypes.c_float(self.eps)


_NO_SCALE = (ctypes.c_void_p(0), 0, ctypes.c_float(0.0))


def gemm_skinny_add_norm_fits(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                              norm_weight: torch.Tensor) -> bool:
    return (_fused_x_ok(x, w) and residual.dtype == torch.bfloat16 and residual.is_cuda
            and residual.dim() == 2 and residual.shape == (x.shape[0], w.shape[0])
            and residual.stride(1) == 1 and norm_weight.dtype == torch.float32
            and norm_weight.is_cuda and norm_weight.is_contiguous()
            and norm_weight.numel() == w.shape[0])


def gemm_skinny_add_norm(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                         norm_weight: torch.Tensor, eps: float, blocked: Optional[torch.Tensor] = None):
    """The product x @ w.T, the residual sum and the part of an RMSNorm that does not need the
    whole row, in one kernel for at most 16 rows of bfloat16 x (see AddNormArgs in
    csrc/gemm.hip): ``residual`` becomes x @ w.T + residual in place; returned are
    y = bfloat16(residual * norm_weight) and the RowScale that y still lacks."""
    if not gemm_skinny_add_norm_fits(x, w, residual, norm_weight):
        raise KernelError("gemm_skinny_add_norm: needs bfloat16 x, w, residual [M, N] with M <= 16, "
                          "K a multiple of 8, aligned rows, a float32 norm weight [N]")
    M, K = x.shape
    N = w.shape[0]
    lib = library.load("gemm")
    count = int(lib.ptl_gemm_skinny_partials(N))
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    partials = torch.empty((M, count), dtype=torch.float32, device=x.device)
    wp, wb = _weight_arg(w, blocked, M, "gemm_skinny_add_norm")
    _check(lib.ptl_gemm_skinny_add_norm_bf16(
        _ptr(y), _ptr(x), wp, wb, _ptr(residual), _ptr(norm_weight), _ptr(partials), M, N, K,
        ctypes.c_long(x.stride(0) if M > 1 else max(K, 8)), ctypes.c_long(N),
        ctypes.c_long(residual.stride(0) if M > 1 else N), _stream()), "gemm_skinny_add_norm")
    return y, RowScale(partials, N, eps)


def row_scale(v: torch.Tensor, scale: RowScale) -> torch.Tensor:
    """v with the factor of ``scale`` applied to its rows (bfloat16 [M, H])."""
    _need_gpu(v)
    if v.dtype != torch.bfloat16 or v.dim() != 2 or not v.is_contiguous():
        raise KernelError("row_scale: needs a contiguous bfloat16 [M, H] tensor")
    M, H = v.shape
    pp, count, eps = scale.args(M, H, "row_scale")
    y = torch.empty_like(v)
    lib = library.load("norm")
    _check(lib.ptl_row_scale_bf16(_ptr(y), _ptr(v), pp, count, M, H, eps, _stream()), "row_scale")
    return y


def _fused_x_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and 0 < x.shape[0] <= FUSED_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(1) == 1
            and (x.shape[0] == 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0 and w.shape[1] == x.shape[1])


# Rows from which, and up to which, the products of csrc/gemm_rows.hip take a decode step (they
# work up to 128). Measured on MI355X at the 1B widths against the library's product followed by
# the separate kernel (cold weights, microseconds at 32 / 64 / 128 rows): output projection + norm
# 9.8 / 11.2 / 14.8 against 11.9 / 12.5 / 12.2; down projection + norm 15.8 / 17.2 / 21.7 against
# 19.5 / 25.9 / 25.1; gate-up + SiLU-multiply 19.5 / 22.7 / 31.2 against 21.5 / 22.3 / 25.5; q|k|v +
# rotation + cache write 10.0 / 13.7 / 18.5 against 13.7 / 14.1 / 17.1; the head of 128,256 columns
# 101 / 112 / 206 against 131 / 137 / 150. Against the fused kernels for at most 16 rows, whole
# decode steps of 16 rows: 1.287 -> 1.243 ms at the 1B widths, 4.73 -> 4.58 ms at the 8B widths,
# 3.04 -> 3.07 ms at the 3B widths (product by product the faster one depends on the shape): from
# 9 rows on a step takes these kernels, where they fit.
ROWS_MIN = 9
ROWS_MAX = {"plain": 64, "add_norm": 64, "gate_up": 64, "qkv": 64}


def _rows_x_ok(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor], use: str = "") -> bool:
    """Whether the kernels for some tens of rows take x with this weight (they read the blocked
    copy) and, with ``use``, whether they are the faster way for that many rows."""
    return (blocked is not None and x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and x.dim() == 2 and ROWS_MIN <= x.shape[0] <= ROWS_MAX.get(use, 128) and x.shape[1] % 32 == 0
            and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.dim() == 2 and w.shape[1] == x.shape[1])


def _rows_weight(w: torch.Tensor, blocked: torch.Tensor, what: str):
    N, K = w.shape
    if (blocked.dtype != torch.bfloat16 or not blocked.is_cuda or not blocked.is_contiguous()
            or tuple(blocked.shape) != (-(-N // 16), K // 32, 16, 32) or blocked.data_ptr() % 16):
        raise KernelError(f"{what}: the blocked copy does not belong to a [{N}, {K}] bfloat16 matrix")
    return _ptr(blocked)


def gemm_rows_fits(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor]) -> bool:
    """Whether ``gemm_rows`` takes the product and is the faster way for it: without slices of K
    it gives every compute unit a workgroup only if the matrix has 64 rows for each (a head)."""
    return _rows_x_ok(x, w, blocked, "plain") and w.shape[0] >= 64 * compute_units(x.device)


def gemm_rows(x: torch.Tensor, w: torch.Tensor, blocked: torch.Tensor,
              out_dtype: Optional[torch.dtype] = None, splits: int = 1) -> torch.Tensor:
    """y = x @ w.T for 9 to 128 rows of bfloat16 x, streaming the blocked copy of w once (see
    csrc/gemm_rows.hip). Output bfloat16 or float32 [M, N]; with ``splits`` > 1 the float32
    partial sums [splits, M, N] over that many slices of K (for ``sum_add_rmsnorm``)."""
    if not _rows_x_ok(x, w, blocked):
        raise KernelError("gemm_rows: needs 9 to 128 rows of bfloat16 x with aligned rows, K a multiple "
                          "of 32 and the blocked copy of w")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype not in (torch.bfloat16, torch.float32) or (splits > 1 and out_dtype != torch.float32):
        raise KernelError("gemm_rows: output is bfloat16 or float32, partial sums are float32")
    y = torch.empty((splits, M, N) if splits > 1 else (M, N), dtype=out_dtype, device=x.device)
    lib = library.load("gemm_rows")
    _check(lib.ptl_rows_gemm_bf16(_ptr(y), _ptr(x), _rows_weight(w, blocked, "gemm_rows"), M, N, K,
                                  ctypes.c_long(x.stride(0)), ctypes.c_long(N),
                                  _F32 if out_dtype == torch.float32 else _BF16, int(splits),
                                  _stream()), "gemm_rows")
    return y


def gemm_rows_splits(M: int, N: int, K: int) -> int:
    """The slices of K that ``gemm_rows`` should leave partial sums of when a norm follows."""
    return int(library.load("gemm_rows").ptl_rows_gemm_splits(int(M), int(N), int(K)))


def sum_add_rmsnorm(partials: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                    eps: float) -> torch.Tensor:
    """y = rmsnorm(bfloat16(sum of partials) + residual) * weight for float32 partial sums
    [splits, M, N] (or a float32 product [M, N]); ``residual`` (bfloat16 [M, N]) becomes the sum
    in place. One kernel (csrc/gemm_rows.hip)."""
    _need_gpu(partials, residual, weight)
    if partials.dim() == 2:
        partials = partials.unsqueeze(0)
    S, M, N = partials.shape
    if (partials.dtype != torch.float32 or not partials.is_contiguous() or residual.dtype != torch.bfloat16
            or residual.shape != (M, N) or not residual.is_contiguous() or weight.dtype != torch.float32
            or weight.shape != (N,) or not weight.is_contiguous() or N % 8 or N > 8192):
        raise KernelError("sum_add_rmsnorm: needs contiguous float32 partial sums [S, M, N], a bfloat16 "
                          "residual [M, N], a float32 weight [N], N a multiple of 8 up to 8192")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=partials.device)
    lib = library.load("gemm_rows")
    _check(lib.ptl_rows_sum_add_rmsnorm(_ptr(y), _ptr(partials), S, _ptr(residual), _ptr(weight), M, N,
                                        ctypes.c_float(eps), _stream()), "sum_add_rmsnorm")
    return y


def gemm_rows_add_rmsnorm_fits(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor],
                               residual: torch.Tensor, norm_weight: torch.Tensor) -> bool:
    N = w.shape[0]
    return (_rows_x_ok(x, w, blocked, "add_norm") and residual.dtype == torch.bfloat16 and residual.is_cuda
            and residual.shape == (x.shape[0], N) and residual.is_contiguous()
            and norm_weight.dtype == torch.float32 and norm_weight.is_cuda and norm_weight.is_contiguous()
            and norm_weight.numel() == N and N % 8 == 0 and N <= 8192)


def gemm_rows_add_rmsnorm(x: torch.Tensor, w: torch.Tensor, blocked: torch.Tensor, residual: torch.Tensor,
                          norm_weight: torch.Tensor, eps: float) -> torch.Tensor:
    """rmsnorm(x @ w.T + residual) * norm_weight for 9 to 128 rows, ``residual`` replaced by the
    sum: the product as float32 partial sums over slices of K (so that a matrix with few rows
    still gives every compute unit a workgroup), then one kernel that adds them up and
    normalises whole rows."""
    M, K = x.shape
    partials = gemm_rows(x, w, blocked, torch.float32, splits=gemm_rows_splits(M, w.shape[0], K))
    return sum_add_rmsnorm(partials, residual, norm_weight, eps)


def gate_up_silu_fits(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor] = None) -> bool:
    """Whether ``gate_up_silu`` is the way to go for x. ``blocked``: the blocked copy of w, which
    the kernel for some tens of rows reads."""
    if _rows_x_ok(x, w, blocked, "gate_up") and w.shape[0] % 64 == 0:
        return True
    return _fused_x_ok(x, w) and w.shape[0] % 32 == 0


def gate_up_silu(x: torch.Tensor, w: torch.Tensor, scale: Optional[RowScale] = None,
                 blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) for w = [Wg; Wu] ([2I, K]) in one kernel: for at most 16 rows
    of bfloat16 x the one of csrc/gemm.hip, from ROWS_MIN rows on, with the blocked copy of w,
    the one of csrc/gemm_rows.hip. ``scale``: the factor that the rows of x still lack (at most
    16 rows); it is applied to both products."""
    rows = scale is None and _rows_x_ok(x, w, blocked) and w.shape[0] % 64 == 0
    if not (rows or (_fused_x_ok(x, w) and w.shape[0] % 32 == 0)):
        raise KernelError("gate_up_silu: needs bfloat16, K a multiple of 8, I a multiple of 16, aligned "
                          "rows, at most 16 of them (up to 128 with the blocked copy of w, K and I "
                          "multiples of 32)")
    M, K = x.shape
    I = w.shape[0] // 2
    out = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
    if rows:
        _check(library.load("gemm_rows").ptl_rows_gate_up_silu(
            _ptr(out), _ptr(x), _rows_weight(w, blocked, "gate_up_silu"), M, I, K,
            ctypes.c_long(x.stride(0)), _stream()), "gate_up_silu")
        return out
    lib = library.load("gemm")
    pp, count, eps = scale.args(M, K, "gate_up_silu") if scale is not None else _NO_SCALE
    wp, wb = _weight_arg(w, blocked, M, "gate_up_silu")
    _check(lib.ptl_gate_up_silu_bf16(_ptr(out), _ptr(x), wp, wb, M, I, K,
                                     ctypes.c_long(x.stride(0) if M > 1 else max(K, 8)),
                                     pp, count, eps, _stream()),
           "gate_up_silu")
    return out


def qkv_rope_store_fits(x: torch.Tensor, w: torch.Tensor, head_dim: int,
                        blocked: Optional[torch.Tensor] = None) -> bool:
    """Whether ``qkv_rope_store`` is the way to go for x. ``blocked``: the blocked copy of w, which
    the kernel for some tens of rows reads."""
    return (_fused_x_ok(x, w) or _rows_x_ok(x, w, blocked, "qkv")) and head_dim % 32 == 0


def qkv_rope_store(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor,
                   inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                   scale: Optional[RowScale] = None, blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q, k, v = x @ w.T (rows of w: q | k | v), q and k rotated, k and v written
    into the cache pages at ``slots``; returns the rotated q [M, Hq, D]. At most 16
    rows of bfloat16 x (see csrc/gemm.hip), or, with the blocked copy of w, ROWS_MIN to 128
    (csrc/gemm_rows.hip); head sizes in steps of 32. ``scale``: the factor that the rows of x
    still lack (at most 16 rows); it is applied to the products."""
    rows = scale is None and _rows_x_ok(x, w, blocked)
    if not ((rows or _fused_x_ok(x, w)) and head_dim % 32 == 0):
        raise KernelError("qkv_rope_store: needs bfloat16, K a multiple of 8, a head size in steps of "
                          "32, aligned rows, at most 16 of them (up to 128 with the blocked copy of w "
                          "and K a multiple of 32)")
    M, K = x.shape
    Hq, Hkv, D = num_heads, num_kv_heads, head_dim
    if w.shape[0] != (Hq + 2 * Hkv) * D:
        raise KernelError(f"qkv_rope_store: weight has {w.shape[0]} rows, "
                          f"({Hq} + 2*{Hkv}) * {D} expected")
    _need_gpu(positions, inv_freq, slots, k_cache, v_cache)
    _i32(positions, "positions")
    if positions.numel() != M:
        raise KernelError("qkv_rope_store: one position per row of x")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != D // 2
                                 or not inv_freq.is_contiguous()):
        raise KernelError(f"qkv_rope_store: inv_freq must be float32 [{D // 2}]")
    if slots is not None:
        if slots.dtype != torch.int32 or slots.numel() != M or not slots.is_contiguous():
            raise KernelError("qkv_rope_store: slots must be contiguous int32 [M]")
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c is None or c.dim() != 4 or c.shape[1:] != (Hkv, page_size, D) \
                    or c.dtype != torch.bfloat16 or not c.is_contiguous():
                raise KernelError(f"qkv_rope_store: {name} must be contiguous bfloat16 "
                                  f"[pages, {Hkv}, {page_size}, {D}]")
    q = torch.empty((M, Hq, D), dtype=torch.bfloat16, device=x.device)
    if rows:
        # the projection as float32 partial sums over slices of K (few rows of W: so that every
        # compute unit gets a workgroup), then one kernel that adds them up, rotates and stores
        partials = gemm_rows(x, w, blocked, torch.float32, splits=gemm_rows_splits(M, w.shape[0], K))
        _check(library.load("gemm_rows").ptl_rows_sum_rope_store(
            _ptr(q), ctypes.c_long(Hq * D), _ptr(partials), partials.shape[0] if partials.dim() == 3 else 1, M,
            _ptr(positions), _ptr(inv_freq), _ptr(slots), _ptr(k_cache), _ptr(v_cache), Hq, Hkv, D,
            int(page_size), _stream()), "qkv_rope_store")
        return q
    lib = library.load("gemm")
    pp, count, eps = scale.args(M, K, "qkv_rope_store") if scale is not None else _NO_SCALE
    wp, wb = _weight_arg(w, blocked, M, "qkv_rope_store")
    _check(lib.ptl_qkv_rope_store_bf16(
        _ptr(q), ctypes.c_long(Hq * D), _ptr(x), wp, wb, M, K,
        ctypes.c_long(x.stride(0) if M > 1 else max(K, 8)), _ptr(positions), _ptr(inv_freq),
        _ptr(slots), _ptr(k_cache), _ptr(v_cache), Hq, Hkv, D, int(page_size), pp, count, eps,
        _stream()),
        "qkv_rope_store")
    return q


def _mask_extras(what: str, Hq: int, window: int, keep_first: int, sink: Optional[torch.Tensor]):
    """The two optional pieces every attention kernel takes: ``keep_first`` (with a window: the
    keys at positions below it stay visible to every later query) and ``sink`` (float32 [Hq]: the
    softmax denominator of head h also holds exp(sink[h]), a term without key and value)."""
    if keep_first < 0 or (keep_first and window <= 0):
        raise KernelError(f"{what}: keep_first goes with a window, and is not negative")
    if sink is not None and (not sink.is_cuda or sink.dtype != torch.float32 or sink.shape != (Hq,)
                             or not sink.is_contiguous()):
        raise KernelError(f"{what}: sink must be a contiguous float32 GPU tensor [{Hq}]")
    return int(keep_first), _ptr(sink)


def attention_generic(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                      block_table: torch.Tensor, work_seq: torch.Tensor, work_qoff: torch.Tensor,
                      scale: float, window: int = 0, keep_first: int = 0,
                      sink: Optional[torch.Tensor] = None) -> None:
    """Attention of a mixed batch over the paged cache (see csrc/attention.hip).
    q [T, Hq, D] (rows may be strided), out [T, Hq, D], caches
    [pages, Hkv, page_size, D], q_start [n+1], ctx_len [n], block_table [n, max_pages],
    work_seq / work_qoff: the list of 16-row query blocks. ``keep_first``, ``sink``: see
    _mask_extras."""
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table, work_seq, work_qoff)
    T, Hq, D = q.shape
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.shape[3] != D:
        raise KernelError("attention: caches must be [pages, Hkv, page_size, D]")
    Hkv, page_size = k_cache.shape[1], k_cache.shape[2]
    if D > 640:
        raise KernelError(f"attention: head size {D} exceeds the kernel's limit of 640")
    if Hq % Hkv:
        raise KernelError(f"attention: {Hq} query heads are not a multiple of {Hkv} kv heads")
    if q.stride(2) != 1 or out.stride(2) != 1 or (Hq > 1 and (q.stride(1) != D or out.stride(1) != D)):
        raise KernelError("attention: q and out need dense heads")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention: q, out and the caches must share one dtype")
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous")
    for name, t in (("q_start", q_start), ("ctx_len", ctx_len), ("work_seq", work_seq),
                    ("work_qoff", work_qoff)):
        _i32(t, name)
    n = ctx_len.numel()
    if q_start.numel() != n + 1 or work_seq.numel() != work_qoff.numel():
        raise KernelError("attention: inconsistent sequence tables")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] < n \
            or block_table.stride(1) != 1:
        raise KernelError("attention: block_table must be int32 [n, max_pages]")
    keep, sk = _mask_extras("attention", Hq, window, keep_first, sink)
    lib = library.load("attention")
    _check(lib.ptl_attention_generic(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
        _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
        int(block_table.stride(0)), _ptr(work_seq), _ptr(work_qoff), int(work_seq.numel()),
        Hq, Hkv, D, page_size, int(window), keep, sk, ctypes.c_float(scale), _dtype_code(q), _stream()),
        "attention")


def _attention_common(out, q, k_cache, v_cache, q_start, ctx_len, block_table, what):
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table)
    T, Hq, D = q.shape
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.shape[3] != D:
        raise KernelError(f"{what}: caches must be [pages, Hkv, page_size, D]")
    Hkv, page_size = k_cache.shape[1], k_cache.shape[2]
    if Hq % Hkv:
        raise KernelError(f"{what}: {Hq} query heads are not a multiple of {Hkv} kv heads")
    if q.stride(2) != 1 or out.stride(2) != 1 or (Hq > 1 and (q.stride(1) != D or out.stride(1) != D)):
        raise KernelError(f"{what}: q and out need dense heads")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError(f"{what}: q, out and the caches must share one dtype")
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError(f"{what}: caches must be contiguous")
    _i32(q_start, "q_start")
    _i32(ctx_len, "ctx_len")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError(f"{what}: block_table must be int32 [n, max_pages]")
    return T, Hq, Hkv, D, page_size


def attention_decode_mfma_fits(dtype, Hq: int, Hkv: int, D: int, page_size: int = 16) -> bool:
    """Whether the matrix-core decode kernel takes this case: bfloat16, head size 32, 64, 96
    or 128, at most 16 heads a kv head, a page size that is a power of two, pages (of all kv
    heads) below 4 GiB."""
    return (dtype == torch.bfloat16 and D % 32 == 0 and 0 < D <= 128 and Hq // Hkv <= 16
            and page_size > 0 and page_size & (page_size - 1) == 0
            and Hkv * page_size * D * 2 < 2 ** 32)


def attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                     block_table: torch.Tensor, n_seq: int, scale: float, window: int = 0,
                     num_splits: int = 1, matrix_cores: bool = False, unroll: int = 0,
                     keep_first: int = 0, sink: Optional[torch.Tensor] = None) -> None:
    """Split-KV attention of the first ``n_seq`` sequences of the tables, each of
    which brings exactly one query token (see csrc/attention.hip). Head sizes in
    steps of 16 up to 256, float32 or bfloat16. ``matrix_cores``: the MFMA
    variant (bfloat16, head sizes 32/64/96/128, at most 16 heads a kv head, a page
    size that is a power of two); ``unroll``: its 16-key tiles per wave and turn
    (1 or 2; 0 leaves the choice to the kernel)."""
    T, Hq, Hkv, D, page_size = _attention_common(out, q, k_cache, v_cache, q_start, ctx_len,
                                                 block_table, "attention_decode")
    if D % 16 or D > 256:
        raise KernelError(f"attention_decode: head size {D} is not a multiple of 16 up to 256")
    if n_seq > ctx_len.numel() or q_start.numel() < n_seq + 1 or block_table.shape[0] < n_seq:
        raise KernelError("attention_decode: tables are shorter than n_seq")
    if num_splits < 1:
        raise KernelError("attention_decode: num_splits must be >= 1")
    keep, sk = _mask_extras("attention_decode", Hq, window, keep_first, sink)
    part_acc = part_ml = None
    if num_splits > 1:
        part_acc = torch.empty((n_seq, Hq, num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_seq, Hq, num_splits, 2), dtype=torch.float32, device=q.device)
    lib = library.load("attention")
    if matrix_cores:
        if (not attention_decode_mfma_fits(q.dtype, Hq, Hkv, D, page_size) or q.stride(0) % 8
                or q.data_ptr() % 16):
            raise KernelError("attention_decode: the matrix-core variant needs bfloat16, a head "
                              "size of 32/64/96/128, at most 16 heads a kv head, a page size that "
                              "is a power of two, aligned q rows")
        _check(lib.ptl_attention_decode_mfma(
            _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
            _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
            int(block_table.stride(0)), _ptr(part_acc), _ptr(part_ml), int(n_seq), Hq, Hkv, D,
            page_size, int(window), keep, sk, ctypes.c_float(scale), int(num_splits), int(unroll),
            _stream()), "attention_decode_mfma")
        return
    _check(lib.ptl_attention_decode(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
        _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
        int(block_table.stride(0)), _ptr(part_acc), _ptr(part_ml), int(n_seq), Hq, Hkv, D, page_size,
        int(window), keep, sk, ctypes.c_float(scale), int(num_splits), _dtype_code(q), _stream()),
        "attention_decode")


def attention_prefill_mfma_fits(dtype: torch.dtype, num_kv_heads: int, head_dim: int,
                                page_size: int) -> bool:
    """Whether ``attention_prefill_mfma`` takes this case: bfloat16, head size 32, 64, 96 or
    128, a page size that is a power of two, pages (of all kv heads) below 4 GiB."""
    return (dtype == torch.bfloat16 and head_dim % 32 == 0 and 0 < head_dim <= 128
            and page_size > 0 and page_size & (page_size - 1) == 0
            and num_kv_heads * page_size * head_dim * 2 < 2 ** 32)


@functools.lru_cache(maxsize=None)
def _compute_units(device_index: int) -> int:
    return int(torch.cuda.get_device_properties(device_index).multi_processor_count)


def compute_units(device) -> int:
    """Compute units of the GPU ``device`` (256 on MI355X)."""
    device = torch.device(device)
    return _compute_units(device.index if device.index is not None else torch.cuda.current_device())


def attention_prefill_mfma_plan(device: torch.device, num_heads: int, head_dim: int,
                                blocks_of_64: int, blocks_of_128: int, max_keys: int = 0):
    """(block_rows, groups) for ``attention_prefill_mfma``, from sweeps on MI355X (one sequence
    of 512 to 16,384 tokens, and 2,048-token portions behind prefixes up to 14,336, head sizes
    64 and 128). With t = the workgroups a head can have resident at once (three a compute unit
    up to head size 64, two above): 128-row blocks (keys and values are staged half as often)
    once there are 1.25 t of them, 64-row blocks before; at head sizes above 64 also from 0.5 t
    on when some sequence has 4,096 keys or more (``max_keys``: the longest context of the
    step, or a bound of it): a portion behind a long prefix has few blocks, all of them long
    (at 32 heads of 128, 2,048 rows on 14,336 keys: 578 against 811 us; with no prefix the two
    are level, at head size 64 they are level throughout). A workgroup for every block while
    there are at most 2 t blocks (the longest start first and the short ones fill in behind
    them), beyond that t workgroups that share the sorted list as a snake, which evens out the
    causal triangle."""
    resident = compute_units(device) * (3 if head_dim <= 64 else 2)
    t = max(1, resident // num_heads)
    wide = 4 * blocks_of_128 >= 5 * t or (head_dim > 64 and max_keys >= 4096 and 2 * blocks_of_128 >= t)
    rows, blocks = (128, blocks_of_128) if wide else (64, blocks_of_64)
    return rows, max(1, blocks if blocks <= 2 * t else t)


def attention_prefill_mfma(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                           block_table: torch.Tensor, work_seq: torch.Tensor,
                           work_qoff: torch.Tensor, scale: float, window: int = 0,
                           block_rows: int = 64, groups: int = 0, keep_first: int = 0,
                           sink: Optional[torch.Tensor] = None) -> None:
    """bfloat16 attention of prompt portions on the matrix cores; the work list
    names query blocks of ``block_rows`` (64 or 128) rows, those with the most
    keys first. ``groups`` workgroups a head share the list (0: one for every
    block). Head sizes 32, 64, 96, 128."""
    T, Hq, Hkv, D, page_size = _attention_common(out, q, k_cache, v_cache, q_start, ctx_len,
                                                 block_table, "attention_prefill_mfma")
    if q.dtype != torch.bfloat16:
        raise KernelError("attention_prefill_mfma: bfloat16 only")
    if D % 32 or D > 128:
        raise KernelError(f"attention_prefill_mfma: head size {D} is not 32, 64, 96 or 128")
    if not attention_prefill_mfma_fits(q.dtype, Hkv, D, page_size):
        raise KernelError(f"attention_prefill_mfma: page size {page_size} is not a power of two "
                          "(or a page of all kv heads reaches 4 GiB)")
    _need_gpu(work_seq, work_qoff)
    _i32(work_seq, "work_seq")
    _i32(work_qoff, "work_qoff")
    if work_seq.numel() != work_qoff.numel():
        raise KernelError("attention_prefill_mfma: inconsistent work list")
    if block_rows not in (64, 128):
        raise KernelError("attention_prefill_mfma: query blocks are 64 or 128 rows")
    if q.stride(0) % 8 or out.stride(0) % 4 or q.data_ptr() % 16 or out.data_ptr() % 8:
        raise KernelError("attention_prefill_mfma: q rows must be 16-byte aligned, out rows 8-byte")
    keep, sk = _mask_extras("attention_prefill_mfma", Hq, window, keep_first, sink)
    lib = library.load("attention_prefill")
    n_work = int(work_seq.numel())
    _check(lib.ptl_attention_prefill_mfma(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
        _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
        int(block_table.stride(0)), _ptr(work_seq), _ptr(work_qoff), n_work,
        min(n_work, int(groups)) if groups > 0 else n_work, int(block_rows), Hq, Hkv, D, page_size,
        int(window), keep, sk, ctypes.c_float(scale), _stream()), "attention_prefill_mfma")


def argmax(logits: torch.Tensor, host_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy token per row of float32 logits [R, V]; ties go to the lowest id. ``host_out``:
    pinned int32 host memory (at least R long) that the kernel fills as well, over the bus;
    it holds the choices once the kernel has ended (an event after it, say)."""
    _need_gpu(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be float32 [R, V] with dense rows")
    R, V = logits.shape
    if host_out is not None and (host_out.is_cuda or not host_out.is_pinned() or host_out.dtype != torch.int32
                                 or not host_out.is_contiguous() or host_out.numel() < R):
        raise KernelError("argmax: host_out must be pinned int32 host memory with a place for every row")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    chunks = -(-V // 4096)
    ws_val = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
    ws_idx = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    lib = library.load("sampling")
    _check(lib.ptl_argmax(_ptr(out), _ptr(logits), R, V, ctypes.c_long(logits.stride(0)),
                          _ptr(ws_val), _ptr(ws_idx), _ptr(host_out), _stream()), "argmax")
    return out


SAMPLE_WIDE_FROM = 16384      # rows at least this long are sampled by many workgroups a row
SAMPLE_WIDE_UP_TO = 64 * 4096


def sample_top_p(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
                 uniform: torch.Tensor, return_probs: bool = False, wide: Optional[bool] = None):
    """One token per row from the nucleus of softmax(logits / temperature).
    temperature, top_p, uniform: float32 [R] on the GPU. ``wide``: spread a row over
    many workgroups (several kernels; None: for rows of vocabulary size) or keep it
    in one (one kernel); both follow the same rule."""
    _need_gpu(logits, temperature, top_p, uniform)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample_top_p: logits must be float32 [R, V] with dense rows")
    R, V = logits.shape
    for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        if t.dtype != torch.float32 or t.numel() != R or not t.is_contiguous():
            raise KernelError(f"sample_top_p: {name} must be float32 [{R}]")
    if wide is None:
        wide = SAMPLE_WIDE_FROM <= V <= SAMPLE_WIDE_UP_TO
    elif wide and V > SAMPLE_WIDE_UP_TO:
        raise KernelError(f"sample_top_p: the many-workgroup form takes rows up to {SAMPLE_WIDE_UP_TO}")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    probs = torch.empty((R, V), dtype=torch.float32, device=logits.device)   # scratch, then result
    lib = library.load("sampling")
    if wide:
        lib.ptl_sample_top_p_wide_workspace.restype = ctypes.c_size_t
        nbytes = int(lib.ptl_sample_top_p_wide_workspace(R, V))
        ws = torch.empty((nbytes // 4,), dtype=torch.float32, device=logits.device)
        _check(lib.ptl_sample_top_p_wide(_ptr(out), _ptr(probs), int(return_probs), _ptr(logits), R, V,
                                         ctypes.c_long(logits.stride(0)), _ptr(temperature),
                                         _ptr(top_p), _ptr(uniform), _ptr(ws), _stream()),
               "sample_top_p")
    else:
        _check(lib.ptl_sample_top_p(_ptr(out), _ptr(probs), int(return_probs), _ptr(logits), R, V,
                                    ctypes.c_long(logits.stride(0)), _ptr(temperature), _ptr(top_p),
                                    _ptr(uniform), _stream()), "sample_top_p")
    return (out, probs) if return_probs else out


def token_logprob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """log_softmax(logits[r])[tokens[r]] for float32 logits [R, V] and int32 tokens [R]."""
    _need_gpu(logits, tokens)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("token_logprob: logits must be float32 [R, V] with dense rows")
    _i32(tokens, "tokens")
    R, V = logits.shape
    if tokens.numel() != R:
        raise KernelError("token_logprob: one token per row")
    out = torch.empty((R,), dtype=torch.float32, device=logits.device)
    lib = library.load("sampling")
    _check(lib.ptl_token_logprob(_ptr(out), _ptr(logits), _ptr(tokens), R, V,
                                 ctypes.c_long(logits.stride(0)), _stream()), "token_logprob")
    return out


def probe_stream_read(buf: torch.Tensor, blocks: int = 512) -> None:
    """Launch the kernel that only reads ``buf`` (see csrc/probe.hip); time it from outside."""
    _need_gpu(buf)
    if not buf.is_contiguous() or buf.data_ptr() % 16:
        raise KernelError("probe_stream_read: a contiguous, 16-byte aligned tensor")
    sink = torch.empty(blocks * 256, dtype=torch.int32, device=buf.device)
    lib = library.load("probe")
    _check(lib.ptl_probe_stream_read(_ptr(buf), ctypes.c_size_t(buf.numel() * buf.element_size()),
                                     int(blocks), _ptr(sink), _stream()), "probe_stream_read")


PROBE_MFMA_FLOPS_PER_ITER = 4 * 8 * 16 * 16 * 32 * 2      # per workgroup of four waves


def probe_mfma(iters: int, blocks: int, device="cuda") -> None:
    """Launch ``blocks`` workgroups of four waves that each issue ``iters`` * 8 independent
    bfloat16 MFMAs (see csrc/probe.hip): blocks * iters * PROBE_MFMA_FLOPS_PER_ITER operations."""
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    lib = library.load("probe")
    _check(lib.ptl_probe_mfma(_ptr(out), int(iters), int(blocks), _stream()), "probe_mfma")


# ---------------------------------------------------------------------------
# The float32 residual stream and its norms (csrc/stream.hip)
def _norm_args(norm):
    """(weight, bias, alpha) of a Dynamic-Tanh norm as kernel arguments; ``norm``: a tuple
    (weight float32 [H], bias float32 [H] or None, alpha) or None."""
    if norm is None:
        return ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_float(0.0)
    w, b, alpha = norm
    return _ptr(w), _ptr(b), ctypes.c_float(alpha)


def _check_norm(norm, H: int, what: str) -> None:
    if norm is None:
        return
    w, b, _ = norm
    _need_gpu(w, b)
    for t in (w, b):
        if t is not None and (t.dtype != torch.float32 or t.shape != (H,) or not t.is_contiguous()):
            raise KernelError(f"{what}: norm weight and bias must be float32 [{H}]")


def _check_stream(stream: torch.Tensor, what: str):
    _need_gpu(stream)
    if stream.dim() != 2 or stream.dtype != torch.float32 or not stream.is_contiguous():
        raise KernelError(f"{what}: the residual stream must be a contiguous float32 [T, H] matrix")
    return stream.shape


def embedding_scaled(table: torch.Tensor, ids: torch.Tensor, scale: float, copies: int = 1) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as float32 (the start of a float32 residual stream),
    ``copies`` times side by side in a row (a model that keeps several streams a token)."""
    _need_gpu(table, ids)
    _i32(ids, "ids")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [V, H] matrix")
    V, H = table.shape
    T = ids.numel()
    if copies < 1:
        raise KernelError("embedding_scaled: at least one copy")
    out = torch.empty((T, copies * H), dtype=torch.float32, device=table.device)
    _check(library.load("stream").ptl_embedding_scaled(_ptr(out), _ptr(table), _ptr(ids), T, H, V,
                                                       ctypes.c_float(scale), int(copies), _dtype_code(table),
                                                       _stream()), "embedding_scaled")
    return out


def embedding_rmsnorm(table: torch.Tensor, ids: torch.Tensor, weight: torch.Tensor, eps: float,
                      scale: float = 1.0) -> torch.Tensor:
    """out[t] = rmsnorm(table[ids[t]] * scale) * weight as float32: a float32 residual stream
    that starts from the normed embedding."""
    _need_gpu(table, ids, weight)
    _i32(ids, "ids")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [V, H] matrix")
    V, H = table.shape
    _f32_vec(weight, H, "embedding_rmsnorm: weight")
    T = ids.numel()
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _check(library.load("stream").ptl_embedding_rmsnorm(_ptr(out), _ptr(table), _ptr(ids), _ptr(weight),
                                                        ctypes.c_float(eps), T, H, V, ctypes.c_float(scale),
                                                        _dtype_code(table), _stream()), "embedding_rmsnorm")
    return out


HYPER_MAX_STREAMS = 16


def hyper_mix(streams: torch.Tensor, num_streams: int, y: Optional[torch.Tensor] = None, mix=None, outc=None,
              inc=None, norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
              out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """Several residual streams a token, ``streams`` float32 [T, S * H] (stream after stream in a
    row). With ``y`` [T, H]: x_t <- sum_s mix[s, t] x_s + outc[t] y for all t at once, in place. With
    ``norm_weight`` [H]: returns rmsnorm(sum_s inc[s] x_s) * norm_weight in ``out_dtype``, read from
    the streams as the update left them. Coefficients are float32 device tensors; None stands for
    the identity (mix), ones (outc, inc)."""
    S = int(num_streams)
    T, SH = _check_stream(streams, "hyper_mix")
    if not 1 <= S <= HYPER_MAX_STREAMS or SH % S:
        raise KernelError(f"hyper_mix: {S} streams do not divide a row of {SH} (at most {HYPER_MAX_STREAMS})")
    H = SH // S
    if y is None and norm_weight is None:
        raise KernelError("hyper_mix: nothing to do")
    if y is not None:
        _need_gpu(y)
        if y.shape != (T, H) or not y.is_contiguous():
            raise KernelError(f"hyper_mix: y must be a contiguous [{T}, {H}] matrix")
    for c, n, what in ((mix, S * S, "mix"), (outc, S, "outc"), (inc, S, "inc"), (norm_weight, H, "norm_weight")):
        if c is not None:
            _f32_vec(c, n, f"hyper_mix: {what}")
    out = None
    if norm_weight is not None:
        out = torch.empty((T, H), dtype=out_dtype or torch.float32, device=streams.device)
    _check(library.load("stream").ptl_hyper_mix(
        _ptr(streams), _ptr(y), _dtype_code(y) if y is not None else _F32, _ptr(mix), _ptr(outc), _ptr(inc),
        _ptr(norm_weight), ctypes.c_float(eps), _ptr(out), _dtype_code(out) if out is not None else _F32,
        T, S, H, _stream()), "hyper_mix")
    return out


def dyt(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], alpha: float,
        out_dtype: torch.dtype) -> torch.Tensor:
    """tanh(alpha x) * weight + bias for rows x [T, H] of float32 or bfloat16."""
    _need_gpu(x)
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("dyt: x must be a contiguous [T, H] matrix")
    T, H = x.shape
    _check_norm((weight, bias, alpha), H, "dyt")
    out = torch.empty((T, H), dtype=out_dtype, device=x.device)
    _check(library.load("stream").ptl_dyt(_ptr(out), _dtype_code(out), _ptr(x), _dtype_code(x), _ptr(weight),
                                          _ptr(bias), ctypes.c_float(alpha), T, H, _stream()), "dyt")
    return out


def stream_add_dyt(stream: torch.Tensor, y: Optional[torch.Tensor], post=None, pre=None,
                   out_dtype: Optional[torch.dtype] = None, want_copy: bool = False):
    """stream += post(y) (plain sum when ``post`` is None, nothing when ``y`` is None), in place;
    returns (pre(stream) in ``out_dtype`` or None, a copy of the new stream in ``out_dtype`` or
    None). ``post`` / ``pre``: (weight, bias, alpha) of Dynamic-Tanh norms."""
    T, H = _check_stream(stream, "stream_add_dyt")
    if y is not None:
        _need_gpu(y)
        if y.shape != stream.shape or not y.is_contiguous():
            raise KernelError("stream_add_dyt: y must be a contiguous matrix of the stream's shape")
    _check_norm(post, H, "stream_add_dyt")
    _check_norm(pre, H, "stream_add_dyt")
    out_dtype = out_dtype or torch.float32
    out = torch.empty((T, H), dtype=out_dtype, device=stream.device) if pre is not None else None
    copy = torch.empty((T, H), dtype=out_dtype, device=stream.device) if want_copy else None
    pw, pb, pa = _norm_args(post)
    qw, qb, qa = _norm_args(pre)
    code = _F32 if out_dtype == torch.float32 else _BF16
    _check(library.load("stream").ptl_stream_add_dyt(
        _ptr(stream), _ptr(y), _dtype_code(y) if y is not None else _F32, pw, pb, pa, _ptr(out), code,
        qw, qb, qa, _ptr(copy), T, H, _stream()), "stream_add_dyt")
    return out, copy


def stream_add_rmsnorm(stream: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, pre=None,
                       out_dtype: Optional[torch.dtype] = None, want_copy: bool = False):
    """stream += y * rsqrt(mean(y^2) + eps) * weight, in place; returns (pre(stream) or None, a
    copy of the new stream or None) as stream_add_dyt does."""
    T, H = _check_stream(stream, "stream_add_rmsnorm")
    _need_gpu(y, weight)
    if y.shape != stream.shape or not y.is_contiguous():
        raise KernelError("stream_add_rmsnorm: y must be a contiguous matrix of the stream's shape")
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"stream_add_rmsnorm: weight must be float32 [{H}]")
    _check_norm(pre, H, "stream_add_rmsnorm")
    out_dtype = out_dtype or torch.float32
    out = torch.empty((T, H), dtype=out_dtype, device=stream.device) if pre is not None else None
    copy = torch.empty((T, H), dtype=out_dtype, device=stream.device) if want_copy else None
    qw, qb, qa = _norm_args(pre)
    code = _F32 if out_dtype == torch.float32 else _BF16
    _check(library.load("stream").ptl_stream_add_rmsnorm(
        _ptr(stream), _ptr(y), _dtype_code(y), _ptr(weight), ctypes.c_float(eps), _ptr(out), code, qw, qb, qa,
        _ptr(copy), T, H, _stream()), "stream_add_rmsnorm")
    return out, copy


def gelu_gather_mul(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col0: int) -> torch.Tensor:
    """out[t, j] = gelu_tanh(z[t, j]) * table[ids[t], col0 + j] for z [T, n]."""
    _need_gpu(z, table, ids)
    _i32(ids, "ids")
    if z.dim() != 2 or not z.is_contiguous() or table.dim() != 2 or not table.is_contiguous() \
            or table.dtype != z.dtype:
        raise KernelError("gelu_gather_mul: z [T, n] and table [V, ld] must be contiguous and of one dtype")
    T, n = z.shape
    V, ld = table.shape
    if ids.numel() != T or col0 < 0 or col0 + n > ld:
        raise KernelError("gelu_gather_mul: one id per row, and the columns must lie inside the table")
    out = torch.empty_like(z)
    _check(library.load("stream").ptl_gelu_gather_mul(_ptr(out), _ptr(z), _ptr(table), _ptr(ids), T, n, ld,
                                                      int(col0), V, _dtype_code(z), _stream()),
           "gelu_gather_mul")
    return out


# ---------------------------------------------------------------------------
# Latent attention (csrc/latent.hip)
def latent_prepare(q_out: torch.Tensor, proj: torch.Tensor, q_off: int, kv_off: int,
                   positions: torch.Tensor, inv_freq: Optional[torch.Tensor], c_weight: Optional[torch.Tensor],
                   eps: float, slots: Optional[torch.Tensor], cache: Optional[torch.Tensor],
                   H: int, dn: int, dr: int, R: int, queries: Optional[torch.Tensor] = None,
                   half_layout: bool = False, mag: float = 1.0) -> None:
    """From the projections ``proj`` [T, >= q_off + H (dn + dr)] of a step: the rotated query
    parts into q_out[:, :, R:] (q_out [T, H, R + dr]), and, when the layer has a down-projection
    (``kv_off`` >= 0: its R + dr columns start there) and ``slots`` are given, the normalised
    latent and the rotated shared key part into ``cache`` [pages, 1, page_size, R + dr] at the
    tokens' slots. inv_freq float32 [pairs], 2 * pairs <= dr: the entries that rotate, as
    neighbouring pairs or, with ``half_layout``, entry i with entry i + pairs; sine and cosine
    times ``mag``. ``queries``: the matrix [T, >= q_off + H (dn + dr)] that holds the queries when
    they are not columns of ``proj``."""
    _need_gpu(q_out, proj, positions, inv_freq, c_weight, slots, cache, queries)
    T = proj.shape[0]
    D = R + dr
    qsrc = proj if queries is None else queries
    if proj.dim() != 2 or proj.stride(1) != 1 or q_out.shape != (T, H, D) or not q_out.is_contiguous() \
            or q_out.dtype != proj.dtype:
        raise KernelError("latent_prepare: proj [T, n] with dense rows, q_out contiguous [T, H, R + dr]")
    if qsrc.dim() != 2 or qsrc.stride(1) != 1 or qsrc.shape[0] != T or qsrc.dtype != proj.dtype:
        raise KernelError("latent_prepare: queries [T, n] with dense rows, of the projections' dtype")
    if q_off < 0 or q_off + H * (dn + dr) > qsrc.shape[1] or (kv_off >= 0 and kv_off + D > proj.shape[1]):
        raise KernelError("latent_prepare: the columns named lie outside the projections")
    _i32(positions, "positions")
    if positions.numel() != T or dr % 2:
        raise KernelError("latent_prepare: one position per token, an even rotated size")
    pairs = 0
    if inv_freq is not None:
        pairs = inv_freq.numel()
        if inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous() or 2 * pairs > dr:
            raise KernelError("latent_prepare: inv_freq must be float32 with at most dr / 2 entries")
    if kv_off >= 0 and slots is not None:
        _i32(slots, "slots")
        if slots.numel() != T:
            raise KernelError("latent_prepare: one slot per token")
        if cache is None or cache.dim() != 4 or cache.shape[1] != 1 or cache.shape[3] != D \
                or cache.dtype != proj.dtype or not cache.is_contiguous():
            raise KernelError(f"latent_prepare: cache must be contiguous [pages, 1, page_size, {D}]")
        if c_weight is None or c_weight.dtype != torch.float32 or c_weight.shape != (R,) \
                or not c_weight.is_contiguous():
            raise KernelError(f"latent_prepare: the latent's norm weight must be float32 [{R}]")
    _check(library.load("latent").ptl_latent_prepare(
        _ptr(q_out), ctypes.c_long(H * D), _ptr(qsrc), ctypes.c_long(qsrc.stride(0)), int(q_off),
        _ptr(proj), ctypes.c_long(proj.stride(0)), int(kv_off),
        _ptr(positions), _ptr(inv_freq), int(pairs), int(bool(half_layout)), ctypes.c_float(mag),
        _ptr(c_weight), ctypes.c_float(eps), _ptr(slots),
        _ptr(cache), T, H, dn, dr, R, _dtype_code(proj), _stream()), "latent_prepare")


def gemm_heads_nt(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor,
                  gate: Optional[torch.Tensor] = None) -> None:
    """out[t, h, :] = x[t, h, :] @ w[h].T for views out [T, H, N], x [T, H, K] (dense last
    dimension, any row and head strides) and w [H, N, K] contiguous; ``gate`` [T, H] (a view
    with stride 1 over the heads): the result of head h of row t times sigmoid(gate[t, h])."""
    _need_gpu(out, x, w, gate)
    if x.dim() != 3 or out.dim() != 3 or w.dim() != 3 or not w.is_contiguous():
        raise KernelError("gemm_heads_nt: x [T, H, K], out [T, H, N], w contiguous [H, N, K]")
    T, H, K = x.shape
    N = w.shape[1]
    if w.shape != (H, N, K) or out.shape != (T, H, N) or x.stride(2) != 1 or out.stride(2) != 1:
        raise KernelError("gemm_heads_nt: shapes do not match, or a last dimension is not dense")
    if not (x.dtype == out.dtype == w.dtype):
        raise KernelError("gemm_heads_nt: one dtype")
    ldg = 0
    if gate is not None:
        if gate.shape != (T, H) or gate.dtype != x.dtype or (H > 1 and gate.stride(1) != 1):
            raise KernelError("gemm_heads_nt: gate must be [T, H] with dense rows")
        ldg = gate.stride(0)
    _check(library.load("latent").ptl_gemm_heads_nt(
        _ptr(out), ctypes.c_long(out.stride(0)), ctypes.c_long(out.stride(1)), _ptr(x),
        ctypes.c_long(x.stride(0)), ctypes.c_long(x.stride(1)), _ptr(w), T, H, N, K, _ptr(gate),
        ctypes.c_long(ldg), _dtype_code(x), _stream()), "gemm_heads_nt")


# ---------------------------------------------------------------------------
# Attention with keys and values of different sizes and several score maps a head
def attention_generic_kv(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                         q_start: torch.Tensor, ctx_len: torch.Tensor, block_table: torch.Tensor,
                         work_seq: torch.Tensor, work_qoff: torch.Tensor, scale: float, maps: int = 1,
                         window: int = 0, keep_first: int = 0, sink: Optional[torch.Tensor] = None) -> None:
    """The vector-FMA attention kernel in its general form (csrc/attention.hip): q [T, Hq, Dk]
    with Hq = heads * maps (head after head, map after map), k_cache [pages, Hkv * maps, page_size,
    Dk], v_cache [pages, Hkv, page_size, Dv], out [T, Hq, Dv] in the caches' dtype or float32.
    Query head j reads key head (its kv head) * maps + j % maps and the values of its kv head."""
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table, work_seq, work_qoff)
    if q.dim() != 3 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError("attention: q [T, Hq, Dk], caches [pages, heads, page_size, size]")
    T, Hq, Dk = q.shape
    pages, Hk, page_size, _ = k_cache.shape
    Hkv, Dv = v_cache.shape[1], v_cache.shape[3]
    if (k_cache.shape[3] != Dk or v_cache.shape[0] != pages or v_cache.shape[2] != page_size
            or maps <= 0 or Hk != Hkv * maps or Hq % maps or (Hq // maps) % Hkv):
        raise KernelError(f"attention: q {tuple(q.shape)}, keys {tuple(k_cache.shape)} and values "
                          f"{tuple(v_cache.shape)} do not fit each other with {maps} maps a head")
    if out.shape != (T, Hq, Dv) or not out.is_contiguous() or not q.is_contiguous():
        raise KernelError(f"attention: q and out [{T}, {Hq}, {Dv}] must be contiguous")
    if max(Dk, Dv) > 640:
        raise KernelError(f"attention: head sizes {Dk}, {Dv} exceed the kernel's limit of 640")
    if not (q.dtype == k_cache.dtype == v_cache.dtype) or out.dtype not in (q.dtype, torch.float32):
        raise KernelError("attention: q and the caches must share one dtype; out has it, or float32")
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous")
    for name, t in (("q_start", q_start), ("ctx_len", ctx_len), ("work_seq", work_seq),
                    ("work_qoff", work_qoff)):
        _i32(t, name)
    n = ctx_len.numel()
    if q_start.numel() != n + 1 or work_seq.numel() != work_qoff.numel():
        raise KernelError("attention: inconsistent sequence tables")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] < n \
            or block_table.stride(1) != 1:
        raise KernelError("attention: block_table must be int32 [n, max_pages]")
    keep, sk = _mask_extras("attention", Hq, window, keep_first, sink)
    _check(library.load("attention").ptl_attention_generic_kv(
        _ptr(out), ctypes.c_long(out.stride(0)), int(out.dtype == torch.float32 and q.dtype != torch.float32),
        _ptr(q), ctypes.c_long(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len),
        _ptr(block_table), int(block_table.stride(0)), _ptr(work_seq), _ptr(work_qoff),
        int(work_seq.numel()), Hq, Hkv, int(maps), Dk, Dv, page_size, int(window), keep, sk,
        ctypes.c_float(scale), _dtype_code(q), _stream()), "attention")


def attention_prefill_mfma_kv_fits(dtype: torch.dtype, num_kv_heads: int, maps: int, Dk: int, Dv: int,
                                   page_size: int) -> bool:
    """Whether the matrix-core kernel for prompt portions takes keys of size Dk with values of
    size Dv: bfloat16, both multiples of 32 up to 128, a page size that is a power of two, pages
    (of all heads) below 4 GiB."""
    return (dtype == torch.bfloat16 and Dk % 32 == 0 and Dv % 32 == 0 and 0 < Dk <= 128 and 0 < Dv <= 128
            and page_size > 0 and page_size & (page_size - 1) == 0
            and num_kv_heads * maps * page_size * Dk * 2 < 2 ** 32 and num_kv_heads * page_size * Dv * 2 < 2 ** 32)


def attention_prefill_mfma_kv(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                              q_start: torch.Tensor, ctx_len: torch.Tensor, block_table: torch.Tensor,
                              work_seq: torch.Tensor, work_qoff: torch.Tensor, scale: float, maps: int = 1,
                              groups: int = 1, window: int = 0, keep_first: int = 0,
                              sink: Optional[torch.Tensor] = None) -> None:
    """The matrix-core kernel for prompt portions in its general form (csrc/attention_prefill.hip):
    shapes as for attention_generic_kv, bfloat16 q and caches, out bfloat16 or float32; the work
    list names 64-row blocks, ``groups`` workgroups a head share it."""
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table, work_seq, work_qoff)
    if q.dim() != 3 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError("attention_prefill_mfma_kv: q [T, Hq, Dk], caches [pages, heads, page_size, size]")
    T, Hq, Dk = q.shape
    pages, Hk, page_size, _ = k_cache.shape
    Hkv, Dv = v_cache.shape[1], v_cache.shape[3]
    if (k_cache.shape[3] != Dk or v_cache.shape[0] != pages or v_cache.shape[2] != page_size
            or maps <= 0 or Hk != Hkv * maps or Hq % maps or (Hq // maps) % Hkv):
        raise KernelError("attention_prefill_mfma_kv: q, keys and values do not fit each other")
    if not attention_prefill_mfma_kv_fits(q.dtype, Hkv, maps, Dk, Dv, page_size):
        raise KernelError("attention_prefill_mfma_kv: bfloat16, sizes that are multiples of 32 up to 128, a "
                          "page size that is a power of two")
    if (out.shape != (T, Hq, Dv) or not out.is_contiguous() or not q.is_contiguous() or q.data_ptr() % 16
            or out.data_ptr() % 16 or out.dtype not in (torch.bfloat16, torch.float32)):
        raise KernelError(f"attention_prefill_mfma_kv: q and out [{T}, {Hq}, {Dv}] must be contiguous and aligned")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention_prefill_mfma_kv: contiguous bfloat16 caches")
    for name, t in (("q_start", q_start), ("ctx_len", ctx_len), ("work_seq", work_seq), ("work_qoff", work_qoff)):
        _i32(t, name)
    n = ctx_len.numel()
    if q_start.numel() != n + 1 or work_seq.numel() != work_qoff.numel():
        raise KernelError("attention_prefill_mfma_kv: inconsistent sequence tables")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] < n \
            or block_table.stride(1) != 1:
        raise KernelError("attention_prefill_mfma_kv: block_table must be int32 [n, max_pages]")
    n_work = int(work_seq.numel())
    if n_work == 0:
        return
    keep, sk = _mask_extras("attention_prefill_mfma_kv", Hq, window, keep_first, sink)
    _check(library.load("attention_prefill").ptl_attention_prefill_mfma_kv(
        _ptr(out), ctypes.c_long(out.stride(0)), int(out.dtype == torch.float32), _ptr(q),
        ctypes.c_long(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len),
        _ptr(block_table), int(block_table.stride(0)), _ptr(work_seq), _ptr(work_qoff), n_work,
        max(1, min(int(groups), n_work)), Hq, Hkv, int(maps), Dk, Dv, page_size, int(window), keep, sk,
        ctypes.c_float(scale), _stream()), "attention_prefill_mfma_kv")


def attention_decode_kv_fits(Dk: int, Dv: int) -> bool:
    """Whether the split-KV kernel takes keys of size Dk with values of size Dv."""
    return Dk % 16 == 0 and Dv % 16 == 0 and 0 < Dk <= 256 and 0 < Dv <= 256


def attention_decode_kv(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                        q_start: torch.Tensor, ctx_len: torch.Tensor, block_table: torch.Tensor, n_seq: int,
                        scale: float, maps: int = 1, num_splits: int = 1, window: int = 0,
                        keep_first: int = 0, sink: Optional[torch.Tensor] = None) -> None:
    """Split-KV attention of the first ``n_seq`` sequences of the tables, each of which brings one
    query token, with keys and values of different sizes and ``maps`` score maps a head (shapes as
    for attention_generic_kv; sizes in steps of 16 up to 256)."""
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table)
    if q.dim() != 3 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError("attention_decode_kv: q [T, Hq, Dk], caches [pages, heads, page_size, size]")
    T, Hq, Dk = q.shape
    pages, Hk, page_size, _ = k_cache.shape
    Hkv, Dv = v_cache.shape[1], v_cache.shape[3]
    if (k_cache.shape[3] != Dk or v_cache.shape[0] != pages or v_cache.shape[2] != page_size
            or maps <= 0 or Hk != Hkv * maps or Hq % maps or (Hq // maps) % Hkv):
        raise KernelError("attention_decode_kv: q, keys and values do not fit each other")
    if not attention_decode_kv_fits(Dk, Dv):
        raise KernelError(f"attention_decode_kv: sizes {Dk}, {Dv} are not multiples of 16 up to 256")
    if out.shape != (T, Hq, Dv) or not out.is_contiguous() or not q.is_contiguous() or q.data_ptr() % 16:
        raise KernelError(f"attention_decode_kv: q and out [{T}, {Hq}, {Dv}] must be contiguous and aligned")
    if not (q.dtype == k_cache.dtype == v_cache.dtype) or out.dtype not in (q.dtype, torch.float32):
        raise KernelError("attention_decode_kv: q and the caches share one dtype; out has it, or float32")
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention_decode_kv: caches must be contiguous")
    _i32(q_start, "q_start")
    _i32(ctx_len, "ctx_len")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attention_decode_kv: block_table must be int32 [n, max_pages]")
    if n_seq > ctx_len.numel() or q_start.numel() < n_seq + 1 or block_table.shape[0] < n_seq or num_splits < 1:
        raise KernelError("attention_decode_kv: tables are shorter than n_seq, or no splits")
    keep, sk = _mask_extras("attention_decode_kv", Hq, window, keep_first, sink)
    part_acc = part_ml = None
    if num_splits > 1:
        part_acc = torch.empty((n_seq, Hq, num_splits, Dv), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_seq, Hq, num_splits, 2), dtype=torch.float32, device=q.device)
    _check(library.load("attention").ptl_attention_decode_kv(
        _ptr(out), ctypes.c_long(out.stride(0)), int(out.dtype == torch.float32 and q.dtype != torch.float32),
        _ptr(q), ctypes.c_long(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len),
        _ptr(block_table), int(block_table.stride(0)), _ptr(part_acc), _ptr(part_ml), int(n_seq), Hq, Hkv,
        int(maps), Dk, Dv, page_size, int(window), keep, sk, ctypes.c_float(scale), int(num_splits),
        _dtype_code(q), _stream()), "attention_decode_kv")


# ---------------------------------------------------------------------------
# Normed queries and keys, results normed head by head (csrc/prepare.hip)
NORM_NONE, NORM_HEAD, NORM_WHOLE = 0, 1, 2
GATE_NONE, GATE_SIGMOID, GATE_SILU = 0, 1, 2


def _f32_vec(t: Optional[torch.Tensor], n: int, what: str) -> None:
    if t is not None and (not t.is_cuda or t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous float32 GPU tensor of {n} numbers")


def _f32_rows(p: torch.Tensor, what: str) -> None:
    if not p.is_cuda or p.dim() != 2 or p.dtype != torch.float32 or p.stride(1) != 1:
        raise KernelError(f"{what} must be a float32 [T, columns] GPU matrix with dense rows")


def qkv_prepare(q_out: torch.Tensor, p: torch.Tensor, q_off: int, k_off: int, v_off: int,
                q_bias, k_bias, v_bias, norm_mode: int, q_weight, k_weight, eps: float,
                rot_dims: int, inv_freq, mag: float, positions: torch.Tensor, slots, k_cache, v_cache,
                Hq: int, Hk: int, Hv: int, Dk: int, Dv: int, page_size: int) -> None:
    """Bias, norm of queries and keys, rotation and cache write for one step (csrc/prepare.hip).
    p float32 [T, columns] holds q (Hq heads of Dk) at q_off, k (Hk of Dk) at k_off and v (Hv of
    Dv) at v_off; k_off < 0: the layer has no keys and values of its own. q_out [T, Hq, Dk] and
    the caches (k [pages, Hk, page_size, Dk], v [pages, Hv, page_size, Dv]) share one dtype."""
    _f32_rows(p, "qkv_prepare: p")
    T = p.shape[0]
    own = k_off >= 0
    nq, nk, nv = Hq * Dk, Hk * Dk, Hv * Dv
    if q_off < 0 or q_off + nq > p.shape[1] or (own and (k_off + nk > p.shape[1] or v_off < 0
                                                         or v_off + nv > p.shape[1])):
        raise KernelError("qkv_prepare: the columns of q, k or v lie outside p")
    if q_out.shape != (T, Hq, Dk) or not q_out.is_contiguous() or not q_out.is_cuda:
        raise KernelError(f"qkv_prepare: q_out must be a contiguous [{T}, {Hq}, {Dk}] GPU tensor")
    _f32_vec(q_bias, nq, "qkv_prepare: q bias")
    nw_q, nw_k = (nq, nk) if norm_mode == NORM_WHOLE else (Dk, Dk)
    if norm_mode != NORM_NONE:
        if q_weight is None or (own and k_weight is None):
            raise KernelError("qkv_prepare: a norm needs its weights")
        _f32_vec(q_weight, nw_q, "qkv_prepare: q norm weight")
    if rot_dims:
        if rot_dims % 2 or rot_dims > Dk:
            raise KernelError(f"qkv_prepare: {rot_dims} rotating entries of {Dk}")
        _f32_vec(inv_freq, rot_dims // 2, "qkv_prepare: frequencies")
    _i32(positions, "positions")
    if positions.numel() != T:
        raise KernelError("qkv_prepare: one position a row")
    write = own and slots is not None
    if own:
        _f32_vec(k_bias, nk, "qkv_prepare: k bias")
        _f32_vec(v_bias, nv, "qkv_prepare: v bias")
        if norm_mode != NORM_NONE:
            _f32_vec(k_weight, nw_k, "qkv_prepare: k norm weight")
    if write:
        _i32(slots, "slots")
        _need_gpu(k_cache, v_cache, slots)
        if (slots.numel() != T or k_cache.dim() != 4 or v_cache.dim() != 4
                or k_cache.shape[1:] != (Hk, page_size, Dk) or v_cache.shape[1:] != (Hv, page_size, Dv)
                or k_cache.shape[0] != v_cache.shape[0] or k_cache.dtype != q_out.dtype
                or v_cache.dtype != q_out.dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
            raise KernelError("qkv_prepare: caches must be contiguous [pages, heads, page_size, size] of "
                              "q_out's dtype, with one slot a row")
    _check(library.load("prepare").ptl_qkv_prepare(
        _ptr(q_out), _ptr(p), ctypes.c_long(p.stride(0)), int(q_off), int(k_off) if own else -1, int(v_off),
        _ptr(q_bias), _ptr(k_bias) if own else None, _ptr(v_bias) if own else None, int(norm_mode),
        _ptr(q_weight), _ptr(k_weight) if own else None, ctypes.c_float(eps), int(rot_dims),
        _ptr(inv_freq) if rot_dims else None, ctypes.c_float(mag), _ptr(positions),
        _ptr(slots) if write else None, _ptr(k_cache) if write else None, _ptr(v_cache) if write else None,
        T, Hq, Hk, Hv, Dk, Dv, int(page_size), _dtype_code(q_out), _stream()), "qkv_prepare")


def head_norm_gate(out: torch.Tensor, a: torch.Tensor, maps: int = 1, lam: float = 0.0, weight=None,
                   weight_per_head: bool = False, mult: float = 1.0, gate: Optional[torch.Tensor] = None,
                   gate_off: int = 0, act: int = GATE_NONE, eps: float = 0.0) -> None:
    """out[t, h, :] = rmsnorm(o)(no weight) * weight * mult * act(gate[t, gate_off + h Dv + :]) with
    o = a[t, h] (maps 1) or a[t, 2h] - lam a[t, 2h + 1] (maps 2), a float32 [T, H * maps, Dv]
    contiguous, out [T, H * Dv] (rows may be strided) float32 or bfloat16, gate a float32 matrix."""
    _need_gpu(out, a, weight, gate)
    if a.dim() != 3 or a.dtype != torch.float32 or not a.is_contiguous() or maps not in (1, 2) or a.shape[1] % maps:
        raise KernelError("head_norm_gate: a must be contiguous float32 [T, H * maps, Dv], maps 1 or 2")
    T, HA, Dv = a.shape
    H = HA // maps
    if out.dim() != 2 or out.shape != (T, H * Dv) or out.stride(1) != 1:
        raise KernelError(f"head_norm_gate: out must be [{T}, {H * Dv}] with dense rows")
    if weight is not None:
        _f32_vec(weight, H * Dv if weight_per_head else Dv, "head_norm_gate: weight")
    ldg = 0
    if gate is not None:
        _f32_rows(gate, "head_norm_gate: gate")
        if gate.shape[0] != T or gate_off < 0 or gate_off + H * Dv > gate.shape[1] or act == GATE_NONE:
            raise KernelError("head_norm_gate: the gate's columns lie outside its matrix, or no activation")
        ldg = gate.stride(0)
    _check(library.load("prepare").ptl_head_norm_gate(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(a), int(maps), ctypes.c_float(lam), _ptr(weight),
        Dv if weight_per_head else 0, ctypes.c_float(mult), _ptr(gate), ctypes.c_long(ldg), int(gate_off),
        int(act), ctypes.c_float(eps), T, H, Dv, _dtype_code(out), _stream()), "head_norm_gate")


def stream_add_rmsnorm_sum(stream: torch.Tensor, y1: torch.Tensor, a: float, y2: Optional[torch.Tensor],
                           b: float, bias: Optional[torch.Tensor], c: float, weight: torch.Tensor,
                           eps: float, out_dtype: Optional[torch.dtype] = None, want_copy: bool = False):
    """stream += rmsnorm(a y1 + b y2 + c bias) * weight in place (y2 and bias optional); returns a
    copy of the new stream in ``out_dtype`` when asked, else None."""
    T, H = _check_stream(stream, "stream_add_rmsnorm_sum")
    _need_gpu(y1, y2, bias, weight)
    for y in (y1, y2):
        if y is not None and (y.shape != stream.shape or not y.is_contiguous() or y.dtype != y1.dtype):
            raise KernelError("stream_add_rmsnorm_sum: the terms must be contiguous matrices of the stream's "
                              "shape and of one dtype")
    _f32_vec(bias, H, "stream_add_rmsnorm_sum: bias")
    _f32_vec(weight, H, "stream_add_rmsnorm_sum: weight")
    out_dtype = out_dtype or torch.float32
    copy = torch.empty((T, H), dtype=out_dtype, device=stream.device) if want_copy else None
    _check(library.load("stream").ptl_stream_add_rmsnorm_sum(
        _ptr(stream), _ptr(y1), ctypes.c_float(a), _ptr(y2), ctypes.c_float(b), _dtype_code(y1), _ptr(bias),
        ctypes.c_float(c), _ptr(weight), ctypes.c_float(eps), _ptr(copy),
        _F32 if out_dtype == torch.float32 else _BF16, T, H, _stream()), "stream_add_rmsnorm_sum")
    return copy


def stream_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """rmsnorm(x) * weight for rows x of a float32 stream, in ``out_dtype``."""
    T, H = _check_stream(x, "stream_rmsnorm")
    _need_gpu(weight)
    _f32_vec(weight, H, "stream_rmsnorm: weight")
    out = torch.empty((T, H), dtype=out_dtype, device=x.device)
    _check(library.load("stream").ptl_stream_rmsnorm(
        _ptr(out), _F32 if out_dtype == torch.float32 else _BF16, _ptr(x), _ptr(weight), ctypes.c_float(eps),
        T, H, _stream()), "stream_rmsnorm")
    return out


# ---------------------------------------------------------------------------
# Matrices carried from token to token (csrc/recurrent.hip)
def recurrent_block_floats(D: int) -> int:
    """Floats that 16 columns of a head's matrix take in a state slot (with n and m behind them)."""
    return 16 * D + D + 4


def recurrent_state_floats(H: int, D: int, Dv: int) -> int:
    """Floats of the matrices of all heads in a state slot."""
    return H * (-(-Dv // 16)) * recurrent_block_floats(D)


def _check_scan(state, q_start, state_slots, H, D, Dv, what):
    _need_gpu(state, q_start, state_slots)
    _i32(q_start, "q_start")
    _i32(state_slots, "state_slots")
    if state.dim() != 2 or state.dtype != torch.float32 or not state.is_contiguous() \
            or state.shape[1] < recurrent_state_floats(H, D, Dv):
        raise KernelError(f"{what}: state must be contiguous float32 [slots, >= {recurrent_state_floats(H, D, Dv)}]")
    n = state_slots.numel()
    if q_start.numel() != n + 1:
        raise KernelError(f"{what}: q_start has one entry more than there are sequences")
    if D > 256:
        raise KernelError(f"{what}: key sizes up to 256, got {D}")
    return n


def conv_prepare(p: torch.Tensor, x_off: int, conv_weight: torch.Tensor, state: torch.Tensor, tail_off: int,
                 q_start: torch.Tensor, state_slots: torch.Tensor, G: int, H: int, D: int, Dv: int,
                 qscale: float):
    """Short causal convolutions over time, SiLU, unit norm of q and k (csrc/recurrent.hip). p
    float32 [T, columns] holds the inputs q | k | v (G heads of D, G of D, H of Dv) from x_off on;
    conv_weight float32 [C, taps]; the state slots hold the last taps - 1 inputs [taps - 1, C] at
    tail_off. Returns float32 q [T, G, D] (unit vectors times qscale), k [T, G, D], v [T, H, Dv]."""
    _f32_rows(p, "conv_prepare: p")
    T = p.shape[0]
    C = 2 * G * D + H * Dv
    n = _check_scan(state, q_start, state_slots, H, D, Dv, "conv_prepare")
    if conv_weight.dim() != 2 or conv_weight.shape[0] != C:
        raise KernelError(f"conv_prepare: conv_weight must be [{C}, taps]")
    taps = conv_weight.shape[1]
    _f32_vec(conv_weight, C * taps, "conv_prepare: conv_weight")
    if x_off < 0 or x_off + C > p.shape[1] or tail_off < 0 or tail_off + (taps - 1) * C > state.shape[1]:
        raise KernelError("conv_prepare: columns outside p, or the tail outside the state")
    qn = torch.empty((T, G, D), dtype=torch.float32, device=p.device)
    kn = torch.empty((T, G, D), dtype=torch.float32, device=p.device)
    vv = torch.empty((T, H, Dv), dtype=torch.float32, device=p.device)
    _check(library.load("recurrent").ptl_conv_prepare(
        _ptr(qn), _ptr(kn), _ptr(vv), _ptr(p), ctypes.c_long(p.stride(0)), int(x_off), _ptr(conv_weight),
        int(taps), _ptr(state), ctypes.c_long(state.stride(0)), ctypes.c_long(tail_off), _ptr(q_start),
        _ptr(state_slots), n, T, G, H, D, Dv, ctypes.c_float(qscale), _stream()), "conv_prepare")
    return qn, kn, vv


def conv_tail_update(p: torch.Tensor, x_off: int, C: int, taps: int, state: torch.Tensor, tail_off: int,
                     q_start: torch.Tensor, state_slots: torch.Tensor) -> None:
    """The slots' last taps - 1 inputs after this step (after conv_prepare has read the old ones)."""
    _f32_rows(p, "conv_tail_update: p")
    _need_gpu(state, q_start, state_slots)
    if state.dim() != 2 or state.dtype != torch.float32 or not state.is_contiguous() \
            or tail_off + (taps - 1) * C > state.shape[1] or x_off + C > p.shape[1]:
        raise KernelError("conv_tail_update: the tail lies outside the state, or the inputs outside p")
    _i32(q_start, "q_start")
    _i32(state_slots, "state_slots")
    _check(library.load("recurrent").ptl_conv_tail_update(
        _ptr(state), ctypes.c_long(state.stride(0)), ctypes.c_long(tail_off), _ptr(p),
        ctypes.c_long(p.stride(0)), int(x_off), _ptr(q_start), _ptr(state_slots), state_slots.numel(),
        int(C), int(taps), _stream()), "conv_tail_update")


# Segments of the delta rule (ptl_delta_scan_segments): 256 tokens, 512 from 2,048 rows on, used from
# 768 rows on. Measured on MI355X, 16 heads of 128 x 128, one sequence, us (one chain / 128 / 256 /
# 512): 512 rows 194 / 152 / 155 / 159; 1,024 rows 364 / 280 / 219 / 274; 2,048 rows 765 / 554 / 397 /
# 360; 4,096 rows 1,471 / 1,104 / 764 / 611. The step from segment to segment (a D x D matrix times
# the state, one after the other) is what short segments pay for.
DELTA_SEGMENTS_FROM = 768


def delta_segment(max_q_len: int) -> int:
    return 512 if max_q_len >= 2048 else 256


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, p: torch.Tensor, a_off: int, b_off: int,
               A_log: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor,
               state_slots: torch.Tensor, max_q_len: int = 0) -> torch.Tensor:
    """The gated delta rule over the rows of every sequence, from and to the state slots. q, k
    float32 [T, G, D], v float32 [T, H, Dv]; the raw gates a (decay) and b (beta) are columns
    a_off + h and b_off + h of the float32 matrix p. Returns float32 [T, H, Dv]. ``max_q_len``: the
    rows of the step's longest sequence (or a bound); from DELTA_SEGMENTS_FROM rows on the
    sequences are worked on in segments side by side (a segment's effect on the state is
    S_end = W S_start + L; W comes from the same walk as L, started from the identity)."""
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    _f32_rows(p, "delta_scan: p")
    n = _check_scan(state, q_start, state_slots, H, D, Dv, "delta_scan")
    for t, shape in ((q, (T, G, D)), (k, (T, G, D)), (v, (T, H, Dv))):
        if t.shape != shape or t.dtype != torch.float32 or not t.is_contiguous() or not t.is_cuda:
            raise KernelError("delta_scan: q, k [T, G, D] and v [T, H, Dv] must be contiguous float32")
    if H % G or min(a_off, b_off) < 0 or max(a_off, b_off) + H > p.shape[1] or p.shape[0] != T:
        raise KernelError("delta_scan: gates outside p, or heads that do not divide")
    _f32_vec(A_log, H, "delta_scan: A_log")
    _f32_vec(dt_bias, H, "delta_scan: dt_bias")
    out = torch.empty((T, H, Dv), dtype=torch.float32, device=q.device)
    pa, pb = p[:, a_off:], p[:, b_off:]
    lib = library.load("recurrent")
    seg_len = delta_segment(int(max_q_len))
    segments = -(-int(max_q_len) // seg_len)
    work_floats = n * segments * H * (-(-Dv // 16) + -(-D // 16)) * 16 * D
    if max_q_len >= DELTA_SEGMENTS_FROM and n * segments <= 65535 and work_floats <= (1 << 27):
        work = torch.empty((work_floats,), dtype=torch.float32, device=q.device)
        _check(lib.ptl_delta_scan_segments(
            _ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(pa), _ptr(pb), ctypes.c_long(p.stride(0)), _ptr(A_log),
            _ptr(dt_bias), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(work), int(segments),
            seg_len, _ptr(q_start), _ptr(state_slots), n, H, G, D, Dv, _stream()), "delta_scan")
        return out
    _check(lib.ptl_delta_scan(
        _ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(pa), _ptr(pb), ctypes.c_long(p.stride(0)), _ptr(A_log),
        _ptr(dt_bias), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(q_start), _ptr(state_slots), n,
        H, G, D, Dv, _stream()), "delta_scan")
    return out


MEMORY_SEGMENT = 128          # tokens of a segment of a long portion (measured: 64 to 512 tried at 512 to 4,096 rows)
MEMORY_SEGMENTS_FROM = 256    # rows of the longest sequence of a step from which segments are used


def memory_scan(p: torch.Tensor, q_off: int, k_off: int, v_off: int, i_off: int, f_off: int,
                i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float, qscale: float, state: torch.Tensor,
                q_start: torch.Tensor, state_slots: torch.Tensor, H: int, D: int, Dv: int,
                max_q_len: int = 0) -> torch.Tensor:
    """The matrix memory with exponential gates and a running maximum over the rows of every
    sequence, from and to the state slots. q, k (H heads of D), v (H of Dv) and the raw gates i, f
    (H each) are columns of the float32 matrix p. Returns float32 [T, H, Dv]. ``max_q_len``: the
    rows of the step's longest sequence (or a bound); from MEMORY_SEGMENTS_FROM rows on the
    sequences are worked on in segments side by side (the transition of this memory is a scalar, so
    the segments' start states follow from what each adds and the product of its decays)."""
    _f32_rows(p, "memory_scan: p")
    T = p.shape[0]
    n = _check_scan(state, q_start, state_slots, H, D, Dv, "memory_scan")
    for off, width in ((q_off, H * D), (k_off, H * D), (v_off, H * Dv), (i_off, H), (f_off, H)):
        if off < 0 or off + width > p.shape[1]:
            raise KernelError("memory_scan: columns outside p")
    _f32_vec(i_bias, H, "memory_scan: i bias")
    _f32_vec(f_bias, H, "memory_scan: f bias")
    out = torch.empty((T, H, Dv), dtype=torch.float32, device=p.device)
    lib = library.load("recurrent")
    segments = -(-int(max_q_len) // MEMORY_SEGMENT)
    work_floats = n * segments * recurrent_state_floats(H, D, Dv)
    if max_q_len >= MEMORY_SEGMENTS_FROM and n * segments <= 65535 and work_floats <= (1 << 27):
        gates = torch.empty((T, H, 4), dtype=torch.float32, device=p.device)
        work = torch.empty((work_floats,), dtype=torch.float32, device=p.device)
        _check(lib.ptl_memory_scan_segments(
            _ptr(out), _ptr(p), ctypes.c_long(p.stride(0)), int(q_off), int(k_off), int(v_off), int(i_off),
            int(f_off), _ptr(i_bias), _ptr(f_bias), ctypes.c_float(cap), ctypes.c_float(qscale), _ptr(state),
            ctypes.c_long(state.stride(0)), _ptr(gates), _ptr(work), int(segments), MEMORY_SEGMENT,
            _ptr(q_start), _ptr(state_slots), n, H, D, Dv, _stream()), "memory_scan")
        return out
    _check(lib.ptl_memory_scan(
        _ptr(out), _ptr(p), ctypes.c_long(p.stride(0)), int(q_off), int(k_off), int(v_off), int(i_off),
        int(f_off), _ptr(i_bias), _ptr(f_bias), ctypes.c_float(cap), ctypes.c_float(qscale), _ptr(state),
        ctypes.c_long(state.stride(0)), _ptr(q_start), _ptr(state_slots), n, H, D, Dv, _stream()),
        "memory_scan")
    return out


# ---------------------------------------------------------------------------
# Routed experts (csrc/moe.hip)
ACT_SILU, ACT_CLAMPED = 0, 1           # gated: act(gate) * up
ACT_RELU2 = 2                          # no gate: relu(up)^2
SCORE_SIGMOID, SCORE_SOFTMAX = 0, 1


def gated_act(gate_up: torch.Tensor, act: int, limit: float = 0.0) -> torch.Tensor:
    """The gated activation ``act`` on a dense gate|up product [T, 2 I] -> [T, I]."""
    _need_gpu(gate_up)
    if gate_up.dim() != 2 or not gate_up.is_contiguous() or gate_up.shape[1] % 2:
        raise KernelError("gated_act: input must be a contiguous [T, 2I] matrix")
    T, I2 = gate_up.shape
    out = torch.empty((T, I2 // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(library.load("moe").ptl_gated_act(_ptr(out), _ptr(gate_up), T, I2 // 2, int(act),
                                             ctypes.c_float(limit), _dtype_code(gate_up), _stream()), "gated_act")
    return out


class Routing:
    """Where the (token, choice) pairs of a step went: see csrc/moe.hip."""
    __slots__ = ("idx", "wgt", "extra", "pos_of", "sorted", "expert_end", "tile_expert", "tile_row0",
                 "max_tiles", "top", "experts", "ident")


def moe_route(logits: torch.Tensor, experts: int, top: int, extra: int = 0,
              renormalize: bool = False, score: int = SCORE_SIGMOID, correction: Optional[torch.Tensor] = None,
              identity: int = 0, renorm_eps: float = 0.0, weight_scale: float = 1.0,
              groups: int = 1, keep_groups: int = 1) -> Routing:
    """Route every row of float32 ``logits`` [T, experts + identity + extra] to ``top`` of its
    ``experts + identity`` router outputs and order the pairs by expert. Scores: the sigmoid of
    the logits, or their softmax over the router outputs; the choice goes by score +
    ``correction`` [experts + identity] when one is given; the weights are the scores
    (``renormalize``: divided by their sum + renorm_eps) times weight_scale. The last
    ``identity`` outputs are experts that return their input: their pairs take no part in the
    products, and ``ident`` [T] holds the sum of their weights a token. ``groups`` > 1: the router
    outputs form that many equal groups of neighbours (at most 64); a group's score is the sum
    of its two largest choice scores (score + correction), and only outputs of the best
    ``keep_groups`` groups can be chosen."""
    _need_gpu(logits)
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1 \
            or logits.shape[1] < experts + extra:
        raise KernelError("moe_route: logits must be float32 [T, experts + extra] with dense rows")
    outputs = experts + identity
    if identity < 0 or logits.shape[1] < outputs + extra:
        raise KernelError("moe_route: logits must be float32 [T, experts + identity + extra]")
    if not 0 < top <= outputs or outputs > 1024 or not 0 <= extra <= 64 or experts < 1:
        raise KernelError(f"moe_route: {top} of {experts} + {identity} experts (+{extra}) is not a case the "
                          "kernel takes")
    if correction is not None:
        _f32_vec(correction, outputs, "moe_route: correction")
    if groups < 1 or (groups > 1 and (groups > 64 or outputs % groups or not 1 <= keep_groups <= groups
                                      or keep_groups * (outputs // groups) < top)):
        raise KernelError(f"moe_route: {groups} groups of which {keep_groups} are kept do not fit "
                          f"{outputs} router outputs with {top} chosen (at most 64 equal groups)")
    T = logits.shape[0]
    A = T * top
    lib = library.load("moe")
    r = Routing()
    r.top, r.experts = top, experts
    dev = logits.device
    r.max_tiles = int(lib.ptl_moe_max_tiles(A, experts))
    ints = torch.empty(3 * A + experts + 2 * r.max_tiles, dtype=torch.int32, device=dev)
    r.idx, r.pos_of, r.sorted = ints[:A], ints[A:2 * A], ints[2 * A:3 * A]
    r.expert_end = ints[3 * A:3 * A + experts]
    r.tile_expert = ints[3 * A + experts:3 * A + experts + r.max_tiles]
    r.tile_row0 = ints[3 * A + experts + r.max_tiles:]
    r.wgt = torch.empty(A, dtype=torch.float32, device=dev)
    r.extra = torch.empty((T, extra), dtype=torch.float32, device=dev) if extra else None
    r.ident = torch.empty(T, dtype=torch.float32, device=dev) if identity else None
    _check(lib.ptl_moe_topk(_ptr(logits), int(logits.stride(0)), T, outputs, top, extra, int(renormalize),
                            int(score), _ptr(correction), experts, ctypes.c_float(renorm_eps),
                            ctypes.c_float(weight_scale), int(groups), int(keep_groups), _ptr(r.idx),
                            _ptr(r.wgt), _ptr(r.extra), _ptr(r.ident), _stream()), "moe_topk")
    _check(lib.ptl_moe_sort(_ptr(r.idx), A, experts, _ptr(r.pos_of), _ptr(r.sorted), _ptr(r.expert_end),
                            _ptr(r.tile_expert), _ptr(r.tile_row0), r.max_tiles, _stream()), "moe_sort")
    return r


def moe_experts(x: torch.Tensor, r: Routing, gate_up: torch.Tensor, down: torch.Tensor, act: int,
                limit: float, weight_on_input: bool, shared: Optional[torch.Tensor] = None,
                shared_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The routed experts on x [T, K]: gate_up [E, 2 I, K] (for an activation without a gate,
    ACT_RELU2: the up matrices [E, I, K]), down [E, N, I]; returns float32 [T, N] = sum over a
    row's choices of its experts' outputs (+ shared_gate[t] * shared[t], + r.ident[t] * x[t] for
    the experts that return their input)."""
    _need_gpu(x, gate_up, down, shared, shared_gate)
    T, K = x.shape
    E, I2, _ = gate_up.shape
    gated = act != ACT_RELU2
    I, N = (I2 // 2 if gated else I2), down.shape[1]
    if r.ident is not None and (N != K or weight_on_input):
        raise KernelError("moe_experts: experts that return their input need a result of the input's size "
                          "and weights on the output")
    if x.stride(1) != 1 or gate_up.shape != (E, (2 if gated else 1) * I, K) or down.shape != (E, N, I) or E != r.experts \
            or not gate_up.is_contiguous() or not down.is_contiguous() \
            or not (x.dtype == gate_up.dtype == down.dtype) or r.idx.numel() != T * r.top:
        raise KernelError("moe_experts: shapes or dtypes do not fit the routing")
    if shared is not None and (shared.shape != (T, N) or shared.dtype != x.dtype or not shared.is_contiguous()):
        raise KernelError("moe_experts: the shared expert's output must be contiguous [T, N]")
    if shared_gate is not None and (shared_gate.dtype != torch.float32 or shared_gate.shape[0] != T
                                    or shared_gate.dim() != 2):
        raise KernelError("moe_experts: the shared expert's gate must be float32 [T, n]")
    lib = library.load("moe")
    A = T * r.top
    code = _dtype_code(x)
    mid = torch.empty((A, I), dtype=x.dtype, device=x.device)
    if gated:
        _check(lib.ptl_moe_gate_up(_ptr(mid), ctypes.c_long(I), _ptr(x), ctypes.c_long(x.stride(0)), _ptr(gate_up),
                                   _ptr(r.tile_expert), _ptr(r.tile_row0), _ptr(r.expert_end), _ptr(r.sorted),
                                   _ptr(r.wgt) if weight_on_input else None, r.max_tiles, A, r.top, I, K, int(act),
                                   ctypes.c_float(limit), code, _stream()), "moe_gate_up")
    else:
        _check(lib.ptl_moe_up(_ptr(mid), ctypes.c_long(I), _ptr(x), ctypes.c_long(x.stride(0)), _ptr(gate_up),
                              _ptr(r.tile_expert), _ptr(r.tile_row0), _ptr(r.expert_end), _ptr(r.sorted),
                              _ptr(r.wgt) if weight_on_input else None, r.max_tiles, A, r.top, I, K, int(act),
                              code, _stream()), "moe_up")
    rows = torch.empty((A, N), dtype=x.dtype, device=x.device)
    _check(lib.ptl_moe_down(_ptr(rows), ctypes.c_long(N), _ptr(mid), ctypes.c_long(I), _ptr(down),
                            _ptr(r.tile_expert), _ptr(r.tile_row0), _ptr(r.expert_end), r.max_tiles, A, N, I,
                            code, _stream()), "moe_down")
    y = torch.empty((T, N), dtype=torch.float32, device=x.device)
    _check(lib.ptl_moe_combine(_ptr(y), _ptr(rows), ctypes.c_long(N), _ptr(r.pos_of),
                               None if weight_on_input else _ptr(r.wgt), r.top, _ptr(shared), _ptr(shared_gate),
                               int(shared_gate.stride(0)) if shared_gate is not None else 0,
                               _ptr(x) if r.ident is not None else None, ctypes.c_long(x.stride(0)),
                               _ptr(r.ident), T, N, code, _stream()), "moe_combine")
    return y


def unary_act(u: torch.Tensor, act: int = ACT_RELU2) -> torch.Tensor:
    """An activation without a gate on a dense product [T, I] (ACT_RELU2: relu(u)^2)."""
    _need_gpu(u)
    if u.dim() != 2 or not u.is_contiguous():
        raise KernelError("unary_act: input must be a contiguous [T, I] matrix")
    out = torch.empty_like(u)
    _check(library.load("moe").ptl_unary_act(_ptr(out), _ptr(u), u.shape[0], u.shape[1], int(act),
                                             _dtype_code(u), _stream()), "unary_act")
    return out


# ---------------------------------------------------------------------------
# The selective scan (csrc/selective.hip)
def selective_state_floats(channels: int, state: int, taps: int) -> int:
    """Floats of a state slot: the states [channels, state], then the convolution's last
    taps - 1 inputs [taps - 1, channels]."""
    return channels * state + (taps - 1) * channels


def selective_conv(p: torch.Tensor, x_off: int, conv_weight: torch.Tensor, conv_bias: Optional[torch.Tensor],
                   state: torch.Tensor, tail_off: int, q_start: torch.Tensor, state_slots: torch.Tensor,
                   max_q_len: int, lp_dtype: Optional[torch.dtype] = None):
    """silu(causal convolution over time + bias) of the channels p[:, x_off : x_off + C] (float32);
    conv_weight float32 [C, taps], the last column is the current token's; inputs before the step's
    first token come from the slots' tails [taps - 1, C] at tail_off. Returns (float32 [T, C], the
    same in ``lp_dtype`` or None)."""
    _f32_rows(p, "selective_conv: p")
    _need_gpu(conv_weight, state, q_start, state_slots)
    T = p.shape[0]
    if conv_weight.dim() != 2:
        raise KernelError("selective_conv: conv_weight must be [C, taps]")
    C, taps = conv_weight.shape
    _f32_vec(conv_weight, C * taps, "selective_conv: conv_weight")
    if conv_bias is not None:
        _f32_vec(conv_bias, C, "selective_conv: conv_bias")
    if state.dim() != 2 or state.dtype != torch.float32 or not state.is_contiguous() or x_off < 0 \
            or x_off + C > p.shape[1] or tail_off < 0 or tail_off + (taps - 1) * C > state.shape[1]:
        raise KernelError("selective_conv: columns outside p, or the tail outside the state")
    _i32(q_start, "q_start")
    _i32(state_slots, "state_slots")
    n = state_slots.numel()
    if q_start.numel() != n + 1:
        raise KernelError("selective_conv: q_start has one entry more than there are sequences")
    xc = torch.empty((T, C), dtype=torch.float32, device=p.device)
    lp = None
    if lp_dtype is not None and lp_dtype != torch.float32:
        lp = torch.empty((T, C), dtype=lp_dtype, device=p.device)
    _check(library.load("selective").ptl_selective_conv(
        _ptr(xc), _ptr(lp), _dtype_code(lp) if lp is not None else _F32, _ptr(p), ctypes.c_long(p.stride(0)),
        int(x_off), _ptr(conv_weight), _ptr(conv_bias), int(taps), _ptr(state), ctypes.c_long(state.stride(0)),
        ctypes.c_long(tail_off), _ptr(q_start), _ptr(state_slots), n, int(max_q_len), C, _stream()),
        "selective_conv")
    return xc, lp


SELECTIVE_SEGMENTS_FROM = 64      # rows of the longest sequence of a step from which segments are used
SELECTIVE_SEGMENT_STATES = 32     # states a channel up to which a lane can hold them all
SELECTIVE_SEGMENT_WAVES = 4096    # waves of a pass that fill the chip; segments are as long as this allows


def selective_segment(n_seqs: int, max_q_len: int, channels: int, rows: int = 0) -> int:
    """Tokens of a segment of a step's long portions: a power of two from 16 to 256, as long as the
    step still has SELECTIVE_SEGMENT_WAVES waves (64 channels a wave and segment). ``rows``: the
    rows of the step when known (a long portion beside single tokens has far fewer segments than
    sequences times the longest one's)."""
    n_seqs = max(1, int(n_seqs))
    rows = min(int(rows), n_seqs * int(max_q_len)) if rows > 0 else n_seqs * int(max_q_len)
    seg = 256
    while seg > 16 and -(-channels // 64) * (rows // seg + n_seqs) < SELECTIVE_SEGMENT_WAVES:
        seg //= 2
    return seg


def selective_scan(xc: torch.Tensor, p: torch.Tensor, z_off: int, r: torch.Tensor, rank: int, b_off: int,
                   c_off: int, w_dt: torch.Tensor, dt_bias: torch.Tensor, A_log: torch.Tensor, D: torch.Tensor,
                   state: torch.Tensor, q_start: torch.Tensor, state_slots: torch.Tensor,
                   out_dtype: torch.dtype, max_q_len: int = 0, seg_len: int = 0) -> torch.Tensor:
    """The recurrence S <- exp(dt A) S + dt x B, y = S C + D x, and the gate y * silu(z), for every
    sequence of the step from its slot's state [C, N] (at the start of the slot), which it leaves
    advanced. xc float32 [T, C]; z = p[:, z_off : z_off + C] (float32); r float32 rows with the
    step input in columns 0..rank-1, B [N] at b_off, C [N] at c_off; w_dt [C, rank], dt_bias [C],
    A_log [C, N], D [C] float32. Returns [T, C] in ``out_dtype``. ``max_q_len``: the rows of the
    step's longest sequence (or a bound); from SELECTIVE_SEGMENTS_FROM rows on, with up to
    SELECTIVE_SEGMENT_STATES states a channel, the sequences are worked on in segments side by side
    (``seg_len`` tokens each, 0: chosen by selective_segment): the transition of a state is a
    scalar, so a segment's start state follows from what the segments before it add to a zero state
    and the sums of their step sizes."""
    _f32_rows(p, "selective_scan: p")
    _f32_rows(r, "selective_scan: r")
    _need_gpu(xc, w_dt, dt_bias, A_log, D, state, q_start, state_slots)
    if xc.dim() != 2 or xc.dtype != torch.float32 or not xc.is_contiguous():
        raise KernelError("selective_scan: xc must be a contiguous float32 [T, C] matrix")
    T, C = xc.shape
    if A_log.dim() != 2 or A_log.shape[0] != C:
        raise KernelError(f"selective_scan: A_log must be [{C}, N]")
    N, R = A_log.shape[1], int(rank)
    _f32_vec(A_log, C * N, "selective_scan: A_log")
    _f32_vec(w_dt, C * R, "selective_scan: w_dt")
    _f32_vec(dt_bias, C, "selective_scan: dt_bias")
    _f32_vec(D, C, "selective_scan: D")
    if p.shape[0] != T or r.shape[0] != T or z_off < 0 or z_off + C > p.shape[1] or R < 1 or R > r.shape[1] \
            or min(b_off, c_off) < 0 or max(b_off, c_off) + N > r.shape[1]:
        raise KernelError("selective_scan: columns outside p or r")
    if N > 256 or 4 * (16 * (R + 2 * N) + 16 * R + 1024) > 150 * 1024:
        raise KernelError(f"selective_scan: {N} states and a step input of {R} are more than the kernel takes")
    if state.dim() != 2 or state.dtype != torch.float32 or not state.is_contiguous() or state.shape[1] < C * N:
        raise KernelError("selective_scan: the state slots must be contiguous float32 rows of at least C * N")
    _i32(q_start, "q_start")
    _i32(state_slots, "state_slots")
    n = state_slots.numel()
    if q_start.numel() != n + 1:
        raise KernelError("selective_scan: q_start has one entry more than there are sequences")
    out = torch.empty((T, C), dtype=out_dtype, device=xc.device)
    z = p[:, z_off:]
    max_q_len = min(int(max_q_len), T)
    if max_q_len >= SELECTIVE_SEGMENTS_FROM and N <= SELECTIVE_SEGMENT_STATES:
        seg_len = int(seg_len) or selective_segment(n, max_q_len, C, T)
        segments = -(-max_q_len // seg_len)
        work_floats = 2 * n * segments * (N + 1) * C
        if segments <= 65535 and work_floats <= (1 << 28) and T <= 64 * 65535:
            dt_work = torch.empty((T, C), dtype=torch.float32, device=xc.device)
            work = torch.empty((work_floats,), dtype=torch.float32, device=xc.device)
            _check(library.load("selective").ptl_selective_scan_segments(
                _ptr(out), _dtype_code(out), _ptr(xc), _ptr(z), ctypes.c_long(p.stride(0)), _ptr(r),
                ctypes.c_long(r.stride(0)), int(b_off), int(c_off), _ptr(w_dt), _ptr(dt_bias), _ptr(A_log),
                _ptr(D), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(dt_work), _ptr(work), int(segments),
                int(seg_len), _ptr(q_start), _ptr(state_slots), n, T, C, N, R,
                0 if out_dtype == torch.float32 else 1, _stream()), "selective_scan")
            return out
    _check(library.load("selective").ptl_selective_scan(
        _ptr(out), _dtype_code(out), _ptr(xc), _ptr(z), ctypes.c_long(p.stride(0)), _ptr(r),
        ctypes.c_long(r.stride(0)), int(b_off), int(c_off), _ptr(w_dt), _ptr(dt_bias), _ptr(A_log), _ptr(D),
        _ptr(state), ctypes.c_long(state.stride(0)), _ptr(q_start), _ptr(state_slots), n, int(max_q_len), C, N, R,
        _stream()), "selective_scan")
    return out
