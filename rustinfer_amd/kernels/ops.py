"""The kernels as functions on torch tensors.

Each function checks devices, dtypes, shapes and contiguity, then calls the HIP entry point
on the current stream.  Tensors only lend their memory: no torch operator runs the model's
arithmetic, with one exception that the reference shares (it calls cuBLASLt for every
product with more than one row, crates/infer-backend-cuda/src/kernels/matmul/mod.rs:187-221):
a bfloat16 product with many rows may go to the library's GEMM.  The library is required:
if it cannot be built or loaded these functions raise.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

# rows at or below which a bfloat16 product uses the weight-streaming kernel
SKINNY_MAX_ROWS = 64
# a bfloat16 product with at least this many rows goes to the library GEMM (0: never)
LIBRARY_GEMM_MIN_ROWS = 65
UNTILED_LIBRARY_MIN_ROWS = 17   # a weight without a second, tile-ordered copy: from this many rows on the GEMM library reads it faster
UNTILED_LIBRARY_LARGE = 20 << 20 # ... and with fewer rows where it has this many elements, see _untiled_to_library
FORCE_LIBRARY_GEMM = False      # every bfloat16 product through the GEMM library, no few-row kernels and none of their fused forms
                                # (the reference's RUSTINFER_FORCE_GEMM, crates/infer-backend-cuda/src/kernels/matmul/mod.rs:188-204)
LIBRARY_GEMM_WORKSPACE_BYTES = 64 << 20


class KernelError(RuntimeError):
    pass


_SCRATCH = {}      # small device buffers the kernels need beside their operands


def _lib():
    return build.load()


def _check(rc: int) -> None:
    if rc != 0:
        raise KernelError(_lib().ri_last_error().decode("utf-8", "replace"))


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_STREAM = None       # the stream of the enclosing stream_scope, if any


def _stream():
    if _STREAM is not None:
        return _STREAM
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class stream_scope:
    """Within the scope every op launches on the stream that was current at its start, without
    asking torch for it each time (that question costs several microseconds, a hundred times a
    step).  The caller must not change the current stream inside the scope."""

    def __enter__(self):
        global _STREAM
        self._outer = _STREAM
        _STREAM = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _STREAM
        _STREAM = self._outer
        return False


class on_stream:
    """Within the scope every op launches on ``stream`` (a ``torch.cuda.Stream``), whatever torch's current
    stream is: for a part that runs two independent chains of kernels side by side.  The caller orders the two
    streams (``wait_stream``) before and after; torch's own current stream, and with it where scratch memory is
    allocated, stays as it is."""

    def __init__(self, stream):
        self._handle = ctypes.c_void_p(stream.cuda_stream)

    def __enter__(self):
        global _STREAM
        self._outer = _STREAM
        _STREAM = self._handle
        return self

    def __exit__(self, *exc):
        global _STREAM
        _STREAM = self._outer
        return False


def _dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU; there is no CPU path")


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}") from None


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None):
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous int32")
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} has {t.numel()} entries, {n} needed")


def _rows2d(t: torch.Tensor, name: str):
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name} must be 2-D with unit column stride, got shape {tuple(t.shape)} strides {t.stride()}")


def embed(ids: torch.Tensor, table: torch.Tensor, out_x: torch.Tensor,
          device_tokens: Optional[torch.Tensor] = None, scale: float = 1.0,
          act: Optional[torch.Tensor] = None) -> None:
    """``out_x[t] = table[ids[t]] * scale``; an id ``-(k+1)`` means ``device_tokens[k]`` (int32, on the
    device).  ``act`` ([T, d] in the table's dtype) takes the same rows rounded to its dtype."""
    _dev(ids, table, out_x, device_tokens, act)
    if device_tokens is not None:
        _i32(device_tokens, "device_tokens")
    T = ids.numel()
    _i32(ids, "ids")
    V, d = table.shape
    if out_x.dtype != torch.float32 or tuple(out_x.shape) != (T, d) or not out_x.is_contiguous():
        raise KernelError(f"embed: out must be contiguous float32 [{T}, {d}]")
    if not table.is_contiguous():
        raise KernelError("embed: table must be contiguous")
    if act is not None and (tuple(act.shape) != (T, d) or not act.is_contiguous() or act.dtype != table.dtype):
        raise KernelError(f"embed: the rounded copy must be contiguous [{T}, {d}] in the table's dtype")
    _check(_lib().ri_embed(_ptr(ids), _ptr(device_tokens), _ptr(table), _dt(table), _ptr(out_x), T, d, V,
                           ctypes.c_float(scale), _ptr(act), _dt(act) if act is not None else 0, _stream()))


def norm_residual(x: torch.Tensor, delta: Optional[torch.Tensor], weight: Optional[torch.Tensor], eps: float,
                  mult: float = 1.0, one_plus: bool = False, act: Optional[torch.Tensor] = None) -> None:
    """The norm on a sub-layer's output, added to the 32-bit residual stream in place:
    ``x += mult * delta * rsqrt(mean(delta^2) + eps) * (1 + weight if one_plus else weight)``.
    ``delta`` is ``[T, d]`` (activations' dtype or 32-bit) or a 32-bit stack ``[P, T, d]`` of partial
    sums.  ``act`` ([T, d]) takes the new ``x`` rounded to its dtype; with ``delta = None`` only that
    copy is made."""
    _dev(x, delta, weight, act)
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("norm_residual: x must be contiguous float32")
    parts, stride, ddt = 1, 0, F32
    if delta is not None:
        if delta.dim() == 3:
            parts, stride = delta.shape[0], delta.stride(0)
        if delta.dim() not in (2, 3) or tuple(delta.shape[-2:]) != (T, d) or delta.stride(-1) != 1 or delta.stride(-2) != d \
                or (delta.dim() == 3 and delta.dtype != torch.float32):
            raise KernelError("norm_residual: delta must be [T, d] or a float32 stack [P, T, d] with contiguous rows")
        if weight is None or weight.dtype != torch.float32 or weight.numel() != d or not weight.is_contiguous():
            raise KernelError(f"norm_residual: weight must be contiguous float32 with {d} entries")
        ddt = _dt(delta)
    elif act is None:
        return
    if act is not None and (tuple(act.shape) != (T, d) or not act.is_contiguous()):
        raise KernelError(f"norm_residual: the rounded copy must be contiguous [{T}, {d}]")
    _check(_lib().ri_norm_residual(_ptr(x), _ptr(delta), ddt, parts, ctypes.c_longlong(stride), _ptr(weight), F32,
                                   int(bool(one_plus)), ctypes.c_float(mult), ctypes.c_float(eps), _ptr(act),
                                   _dt(act) if act is not None else 0, T, d, _stream()))


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None,
                x_rows: Optional[torch.Tensor] = None, groups: int = 1) -> None:
    """``groups > 1``: every row is normed in that many equal consecutive parts, each divided by its own
    root mean square.  ``out`` may be 32-bit whatever the delta's dtype (a consumer that rounds later).
    ``x += delta`` (32-bit residual, in place unless ``rows`` gathers), ``out = rmsnorm(x) * weight``.
    ``delta`` is ``[T, d]`` in the activations' dtype or 32-bit, or a stack ``[P, T, d]`` of 32-bit
    partial sums that are added up here.  With ``rows``, ``x_rows`` ([len(rows), d], 32-bit) takes
    the sums ``x + delta`` of those rows: the residual stream cut down to them."""
    _dev(x, delta, weight, out, rows, x_rows)
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("add_rmsnorm: x must be contiguous float32")
    n_out = rows.numel() if rows is not None else T
    if rows is not None:
        _i32(rows, "rows")
    if tuple(out.shape) != (n_out, d) or not out.is_contiguous():
        raise KernelError(f"add_rmsnorm: out must be contiguous [{n_out}, {d}], got {tuple(out.shape)}")
    parts, stride, ddt = 1, 0, _dt(out)
    if delta is not None:
        if delta.dim() == 3:
            parts, stride = delta.shape[0], delta.stride(0)
        if tuple(delta.shape[-2:]) != (T, d) or delta.stride(-1) != 1 or delta.stride(-2) != d \
                or (delta.dim() == 3 and delta.dtype != torch.float32) or delta.dim() not in (2, 3):
            raise KernelError("add_rmsnorm: delta must be [T, d] or a float32 stack [P, T, d] with contiguous rows")
        if delta.dtype not in (out.dtype, torch.float32) and out.dtype != torch.float32:
            raise KernelError("add_rmsnorm: delta must be in the dtype of out or float32")
        ddt = _dt(delta)
    if weight.numel() != d or not weight.is_contiguous():
        raise KernelError(f"add_rmsnorm: weight must have {d} entries")
    if groups < 1 or d % groups:
        raise KernelError(f"add_rmsnorm: {d} values do not split into {groups} equal parts")
    if x_rows is not None and (rows is None or tuple(x_rows.shape) != (n_out, d) or x_rows.dtype != torch.float32
                               or not x_rows.is_contiguous()):
        raise KernelError(f"add_rmsnorm: x_rows goes with rows and must be contiguous float32 [{n_out}, {d}]")
    _check(_lib().ri_add_rmsnorm(_ptr(x), _ptr(delta), ddt, parts, ctypes.c_longlong(stride), _ptr(weight),
                                 _dt(weight), _ptr(out), _dt(out), n_out, d, ctypes.c_float(eps),
                                 _ptr(rows), _ptr(x_rows), int(groups), _stream()))


def add_rmsnorm_shift(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float, out: torch.Tensor,
                      mix: torch.Tensor, state: torch.Tensor, ctx, groups: int = 1) -> None:
    """``add_rmsnorm`` and ``token_shift`` in one pass, for a step whose every row is one token (row b is token
    b): ``x += delta``, ``h = rmsnorm(x) * weight`` (in ``groups`` parts), ``out = h + (prev - h) * mix`` with
    ``prev`` the request's last ``h`` from ``state [slots, d]`` (zeros at position 0), which ``h`` replaces.
    ``weight``, ``mix`` and ``state`` 32-bit."""
    _dev(x, delta, weight, out, mix, state)
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or tuple(out.shape) != (T, d) or not out.is_contiguous():
        raise KernelError("add_rmsnorm_shift: contiguous float32 x [T, d] and contiguous out [T, d] expected")
    if T > ctx.num_rows or ctx.max_q_len != 1:
        raise KernelError("add_rmsnorm_shift: only for steps whose every row is one token")
    parts, stride, ddt = 1, 0, F32
    if delta is not None:
        if delta.dim() == 3:
            parts, stride = delta.shape[0], delta.stride(0)
        if delta.dim() not in (2, 3) or tuple(delta.shape[-2:]) != (T, d) or delta.stride(-1) != 1 or delta.stride(-2) != d \
                or (delta.dim() == 3 and delta.dtype != torch.float32):
            raise KernelError("add_rmsnorm_shift: delta must be [T, d] or a float32 stack [P, T, d] with contiguous rows")
        ddt = _dt(delta)
    _f32_vec(weight, d, "add_rmsnorm_shift: the weight")
    _f32_vec(mix, d, "add_rmsnorm_shift: the mixing weights")
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != d or not state.is_contiguous():
        raise KernelError(f"add_rmsnorm_shift: state must be contiguous float32 [slots, {d}]")
    if groups < 1 or d % groups:
        raise KernelError(f"add_rmsnorm_shift: {d} values do not split into {groups} equal parts")
    _i32(ctx.positions, "positions", T)
    _i32(ctx.state_slots, "state_slots", ctx.num_rows)
    _check(_lib().ri_add_rmsnorm_shift(_ptr(x), _ptr(delta), ddt, parts, ctypes.c_longlong(stride), _ptr(weight), _ptr(out),
                                       _dt(out), T, d, ctypes.c_float(eps), int(groups), _ptr(mix), _ptr(state), state.shape[0],
                                       _ptr(ctx.state_slots), _ptr(ctx.positions), _stream()))


def _check_cache(k_cache, v_cache, Hkv, hd, page, act_dtype, name):
    if k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (Hkv, page, hd) or v_cache.dim() != 4 \
            or tuple(v_cache.shape) != (k_cache.shape[0], Hkv, hd, page):
        raise KernelError(f"{name}: caches must be k [pages, {Hkv}, {page}, {hd}] and v [pages, {Hkv}, {hd}, {page}], "
                          f"got {tuple(k_cache.shape)} and {tuple(v_cache.shape)}")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise KernelError(f"{name}: cache must be contiguous")
    if k_cache.dtype != act_dtype or v_cache.dtype != act_dtype:
        raise KernelError(f"{name}: cache dtype {k_cache.dtype} differs from the activations' {act_dtype}")


def rope_kv_write(qkv: torch.Tensor, H: int, Hkv: int, hd: int, rotary, positions: torch.Tensor,
                  row_of_token: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  block_table: torch.Tensor, page: int, write_kv: bool = True) -> None:
    _dev(qkv, positions, row_of_token, k_cache, v_cache, block_table)
    _rows2d(qkv, "qkv")
    T, width = qkv.shape
    has_kv = width >= H * hd + 2 * Hkv * hd
    if width not in (H * hd, H * hd + 2 * Hkv * hd):
        raise KernelError(f"rope_kv_write: row width {width} is neither q nor q+k+v for H={H} Hkv={Hkv} hd={hd}")
    _i32(positions, "positions", T)
    _i32(row_of_token, "row_of_token", T)
    cos = sin = None
    rot = 0
    rows = 0
    if rotary is not None:
        cos, sin, rot = rotary
        _dev(cos, sin)
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape \
                or cos.dim() != 2 or cos.shape[1] * 2 != rot or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("rope_kv_write: cos/sin must be contiguous float32 [positions, rot_dim/2]")
        rows = cos.shape[0]
    if write_kv:
        _check_cache(k_cache, v_cache, Hkv, hd, page, qkv.dtype, "rope_kv_write")
        _i32(block_table, "block_table")
        if block_table.dim() != 2:
            raise KernelError("rope_kv_write: block_table must be [rows, max_blocks]")
    max_blocks = block_table.shape[1] if block_table is not None and block_table.dim() == 2 else 0
    _check(_lib().ri_rope_kv_write(
        _ptr(qkv), _dt(qkv), T, qkv.stride(0), H, Hkv, hd, rot, _ptr(cos), _ptr(sin), rows,
        _ptr(positions), _ptr(row_of_token), _ptr(k_cache), _ptr(v_cache),
        k_cache.shape[0] if k_cache is not None else 0, _ptr(block_table), max_blocks, page,
        int(has_kv), int(bool(write_kv)), _stream()))


def qkv_rope_weight(w_qkv: torch.Tensor, hd: int) -> Optional[torch.Tensor]:
    """The fused q/k/v weight ``[(H + 2 Hkv) hd, K]`` in the form ``qkv_rope_fused`` reads: rows
    permuted within each head so that a 16-row tile holds 8 features of the first half and their 8
    rotary partners, then tile order (``tile_weight``).  None if the shape does not allow it."""
    N, K = w_qkv.shape
    if w_qkv.dtype != torch.bfloat16 or hd % 16 or N % hd or K % 32:
        return None
    r = torch.arange(N, device=w_qkv.device)
    head, within = r // hd, r % hd
    j, rr = within // 16, within % 16
    order = head * hd + torch.where(rr < 8, 8 * j + rr, hd // 2 + 8 * j + (rr - 8))
    return tile_weight(w_qkv[order].contiguous())


def _scale_args(scale, M: int, who: str):
    """``scale`` = (ssq [M, P] float32, eps) of a norm whose factor this product applies itself
    (see ``linear_residual``), or None."""
    if scale is None:
        return ctypes.c_void_p(0), 0, ctypes.c_float(0.0)
    ssq, eps = scale
    _dev(ssq)
    if ssq.dtype != torch.float32 or ssq.dim() != 2 or ssq.shape[0] != M or not ssq.is_contiguous():
        raise KernelError(f"{who}: the partial sums of squares must be contiguous float32 [{M}, parts]")
    return _ptr(ssq), ssq.shape[1], ctypes.c_float(eps)


def qkv_rope_fused(x: torch.Tensor, w_fused: torch.Tensor, qkv: torch.Tensor, H: int, Hkv: int, hd: int,
                   rotary, positions: torch.Tensor, row_of_token: torch.Tensor, k_cache: torch.Tensor,
                   v_cache: torch.Tensor, block_table: torch.Tensor, page: int, scale=None) -> bool:
    """For at most 64 single tokens: q/k/v projection, rotation by position and the write of k and v
    into the cache in one kernel; rotated q lands in the first H*hd columns of ``qkv``.  Returns False
    (and does nothing) where the fused form does not apply; the caller then runs the separate kernels.
    ``scale``: see ``linear``."""
    M, K = x.shape
    if FORCE_LIBRARY_GEMM or rotary is None or w_fused is None or x.dtype != torch.bfloat16 or not (0 < M <= SKINNY_MAX_ROWS):
        return False
    cos, sin, rot = rotary
    if rot != hd or x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16 or qkv.dtype != torch.bfloat16:
        return False
    _dev(x, w_fused, qkv, cos, sin, positions, row_of_token, k_cache, v_cache, block_table)
    N = (H + 2 * Hkv) * hd
    if tuple(w_fused.shape) != (N, K) or not w_fused.is_contiguous() or qkv.shape[0] != M or qkv.shape[1] < H * hd:
        raise KernelError("qkv_rope_fused: shapes do not fit")
    _rows2d(qkv, "qkv")
    _check_cache(k_cache, v_cache, Hkv, hd, page, x.dtype, "qkv_rope_fused")
    _i32(positions, "positions", M)
    _i32(row_of_token, "row_of_token", M)
    _i32(block_table, "block_table")
    if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] * 2 != hd or not cos.is_contiguous():
        raise KernelError("qkv_rope_fused: cos/sin must be contiguous float32 [positions, head_dim/2]")
    lds_rows = (M >= QKV_ROPE_LDS_MIN_ROWS and N >= QKV_ROPE_LDS_MIN_COLUMNS) or (M >= ROWS_LDS_MIN_ROWS and N * K >= QKV_ROPE_LDS_LARGE)
    if scale is None and lds_rows and K % 32 == 0 and hd % 16 == 0:
        # 33..64 tokens, or 17 and more over a large weight: the kernel whose blocks share the activations through LDS
        _check(_lib().ri_gemm_rows_qkv_rope(
            _ptr(x), x.stride(0), _ptr(w_fused), _ptr(qkv), qkv.stride(0), M, K, H, Hkv, hd, _ptr(cos), _ptr(sin),
            cos.shape[0], _ptr(positions), _ptr(row_of_token), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0],
            _ptr(block_table), block_table.shape[1], page, _stream()))
        return True
    sq, sp, se = _scale_args(scale, M, "qkv_rope_fused")
    _check(_lib().ri_gemm_qkv_rope(
        _ptr(x), x.stride(0), _ptr(w_fused), _ptr(qkv), qkv.stride(0), M, K, H, Hkv, hd, _ptr(cos), _ptr(sin),
        cos.shape[0], _ptr(positions), _ptr(row_of_token), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0],
        _ptr(block_table), block_table.shape[1], page, sq, sp, se, _stream()))
    return True


# A norm between two products of few rows has no kernel of its own: the product before it adds its
# sums to the residual stream and leaves (x * w_norm) and partial sums of x^2 (``linear_residual``),
# the product after it multiplies its sums by rsqrt(mean(x^2) + eps) (``scale=`` of ``linear``,
# ``linear_swiglu``, ``qkv_rope_fused``).  Up to this many rows (one tile of the matrix cores).
DEFERRED_NORM_MAX_ROWS = 16


def linear_residual_ok(M: int, w: torch.Tensor, w_tiled: Optional[torch.Tensor], norm_weight: torch.Tensor) -> bool:
    """Whether ``linear_residual`` takes ``M`` rows against ``w [N, K]`` before a norm with this weight."""
    N, K = w.shape
    return (not FORCE_LIBRARY_GEMM and w.dtype == torch.bfloat16 and w_tiled is not None and 0 < M <= DEFERRED_NORM_MAX_ROWS
            and N % 16 == 0 and K % 32 == 0 and norm_weight.dtype in _DT and norm_weight.numel() == N
            and norm_weight.is_contiguous())


RESIDUAL_FORM_LARGE = 32 << 20  # elements of a weight from which the residual form's weaknesses cost more than a norm kernel


def linear_residual_pays(M: int, w: torch.Tensor) -> bool:
    """Whether ``linear_residual`` is the faster way for ``M`` rows against ``w [N, K]``, compared
    with partial sums over slices of K and the norm's own kernel (which costs 4.6 us).  A block of
    the residual form owns 16 whole columns: it cannot divide K between blocks, so every block asks
    for all of its rows' activations (beyond eight rows that shows), and 320 blocks on 256 compute
    units take as long as 512.  Measured, us, residual form / partial sums, at 1, 8, 16 rows:
    4096 x 14336: 22.6 24.9 31.7 / 21.3 22.0 21.9; 4096 x 4096: 9.0 9.6 10.9 / 8.2 9.2 9.5;
    5120 x 13824: 31.7 38.1 49.2 / 26.3 26.6 27.6; 5120 x 5120: 13.3 16.4 20.7 / 13.4 13.1 13.3;
    8192 x 8192: 25.1 28.5 34.9 / 25.1 24.8 25.3; 3072 x 8192: 12.9 15.7 17.8 / 12.3 13.9 12.7."""
    N, K = w.shape
    if N * K < RESIDUAL_FORM_LARGE:
        return True
    tiles = N // 16
    blocks = tiles * 2 if tiles <= 128 else tiles
    at_once = 256 * -(-blocks // 256)
    return M <= 8 and blocks * 4 >= at_once * 3


def linear_residual(act: torch.Tensor, w: torch.Tensor, w_tiled: Optional[torch.Tensor], x: torch.Tensor,
                    norm_weight: torch.Tensor, workspace, name: str):
    """``x += act @ w^T`` in place (32-bit residual stream), and for the norm that follows:
    ``a = x * norm_weight`` in bfloat16 and partial sums of ``x^2``, ``ssq [M, P]``.  Returns
    ``(a, ssq)``.  For the shapes ``linear_residual_ok`` accepts."""
    M, K = act.shape
    N = w.shape[0]
    if not linear_residual_ok(M, w, w_tiled, norm_weight) or not _skinny_ok(act, w, M, K) or w.shape[1] != K:
        raise KernelError(f"linear_residual: {tuple(act.shape)} x {tuple(w.shape)}^T is not a shape this form takes")
    _dev(act, w_tiled, x, norm_weight)
    _tiled_ok(w, w_tiled)
    if x.dtype != torch.float32 or tuple(x.shape) != (M, N) or not x.is_contiguous():
        raise KernelError(f"linear_residual: x must be contiguous float32 [{M}, {N}]")
    lib = _lib()
    parts = lib.ri_gemm_skinny_residual_parts(N)      # a slot of partial sums for every 16 (or 8) columns
    a = workspace.get(name + ".a", M, N, torch.bfloat16)
    ssq = workspace.get(name + ".ssq", M, parts, torch.float32)
    _check(lib.ri_gemm_skinny_residual(_ptr(act), act.stride(0), _ptr(w_tiled), M, N, K, _ptr(x), _ptr(norm_weight),
                                       _dt(norm_weight), _ptr(a), _ptr(ssq), _stream()))
    return a, ssq


DECODE_PAIR_BLOCKS = 0          # blocks of several waves a (kv head, token) pair in single-token attention: 0 the kernel's own choice, 1 one or the split form
PREFILL_KEY_RANGES = 0          # ranges of keys a prompt portion's attention is divided into: 0 the kernel's own choice, 1 none, n that many


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, H: int, Hkv: int, hd: int,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    page: int, ctx, scale: float, window: int = 0) -> None:
    """Attention of the step's tokens (q in the first H*hd columns of ``qkv``) over the cache."""
    _dev(qkv, out, k_cache, v_cache, block_table)
    _rows2d(qkv, "qkv")
    _rows2d(out, "out")
    T = qkv.shape[0]
    if out.shape[0] != T or out.shape[1] != H * hd or out.dtype != qkv.dtype:
        raise KernelError(f"paged_attention: out must be [{T}, {H * hd}] of {qkv.dtype}")
    if qkv.shape[1] < H * hd:
        raise KernelError("paged_attention: qkv narrower than the query heads")
    _check_cache(k_cache, v_cache, Hkv, hd, page, qkv.dtype, "paged_attention")
    _i32(block_table, "block_table")
    if block_table.dim() != 2 or block_table.shape[0] < ctx.num_rows:
        raise KernelError("paged_attention: block_table must be [rows, max_blocks]")
    _i32(ctx.row_of_token, "row_of_token", T)
    _i32(ctx.positions, "positions", T)
    _i32(ctx.kv_lens, "kv_lens", ctx.num_rows)
    lib = _lib()
    if qkv.dtype == torch.bfloat16 and lib.ri_attention_decode_supported(H, Hkv, hd, page):
        # matrix-core kernels: rows of one token go to the split-key kernel, longer portions to the
        # tiled one; a mixed step launches both, each leaving the other's rows alone
        # rows of one token: their number (or an upper bound) if the step says so, else whether there are any
        num_single = getattr(ctx, "num_single", None)
        host_q = getattr(ctx, "host_q_lens", None)
        any_single = ctx.max_q_len == 1 or (num_single > 0 if num_single is not None
                                            else host_q is None or any(n == 1 for n in host_q))
        if ctx.max_q_len > 1:
            _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
            _i32(ctx.q_start, "q_start", ctx.num_rows)
            # short portions behind many cached keys: the keys divided between blocks, the
            # ranges' results in a workspace (none where the entry point would not divide them)
            prefix, portion_kv = getattr(ctx, "portion_prefix", None), getattr(ctx, "portion_kv_len", None)
            if prefix is None or not portion_kv:         # a context that does not say: bounds from what it does
                prefix, portion_kv = max(int(ctx.max_kv_len) - int(ctx.max_q_len), 0), int(ctx.max_kv_len)
            # the rows of several tokens, if the step lists them and single tokens take rows too
            listed, n_listed = getattr(ctx, "portion_rows", None), int(getattr(ctx, "num_portion", 0) or 0)
            if listed is None or not any_single or not (0 < n_listed < ctx.num_rows):
                listed, n_listed = None, 0
            else:
                _i32(listed, "portion_rows", n_listed)
            lib.ri_attention_prefill_workspace.restype = ctypes.c_size_t
            need = lib.ri_attention_prefill_workspace(H, Hkv, hd, page, int(window), T, int(prefix),
                                                      int(portion_kv), PREFILL_KEY_RANGES)
            ws = ctx.workspace.get("attn.prefill_ranges", (need + 3) // 4, 1, torch.float32) if need else None
            _check(lib.ri_attention_prefill(
                _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _ptr(k_cache), _ptr(v_cache),
                k_cache.shape[0], page, H, Hkv, hd, _ptr(block_table), block_table.shape[1],
                _ptr(ctx.cu_q), _ptr(ctx.q_start), _ptr(ctx.kv_lens), ctx.num_rows, int(ctx.max_q_len), T,
                ctypes.c_float(scale), int(window), 2 if any_single else 1, int(prefix), int(portion_kv),
                PREFILL_KEY_RANGES, _ptr(ws) if ws is not None else ctypes.c_void_p(0),
                ctypes.c_size_t(need), _ptr(listed) if listed is not None else ctypes.c_void_p(0),
                n_listed, _stream()))
        if any_single:
            rows_only = ctx.max_q_len > 1
            # beside prompt portions: the list of the single tokens, if the step brings one
            single = getattr(ctx, "single_tokens", None) if rows_only else None
            if single is not None:
                _i32(single, "single_tokens", int(getattr(ctx, "num_single", 0) or 0))
            lib.ri_attention_decode_workspace.restype = ctypes.c_size_t
            need = lib.ri_attention_decode_workspace(ctx.num_rows, H, hd, ctx.max_kv_len)
            # (one buffer that grows: its size changes with every key the requests gain)
            ws = ctx.workspace.get("attn.decode_partials", (need + 3) // 4, 1, torch.float32)
            _check(lib.ri_attention_decode(
                _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _ptr(k_cache), _ptr(v_cache),
                k_cache.shape[0], page, H, Hkv, hd, _ptr(block_table), block_table.shape[1],
                _ptr(ctx.row_of_token), _ptr(ctx.positions), _ptr(ctx.kv_lens),
                _ptr(ctx.cu_q) if rows_only else ctypes.c_void_p(0), T, ctx.num_rows, int(ctx.max_kv_len),
                ctypes.c_float(scale), int(window), _ptr(ws), ctypes.c_size_t(ws.numel() * 4),
                int(getattr(ctx, "num_single", 0) or 0), _ptr(single) if single is not None else ctypes.c_void_p(0),
                DECODE_PAIR_BLOCKS, _stream()))
        return
    if qkv.dtype == torch.float32 and ctx.max_q_len == 1 and lib.ri_attention_exact_supported(H, Hkv, hd, page):
        # the exact path, single tokens only: the keys of a token split over waves, and a token's
        # output the same bits as the tiled kernel below gives it beside a prompt portion
        lib.ri_attention_exact_decode_workspace.restype = ctypes.c_size_t
        need = lib.ri_attention_exact_decode_workspace(T, H, hd, int(ctx.max_kv_len))
        ws = ctx.workspace.get("attn.exact_partials", need, 1, torch.float32)
        _check(lib.ri_attention_exact_decode_f32(
            _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _ptr(k_cache), _ptr(v_cache),
            k_cache.shape[0], page, H, Hkv, hd, _ptr(block_table), block_table.shape[1],
            _ptr(ctx.row_of_token), _ptr(ctx.positions), _ptr(ctx.kv_lens), T, int(ctx.max_kv_len),
            ctypes.c_float(scale), int(window), _ptr(ws), ctypes.c_size_t(ws.numel()), _stream()))
        return
    if qkv.dtype == torch.float32 and ctx.max_q_len > 1 and lib.ri_attention_exact_supported(H, Hkv, hd, page):
        # the exact path with prompt portions in the step: keys and values read once a tile of queries
        _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
        _i32(ctx.q_start, "q_start", ctx.num_rows)
        _check(lib.ri_attention_exact_f32(
            _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _ptr(k_cache), _ptr(v_cache),
            k_cache.shape[0], page, H, Hkv, hd, _ptr(block_table), block_table.shape[1],
            _ptr(ctx.cu_q), _ptr(ctx.q_start), _ptr(ctx.kv_lens), ctx.num_rows, T,
            ctypes.c_float(scale), int(window), _stream()))
        return
    _check(lib.ri_attention_generic(
        _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _dt(qkv), _ptr(k_cache), _ptr(v_cache),
        k_cache.shape[0], page, H, Hkv, hd, _ptr(block_table), block_table.shape[1],
        _ptr(ctx.row_of_token), _ptr(ctx.positions), _ptr(ctx.kv_lens), T,
        ctypes.c_float(scale), int(window), _stream()))


def attention_kernel_note(dtype: torch.dtype, H: int, Hkv: int, hd: int, page: int) -> Optional[str]:
    """Why attention with these sizes runs on the plain kernel (one thread a query head and key,
    several times slower) instead of the tiled ones, or None if it does not."""
    lib = _lib()
    if dtype == torch.bfloat16 and not lib.ri_attention_decode_supported(H, Hkv, hd, page):
        why = []
        if hd not in (64, 128):
            why.append(f"head size {hd} (they take 64 and 128)")
        if page % 16:
            why.append(f"pages of {page} tokens (they take multiples of 16: paged_block_size = 16)")
        if Hkv > 0 and H % Hkv == 0 and H // Hkv > 16:
            why.append(f"{H // Hkv} query heads a key/value head (they take up to 16)")
        return "attention runs on the plain kernels, not on the matrix cores: " + ", ".join(why or ["sizes not taken"])
    if dtype == torch.float32 and not lib.ri_attention_exact_supported(H, Hkv, hd, page):
        return (f"32-bit attention runs on the plain kernel: head size {hd} and {H // max(Hkv, 1)} query heads a "
                f"key/value head are beyond what the tiled 32-bit kernels take (128, 32)")
    return None


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _dev(gate_up, out)
    T, two_i = gate_up.shape
    I = two_i // 2
    if two_i != 2 * I or tuple(out.shape) != (T, I) or out.dtype != gate_up.dtype \
            or not gate_up.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"swiglu: want contiguous [{T}, 2I] -> [{T}, I] of one dtype")
    _check(_lib().ri_swiglu(_ptr(gate_up), _ptr(out), _dt(out), T, I, _stream()))


def tile_weight(w: torch.Tensor) -> Optional[torch.Tensor]:
    """A copy of ``w[N, K]`` in the order the weight-streaming kernel reads it:
    ``[N/16][K/32][64 lanes][8]`` with lane ``g * 16 + r`` holding ``w[16 nt + r, 32 ks + 8 g : +8]``.
    None if the shape has no such form (N % 16 or K % 32) or the dtype is not bfloat16."""
    N, K = w.shape
    if w.dtype != torch.bfloat16 or N % 16 or K % 32:
        return None
    return w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(N, K)


def _untiled_to_library(x, w, w_tiled, M: int, fused_activation: bool = False) -> bool:
    """Whether a bfloat16 product of few rows against a weight that has no second copy goes to the
    GEMM library rather than to the few-row kernel's row-major form (16 rows of 64 bytes a load
    instruction, a third slower than the tile order).  Measured, us, few-row kernel / library, at
    1, 8, 16, 32, 64 rows: 6144 x 4096: 15 18 21 23 44 / 11 12 12 13 15; 4096 x 4096: 11 11 13 13
    17 / 12 13 13 10 13; 4096 x 14336: 30 35 39 40 46 / 25 26 27 30 39; 8192 x 28672: 115 132 156
    156 170 / 90 89 91 101 150; gate/up with SwiGLU (the library's product and the activation
    kernel) 14336 x 4096: 54 57 62 77 88 / 63 63 64 58 58; 28672 x 8192: 198 204 222 284 351 / 190
    182 184 179 192."""
    if w_tiled is not None or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    if M >= UNTILED_LIBRARY_MIN_ROWS:
        return True
    return not fused_activation and w.shape[0] * w.shape[1] >= UNTILED_LIBRARY_LARGE


def _skinny_ok(x, w, M, K):
    return (not FORCE_LIBRARY_GEMM and x.dtype == torch.bfloat16 and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


QKV_ROPE_LDS_MIN_ROWS = 33      # the fused q/k/v projection takes the LDS kernel from this many tokens on ...
QKV_ROPE_LDS_MIN_COLUMNS = 4096 # ... and columns (128 blocks of 32; in a step of 64 tokens, us: 6144 columns 28.0 -> 24.8,
                                # 5120: 22.6 -> 20.3, 3072: 13.9 -> 14.9)
QKV_ROPE_LDS_LARGE = 40 << 20   # ... and from 17 tokens on where the weight has this many elements (product alone at 24
                                # rows, us: 12288 x 4096 27.3 -> 23.5, 15360 x 5120 35.9 -> 28.8, 10240 x 8192 49.0 -> 42.4;
                                # 6144 x 4096 15.4 -> 16.3, 5120 x 3072 12.5 -> 12.5)
F32_ROWS_MAX = 64               # the exact path's few-row kernel, 16 rows a pass over the weights
ROWS_LDS_MIN_ROWS = 17          # from here to 64 rows, products whose partial sums a norm adds up take the LDS kernel
ROWS_LDS_WIDE_COLUMNS = 16384   # whole products (no slices of K) take it from this many columns on: the output head, 250 -> 205 us at 64 rows
ROWS_LDS_SWIGLU_MIN_ROWS = 33   # the fused gate/up product only with more rows, and with columns enough for its blocks


def _swiglu_groups(I: int) -> int:
    """Wave groups a block of the LDS kernel for a fused gate/up product of ``I`` columns with more
    than 32 rows (0: the few-row kernel does better).  A block of four groups of two waves owns 32
    columns and one of two groups of four waves 64: either takes the LDS of a whole compute unit,
    so its blocks should be most of 256 and no more; a block of one group of four waves owns 64
    columns and half that LDS, which is the form for more than 256 such blocks.  Measured at 64
    rows, us, few-row kernel / one / two / four groups: I = 8192, K = 2048: 22 / 25 / 22 / 18;
    8192 x 3072: 32 / 36 / 32 / 25; 11008 x 4096: 62 / 52 / 44 / 54; 14336 x 4096: 57 / 56 / 50 /
    58; 13824 x 5120: 83 / 66 / 58 / 71; 28672 x 8192: 194 / 159 / 179 / 208."""
    b64, b32 = (I + 63) // 64, (I + 31) // 32
    if 128 <= b32 <= 256:
        return 4
    if 154 <= b64 <= 256:
        return 2
    if b64 > 256:
        return 1
    return 0


def _rows_ok(x, w, w_tiled, M, N, K, min_rows=None):
    """Whether the kernel that shares a block's activations through LDS takes this product."""
    lo = ROWS_LDS_MIN_ROWS if min_rows is None else min_rows
    return (not FORCE_LIBRARY_GEMM and w_tiled is not None and x.dtype == torch.bfloat16 and lo <= M <= SKINNY_MAX_ROWS and N % 16 == 0
            and K % 32 == 0 and x.stride(0) % 8 == 0 and x.stride(1) == 1 and x.data_ptr() % 16 == 0 and _tiled_ok(w, w_tiled))


def _tiled_ok(w, w_tiled):
    if w_tiled is None:
        return False
    if w_tiled.shape != w.shape or w_tiled.dtype != w.dtype or not w_tiled.is_contiguous() \
            or w_tiled.device != w.device:
        raise KernelError("the tile-ordered copy does not match the weight")
    return True


_LIBRARY_WS = {}
NO_LIBRARY_KERNEL = 2          # ri_gemm_library_bf16: the library offers no kernel, nothing was launched
_LIBRARY_REFUSED = set()       # (N, K, strides, out dtype) for which it said so


def _library_workspace(device) -> torch.Tensor:
    """Device memory the GEMM library may use for split products: one buffer a device, kept."""
    ws = _LIBRARY_WS.get(device)
    if ws is None:
        ws = _LIBRARY_WS[device] = torch.empty(LIBRARY_GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def set_gemm_tuning(on: bool, file: Optional[str] = None) -> None:
    """With tuning on, the first bfloat16 product of more than 64 rows of a (row bucket, N, K) times
    every kernel of the GEMM library that takes the problem and keeps the fastest (about a second a
    shape; row counts share a bucket: the next multiple of 16 up to 256 rows, of 32 up to 512, of 128 up
    to 2,048, of 512 beyond).  The library's own first
    choice is 3-8 % slower than its best for prompt portions of 2,048 rows.  ``file`` keeps the
    choices between processes; by default it lies beside the kernel library.  The first product of a
    shape must not fall into a graph capture (the engine's warm-up pass sees to that)."""
    import os
    lib = _lib()
    if on and file is None:
        file = os.path.join(os.path.dirname(build.lib_path() or build.build()), "gemm_tuned.txt")
    _check(lib.ri_gemm_library_set_tuning(1 if on else 0, file.encode() if (on and file) else None))


def gemm_library_stats():
    """(shapes whose descriptors are kept, times the GEMM library was asked to choose a kernel)."""
    a, b = ctypes.c_int(0), ctypes.c_int(0)
    _check(_lib().ri_gemm_library_stats(ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def gemm_library_reset() -> None:
    """Forget the GEMM library's kept descriptors and untuned kernel choices."""
    _check(_lib().ri_gemm_library_reset())
    _LIBRARY_REFUSED.clear()


def gemm_tuned_shapes() -> int:
    """How many (row bucket, N, K) have a tuned kernel choice so far (made now or read from the file)."""
    return int(_lib().ri_gemm_library_tuned_shapes())


def linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, w_tiled: Optional[torch.Tensor] = None,
           scale=None) -> None:
    """``out[M, N] = x[M, K] @ w[N, K]^T``; ``out`` may be float32 for bfloat16 operands.
    ``w_tiled`` (from ``tile_weight``) is read instead of ``w`` where the kernel has a use for it.
    ``scale = (ssq [M, P], eps)``: the rows of ``x`` are ``(r * w_norm)`` of a norm this product
    finishes: row m of the result is multiplied by ``rsqrt(sum(ssq[m]) / K + eps)`` (few bfloat16
    rows only)."""
    _dev(x, w, out)
    _rows2d(x, "x")
    _rows2d(w, "w")
    _rows2d(out, "out")
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(out.shape) != (M, N) or x.dtype != w.dtype:
        raise KernelError(f"linear: shapes {tuple(x.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)} or dtypes do not fit")
    if M == 0:
        return
    lib = _lib()
    if scale is None and N >= ROWS_LDS_WIDE_COLUMNS and out.dtype in (torch.bfloat16, torch.float32) \
            and out.stride(0) % 4 == 0 and _rows_ok(x, w, w_tiled, M, N, K):
        # 17..64 rows against a very wide matrix (the output head): activations shared through LDS
        _check(lib.ri_gemm_rows_bf16(_ptr(x), x.stride(0), _ptr(w_tiled), _ptr(out), out.stride(0), M, N, K, _dt(out), 0, 1,
                                     ctypes.c_longlong(0), 1, 1, _stream()))
        return
    to_library = scale is None and out.dtype in (torch.bfloat16, torch.float32) and _untiled_to_library(x, w, w_tiled, M) \
        and (N, K, x.stride(0), w.stride(0), out.stride(0), out.dtype) not in _LIBRARY_REFUSED
    if x.dtype == torch.bfloat16 and not to_library:
        if _skinny_ok(x, w, M, K):
            tiled = _tiled_ok(w, w_tiled)
            sq, sp, se = _scale_args(scale, M, "linear")
            _check(lib.ri_gemm_skinny_bf16(_ptr(x), x.stride(0), _ptr(w_tiled if tiled else w), w.stride(0),
                                           _ptr(out), out.stride(0), M, N, K, _dt(out), 0, 1,
                                           ctypes.c_longlong(0), int(tiled), sq, sp, se, _stream()))
            return
    if scale is not None:
        raise KernelError("linear: row factors of a deferred norm go with the few-row bfloat16 kernel only")
    if x.dtype == torch.bfloat16:
        if ((LIBRARY_GEMM_MIN_ROWS and M >= LIBRARY_GEMM_MIN_ROWS) or FORCE_LIBRARY_GEMM or to_library) \
                and out.dtype in (torch.bfloat16, torch.float32):
            shape = (N, K, x.stride(0), w.stride(0), out.stride(0), out.dtype)
            if shape not in _LIBRARY_REFUSED:
                ws = _library_workspace(x.device)
                rc = lib.ri_gemm_library_bf16(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0),
                                              M, N, K, int(out.dtype == torch.float32), _ptr(ws),
                                              ctypes.c_size_t(ws.numel()), _stream())
                if rc == 0:
                    return
                if rc != NO_LIBRARY_KERNEL:
                    _check(rc)
                # the library has nothing for this problem (a K or a row stride that is no multiple of
                # 8, say): this engine's own tiled kernel takes any shape; the library is not asked again
                _LIBRARY_REFUSED.add(shape)
                if to_library and _skinny_ok(x, w, M, K):       # few rows after all: the few-row kernel's row-major form
                    _check(lib.ri_gemm_skinny_bf16(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0),
                                                   M, N, K, _dt(out), 0, 1, ctypes.c_longlong(0), 0,
                                                   ctypes.c_void_p(0), 0, ctypes.c_float(0.0), _stream()))
                    return
    if x.dtype == torch.float32 and out.dtype == torch.float32 and M <= F32_ROWS_MAX and K % 4 == 0 and x.stride(0) % 4 == 0 \
            and w.stride(0) % 4 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0:
        # the exact path with few rows: weights streamed once, the same 64-bit sums as the tiled kernel
        _check(lib.ri_gemm_rows_f32(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), M, N, K, _stream()))
        return
    _check(lib.ri_gemm_tiled(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0),
                             M, N, K, _dt(x), _dt(out), _stream()))


def linear_delta(x: torch.Tensor, w: torch.Tensor, workspace, name: str,
                 w_tiled: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ w^T`` as a residual delta for ``add_rmsnorm``: ``[M, N]`` in the dtype of ``x``, or,
    for few bfloat16 rows and few output columns, a float32 stack ``[P, M, N]`` of partial sums
    over slices of K (so that the product still fills the chip) which the norm adds up."""
    _dev(x, w)
    _rows2d(x, "x")
    _rows2d(w, "w")
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K or x.dtype != w.dtype:
        raise KernelError(f"linear_delta: shapes {tuple(x.shape)} x {tuple(w.shape)}^T or dtypes do not fit")
    lib = _lib()
    if _rows_ok(x, w, w_tiled, M, N, K):
        # 17..64 rows: the kernel that shares the activations of a block through LDS
        parts, groups = ctypes.c_int(0), ctypes.c_int(0)
        _check(lib.ri_gemm_rows_plan(M, N, K, 1, ctypes.byref(parts), ctypes.byref(groups)))
        parts, groups = parts.value, groups.value
        if parts > 1:
            stack = workspace.get(name + ".parts", parts * M, N, torch.float32).view(parts, M, N)
            _check(lib.ri_gemm_rows_bf16(_ptr(x), x.stride(0), _ptr(w_tiled), _ptr(stack), N, M, N, K, F32, 0, parts,
                                         ctypes.c_longlong(M * N), 1, groups, _stream()))
            return stack
    if _skinny_ok(x, w, M, K) and N % 4 == 0 and not _untiled_to_library(x, w, w_tiled, M):
        parts = lib.ri_gemm_skinny_parts(M, N, K)
        if parts > 1:
            tiled = _tiled_ok(w, w_tiled)
            stack = workspace.get(name + ".parts", parts * M, N, torch.float32).view(parts, M, N)
            _check(lib.ri_gemm_skinny_bf16(_ptr(x), x.stride(0), _ptr(w_tiled if tiled else w), w.stride(0),
                                           _ptr(stack), N, M, N, K, F32, 0, parts, ctypes.c_longlong(M * N),
                                           int(tiled), ctypes.c_void_p(0), 0, ctypes.c_float(0.0), _stream()))
            return stack
    out = workspace.get(name, M, N, out_dtype or x.dtype)     # out_dtype: 32-bit sums of a bfloat16 product left unrounded
    linear(x, w, out, w_tiled)
    return out


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor,
                  scratch: Optional[torch.Tensor] = None, w_tiled: Optional[torch.Tensor] = None,
                  scale=None) -> None:
    """``out[M, I] = silu(x @ gate^T) * (x @ up^T)`` with ``w_gate_up = [gate; up]`` stacked
    ``[2I, K]``.  Few bfloat16 rows: one fused kernel; otherwise the product into ``scratch``
    ``[M, 2I]`` and the activation kernel.  ``scale``: see ``linear``."""
    _dev(x, w_gate_up, out)
    _rows2d(x, "x")
    _rows2d(w_gate_up, "w_gate_up")
    _rows2d(out, "out")
    M, K = x.shape
    I = w_gate_up.shape[0] // 2
    if w_gate_up.shape != (2 * I, K) or tuple(out.shape) != (M, I) or x.dtype != w_gate_up.dtype \
            or out.dtype != x.dtype:
        raise KernelError("linear_swiglu: shapes or dtypes do not fit")
    if M == 0:
        return
    groups = _swiglu_groups(I)
    if scale is None and groups and _rows_ok(x, w_gate_up, w_tiled, M, I, K, ROWS_LDS_SWIGLU_MIN_ROWS):
        # many rows and blocks enough for the chip: activations shared through LDS
        _check(_lib().ri_gemm_rows_bf16(_ptr(x), x.stride(0), _ptr(w_tiled), _ptr(out), out.stride(0), M, I, K, BF16, 1, 1,
                                        ctypes.c_longlong(0), 1, groups, _stream()))
        return
    if _skinny_ok(x, w_gate_up, M, K) and not (scale is None and scratch is not None and tuple(scratch.shape) == (M, 2 * I)
                                              and _untiled_to_library(x, w_gate_up, w_tiled, M, fused_activation=True)):
        tiled = _tiled_ok(w_gate_up, w_tiled) and I % 16 == 0
        sq, sp, se = _scale_args(scale, M, "linear_swiglu")
        _check(_lib().ri_gemm_skinny_bf16(_ptr(x), x.stride(0), _ptr(w_tiled if tiled else w_gate_up),
                                          w_gate_up.stride(0), _ptr(out), out.stride(0), M, I, K, BF16, 1, 1,
                                          ctypes.c_longlong(0), int(tiled), sq, sp, se, _stream()))
        return
    if scale is not None:
        raise KernelError("linear_swiglu: row factors of a deferred norm go with the few-row bfloat16 kernel only")
    if scratch is None or tuple(scratch.shape) != (M, 2 * I):
        raise KernelError("linear_swiglu: needs scratch [M, 2I] for this size")
    linear(x, w_gate_up, scratch)
    swiglu(scratch, out)


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    _dev(logits, out)
    _rows2d(logits, "logits")
    R, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("argmax: logits must be float32")
    _i32(out, "out", R)
    lib = _lib()
    need = 2 * R * lib.ri_argmax_slices(V)
    key = (logits.device, "argmax")
    scratch = _SCRATCH.get(key)
    if scratch is None or scratch.numel() < need:
        scratch = torch.empty(max(need, 8192), dtype=torch.int32, device=logits.device)
        _SCRATCH[key] = scratch
    _check(lib.ri_argmax(_ptr(logits), R, V, logits.stride(0), _ptr(out), _ptr(scratch), _stream()))


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, draws: torch.Tensor, out: torch.Tensor,
           logprobs: Optional[torch.Tensor] = None, top_ids: Optional[torch.Tensor] = None,
           top_logprobs: Optional[torch.Tensor] = None, want_top: Optional[torch.Tensor] = None) -> None:
    """One token per row of ``logits``: greedy where temperature is 0, else a draw from the
    filtered softmax with the row's uniform number ``draws`` (float64 in [0, 1)).
    ``logprobs`` (float32 [R]) takes ln p of the chosen token among the kept ones (greedy rows:
    log-softmax of the raw logits); ``top_ids`` / ``top_logprobs`` (int32 / float32 [R, 5]) the five
    most probable kept tokens of the rows whose ``want_top`` (int32 [R], all if None) is not 0,
    -1 / -inf where there are none."""
    _dev(logits, temperature, top_k, top_p, min_p, draws, out, logprobs, top_ids, top_logprobs, want_top)
    _rows2d(logits, "logits")
    R, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p"), (min_p, torch.float32, "min_p"),
                        (draws, torch.float64, "draws"), (out, torch.int32, "out")):
        if t.dtype != dt or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be contiguous {dt} with {R} entries")
    if (top_ids is None) != (top_logprobs is None):
        raise KernelError("sample: top_ids and top_logprobs come together")
    for t, dt, n, name in ((logprobs, torch.float32, R, "logprobs"), (top_ids, torch.int32, 5 * R, "top_ids"),
                           (top_logprobs, torch.float32, 5 * R, "top_logprobs"), (want_top, torch.int32, R, "want_top")):
        if t is not None and (t.dtype != dt or t.numel() < n or not t.is_contiguous()):
            raise KernelError(f"sample: {name} must be contiguous {dt} with {n} entries")
    lib = _lib()
    lib.ri_sample_scratch_bytes.restype = ctypes.c_size_t
    need = lib.ri_sample_scratch_bytes(R, V)
    key = (logits.device, "sample")
    scratch = _SCRATCH.get(key)
    if scratch is None or scratch.numel() * 8 < need:
        scratch = torch.empty((need + 7) // 8, dtype=torch.int64, device=logits.device)
        _SCRATCH[key] = scratch
    _check(lib.ri_sample(_ptr(logits), R, V, logits.stride(0), _ptr(temperature), _ptr(top_k),
                         _ptr(top_p), _ptr(min_p), _ptr(draws), _ptr(out), _ptr(scratch),
                         ctypes.c_size_t(scratch.numel() * 8), _ptr(logprobs), _ptr(top_ids),
                         _ptr(top_logprobs), _ptr(want_top), _stream()))


def measure_peaks(device="cuda:0", read_bytes: int = 4 << 30, reps: int = 5):
    """What the GPU reaches with nothing in the way, measured now: GB/s of a kernel that only reads
    ``read_bytes`` of device memory and of one that copies it (bytes read plus bytes written),
    TFLOP/s of a loop of bfloat16 matrix instructions on registers and of a loop of 32-bit FMAs
    (this library is compiled without packed 32-bit instructions, which halves that figure).
    Returns ``{"hbm_read_gbs", "hbm_copy_gbs", "mfma_bf16_tflops", "fma_f32_tflops"}``."""
    dev = torch.device(device)
    lib = _lib()
    buf = torch.empty(read_bytes, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).fill_(0x01020304)
    sink = torch.zeros(4096, dtype=torch.int32, device=dev)
    out = {}
    with torch.cuda.device(dev):
        for what, name, unit in ((0, "hbm_read_gbs", 1e9), (1, "hbm_copy_gbs", 1e9),
                                 (2, "mfma_bf16_tflops", 1e12), (3, "fma_f32_tflops", 1e12)):
            work = ctypes.c_double(0.0)
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            args = (what, _ptr(buf), ctypes.c_size_t(buf.numel()), _ptr(sink))
            _check(lib.ri_measure_peak(*args, 2, ctypes.byref(work), stream))          # warm-up
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _check(lib.ri_measure_peak(*args, reps, ctypes.byref(work), stream))
            e1.record()
            e1.synchronize()
            out[name] = round(work.value * reps / (e0.elapsed_time(e1) * 1e-3) / unit, 1)
    return out


# ---------------------------------------------------------------------------
# elementwise functions on columns of a wider buffer, the output head's soft cap
# ---------------------------------------------------------------------------
UNARY = {"relu2": 0, "tanh": 1}


def unary(name: str, x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = f(x)`` for ``f`` in ``UNARY`` (the square of relu, tanh), 32-bit arithmetic; ``x`` and
    ``out`` are ``[T, n]`` with unit column stride and any row stride (``out`` may be ``x``)."""
    _dev(x, out)
    _rows2d(x, "x")
    _rows2d(out, "out")
    if name not in UNARY or x.shape != out.shape or x.dtype != out.dtype:
        raise KernelError(f"unary: unknown function {name!r}, or shapes / dtypes differ")
    T, n = x.shape
    _check(_lib().ri_unary(_ptr(x), x.stride(0), _ptr(out), out.stride(0), _dt(x), T, n, UNARY[name], _stream()))


def scale_softcap(logits: torch.Tensor, scale: float, cap: float) -> None:
    """``logits <- cap * tanh(logits * scale / cap)`` in place (``cap <= 0``: the scale alone)."""
    _dev(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
        raise KernelError("scale_softcap: logits must be contiguous float32 [rows, vocab]")
    _check(_lib().ri_scale_softcap(_ptr(logits), logits.shape[0], logits.shape[1], ctypes.c_float(scale),
                                   ctypes.c_float(cap), _stream()))


# ---------------------------------------------------------------------------
# attention with key and value heads of different sizes, a window and turned values
# ---------------------------------------------------------------------------
def _rot_tables(tables, size: int, who: str):
    """(cos, sin, rows) pointers of a rotation's tables ``[positions, size / 2]``, or nulls."""
    if tables is None:
        return ctypes.c_void_p(0), ctypes.c_void_p(0), 0
    cos, sin = tables[0], tables[1]
    _dev(cos, sin)
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2 \
            or cos.shape[1] * 2 != size or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError(f"{who}: cos/sin must be contiguous float32 [positions, {size // 2}]")
    return _ptr(cos), _ptr(sin), cos.shape[0]


def _check_cache_kv(k_cache, v_cache, Hkv, dk, dv, page, act_dtype, name):
    if k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (Hkv, page, dk) or v_cache.dim() != 4 \
            or tuple(v_cache.shape) != (k_cache.shape[0], Hkv, dv, page):
        raise KernelError(f"{name}: caches must be k [pages, {Hkv}, {page}, {dk}] and v [pages, {Hkv}, {dv}, {page}], "
                          f"got {tuple(k_cache.shape)} and {tuple(v_cache.shape)}")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise KernelError(f"{name}: cache must be contiguous")
    if k_cache.dtype != act_dtype or v_cache.dtype != act_dtype:
        raise KernelError(f"{name}: cache dtype {k_cache.dtype} differs from the activations' {act_dtype}")


def rotate_kv_write(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], H: int, Hkv: int,
                    dk: int, dv: int, rotary, value_rotary, positions: torch.Tensor, row_of_token: torch.Tensor,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, page: int,
                    write_kv: bool = True, interleaved_values: bool = False, unit_eps: float = 0.0) -> None:
    """``unit_eps > 0``: every head of q and k is also divided by ``sqrt(mean(.^2) + unit_eps)`` (a rotation
    leaves that mean as it is, so it does not matter on which side of it the division stands).
    Rotate ``q [T, H dk]`` in place (``rotary = (cos, sin, rot_dim)``: the first ``rot_dim``
    features of a head, feature i with i + rot_dim/2) and write this step's keys (rotated the same
    way) and values into their pages.  ``value_rotary = (cos, sin)`` ``[positions, dv/2]``: a value
    is cached turned by its position over all its features, pair m = (m, m + dv/2), or
    (2m, 2m + 1) with ``interleaved_values``.  q, k, v may be columns of one wider buffer."""
    _dev(q, k, v, positions, row_of_token, k_cache, v_cache, block_table)
    _rows2d(q, "q")
    T = q.shape[0]
    if q.shape[1] != H * dk:
        raise KernelError(f"rotate_kv_write: q must be [T, {H * dk}]")
    _i32(positions, "positions", T)
    _i32(row_of_token, "row_of_token", T)
    rot = 0
    cos = sin = ctypes.c_void_p(0)
    rows = 0
    if rotary is not None:
        rot = int(rotary[2])
        cos, sin, rows = _rot_tables(rotary, rot, "rotate_kv_write")
    vcos, vsin, vrows = _rot_tables(value_rotary, dv, "rotate_kv_write (values)")
    if write_kv:
        _rows2d(k, "k")
        _rows2d(v, "v")
        if tuple(k.shape) != (T, Hkv * dk) or tuple(v.shape) != (T, Hkv * dv) or k.dtype != q.dtype or v.dtype != q.dtype:
            raise KernelError(f"rotate_kv_write: k must be [T, {Hkv * dk}] and v [T, {Hkv * dv}] of {q.dtype}")
        _check_cache_kv(k_cache, v_cache, Hkv, dk, dv, page, q.dtype, "rotate_kv_write")
        _i32(block_table, "block_table")
        if block_table.dim() != 2:
            raise KernelError("rotate_kv_write: block_table must be [rows, max_blocks]")
    _check(_lib().ri_rotate_kv_write(
        _ptr(q), q.stride(0), _ptr(k), k.stride(0) if k is not None else 0, _ptr(v), v.stride(0) if v is not None else 0,
        _dt(q), T, H, Hkv, dk, dv, rot, cos, sin, rows, vcos, vsin, vrows, int(bool(interleaved_values)),
        _ptr(positions), _ptr(row_of_token), _ptr(k_cache), _ptr(v_cache),
        k_cache.shape[0] if k_cache is not None else 0, _ptr(block_table),
        block_table.shape[1] if block_table is not None and block_table.dim() == 2 else 0, page,
        int(bool(write_kv)), ctypes.c_float(unit_eps), _stream()))


WINDOW_ATTENTION_MFMA = True     # steps with prompt portions take the matrix-instruction kernel (False: the FMA one, for comparison)


def window_attention_supported(H: int, Hkv: int, dk: int, dv: int) -> bool:
    return bool(_lib().ri_attention_window_supported(H, Hkv, dk, dv))


def window_attention(q: torch.Tensor, out: torch.Tensor, H: int, Hkv: int, dk: int, dv: int,
                     k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, page: int,
                     ctx, scale: float, window: int = 0, value_rotary=None,
                     interleaved_values: bool = False, sink: Optional[torch.Tensor] = None,
                     keep_first: int = 0, sigmoid_bias: Optional[torch.Tensor] = None) -> None:
    """Attention of the step's tokens (rotated queries ``q [T, H dk]``) over the cache into
    ``out [T, H dv]``: keys of size ``dk``, values of size ``dv``, the last ``window`` positions
    (0: all).  ``value_rotary``: the cached values are turned by their positions, and each sum is
    turned back by its query's.  ``sink`` (32-bit, one number a query head): ``exp(sink_h)`` joins the
    softmax's denominator, with no key and no value.  ``keep_first``: with a window, the first so many
    positions of a request stay in sight of every later query.  ``sigmoid_bias`` (32-bit, one number a
    query head): no softmax; a visible key's weight is ``sigmoid(score + sigmoid_bias[h])``, and the
    weights are not normalised over the keys."""
    _dev(q, out, k_cache, v_cache, block_table, sink, sigmoid_bias)
    _f32_vec(sink, H, "window_attention: the sink")
    _f32_vec(sigmoid_bias, H, "window_attention: the sigmoids' bias")
    if sink is not None and sigmoid_bias is not None:
        raise KernelError("window_attention: sigmoid weights take no sink")
    keep_first = int(keep_first) if window else 0
    _rows2d(q, "q")
    _rows2d(out, "out")
    T = q.shape[0]
    if q.shape[1] != H * dk or tuple(out.shape) != (T, H * dv) or out.dtype != q.dtype:
        raise KernelError(f"window_attention: q must be [T, {H * dk}] and out [T, {H * dv}] of one dtype")
    _check_cache_kv(k_cache, v_cache, Hkv, dk, dv, page, q.dtype, "window_attention")
    _i32(block_table, "block_table")
    if block_table.dim() != 2 or block_table.shape[0] < ctx.num_rows:
        raise KernelError("window_attention: block_table must be [rows, max_blocks]")
    _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
    _i32(ctx.q_start, "q_start", ctx.num_rows)
    _i32(ctx.kv_lens, "kv_lens", ctx.num_rows)
    vcos, vsin, vrows = _rot_tables(value_rotary, dv, "window_attention (values)")
    lib = _lib()
    if ctx.max_q_len > 1 and WINDOW_ATTENTION_MFMA and lib.ri_attention_window_mfma_supported(H, Hkv, dk, dv):
        # steps with prompt portions: both products on the 32-bit matrix instructions
        _check(lib.ri_attention_window_mfma(
            _ptr(q), q.stride(0), _ptr(out), out.stride(0), _dt(q), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], page,
            H, Hkv, dk, dv, _ptr(block_table), block_table.shape[1], _ptr(ctx.cu_q), _ptr(ctx.q_start), _ptr(ctx.kv_lens),
            ctx.num_rows, T, ctypes.c_float(scale), int(window), vcos, vsin, vrows, int(bool(interleaved_values)), _ptr(sink),
            keep_first, _ptr(sigmoid_bias), _stream()))
        return
    # a step of single tokens divides each row's keys between blocks, through a workspace
    single, ws, need = int(ctx.max_q_len == 1 and T <= ctx.num_rows), None, 0
    if single:
        lib.ri_attention_window_workspace.restype = ctypes.c_size_t
        need = lib.ri_attention_window_workspace(T, H, dk, dv, int(window), int(ctx.max_kv_len), keep_first)
        if need:
            ws = ctx.workspace.get("attn.window_partials", need, 1, torch.float32)
    _check(lib.ri_attention_window(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _dt(q), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], page,
        H, Hkv, dk, dv, _ptr(block_table), block_table.shape[1], _ptr(ctx.cu_q), _ptr(ctx.q_start), _ptr(ctx.kv_lens),
        ctx.num_rows, T, ctypes.c_float(scale), int(window), vcos, vsin, vrows, int(bool(interleaved_values)),
        single, int(ctx.max_kv_len), _ptr(ws), ctypes.c_size_t(need), _ptr(sink), keep_first, _ptr(sigmoid_bias), _stream()))


# ---------------------------------------------------------------------------
# mixers with a matrix of state for each head
# ---------------------------------------------------------------------------
def linear_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, out: torch.Tensor, ctx,
                H: int, dk: int, dv: int, decay: Optional[torch.Tensor] = None, silu_in: bool = False,
                wl: Optional[torch.Tensor] = None, al: Optional[torch.Tensor] = None,
                w0: Optional[torch.Tensor] = None, ab: Optional[torch.Tensor] = None,
                unit_eps: float = 1e-6, decay_c: float = 1.0, rotary=None, k_scale: float = 1.0) -> None:
    """Walk each request's tokens of the step through its state ``state[slot] [H, dk, dv]`` (32-bit):
    ``S <- diag(w) S - (a u)(u^T S) + k v^T``, ``out_t = S^T r`` (32-bit ``[T, H dv]``).
    With ``decay [H]``: ``w`` is the head's constant, no second term, and r, k, v pass through silu if
    ``silu_in``.  With ``wl, al [T, H dk]`` and 32-bit ``w0, ab [H dk]``: ``u = k / sqrt(|k|^2 + unit_eps)``,
    ``w = exp(-decay_c sigmoid(wl + w0))``, ``a = sigmoid(al + ab)``.  A request's first tokens
    (``q_start == 0``) start from zeros.  Decay form only: ``rotary = (cos, sin, rot_dim)`` turns r and
    k by the token's position over their first ``rot_dim`` features (feature i with i + rot_dim/2), in
    32-bit, and ``k_scale`` multiplies k after that."""
    _dev(r, k, v, state, out, decay, wl, al, w0, ab)
    for t, name in ((r, "r"), (k, "k"), (v, "v"), (out, "out")):
        _rows2d(t, name)
    T = r.shape[0]
    delta = decay is None
    if tuple(r.shape) != (T, H * dk) or tuple(k.shape) != (T, H * dk) or tuple(v.shape) != (T, H * dv) \
            or tuple(out.shape) != (T, H * dv) or out.dtype != torch.float32 or k.dtype != r.dtype or v.dtype != r.dtype:
        raise KernelError("linear_scan: r, k [T, H dk], v [T, H dv] of one dtype and 32-bit out [T, H dv] expected")
    if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (H, dk, dv) or not state.is_contiguous():
        raise KernelError(f"linear_scan: state must be contiguous float32 [slots, {H}, {dk}, {dv}]")
    if delta:
        for t, name in ((wl, "wl"), (al, "al")):
            if t is None or tuple(t.shape) != (T, H * dk) or t.dtype != r.dtype or t.stride(1) != 1:
                raise KernelError(f"linear_scan: {name} must be [T, {H * dk}] of {r.dtype}")
        for t, name in ((w0, "w0"), (ab, "ab")):
            if t is None or t.dtype != torch.float32 or t.numel() != H * dk or not t.is_contiguous():
                raise KernelError(f"linear_scan: {name} must be contiguous float32 with {H * dk} entries")
    elif decay.dtype != torch.float32 or decay.numel() != H or not decay.is_contiguous():
        raise KernelError(f"linear_scan: decay must be contiguous float32 with {H} entries")
    _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
    _i32(ctx.q_start, "q_start", ctx.num_rows)
    _i32(ctx.state_slots, "state_slots", ctx.num_rows)
    rot, rcos, rsin, rrows = 0, ctypes.c_void_p(0), ctypes.c_void_p(0), 0
    if rotary is not None:
        rot = int(rotary[2])
        rcos, rsin, rrows = _rot_tables(rotary, rot, "linear_scan")
    _check(_lib().ri_linear_scan(
        _ptr(r), r.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0),
        _ptr(wl), wl.stride(0) if wl is not None else 0, _ptr(al), al.stride(0) if al is not None else 0, _dt(r),
        _ptr(w0), _ptr(ab), _ptr(decay), int(delta), int(bool(silu_in)), ctypes.c_float(unit_eps),
        ctypes.c_float(decay_c), _ptr(state), state.shape[0], _ptr(out), out.stride(0),
        _ptr(ctx.cu_q), _ptr(ctx.q_start), _ptr(ctx.state_slots), ctx.num_rows, T, H, dk, dv,
        rcos, rsin, rot, rrows, max(int(ctx.max_kv_len) - 1, 0), ctypes.c_float(k_scale), _stream()))


def gated_group_norm(o: torch.Tensor, weight: Optional[torch.Tensor], gate: Optional[torch.Tensor], out: torch.Tensor,
                     group: int, eps: float, gate_activation: str = "sigmoid", gate_first: bool = False) -> None:
    """``out = o / sqrt(mean over each group of `group` features (o^2) + eps) * weight * sigmoid(gate)``;
    ``o`` 32-bit ``[T, n]``, ``gate`` and ``out`` activations (columns of wider buffers allowed).
    ``weight = None``: no weight; ``gate_activation = "silu"``: ``silu(gate)`` in place of the sigmoid.
    ``gate_first``: the gate multiplies ``o`` before the norm, ``out = norm(o * act(gate)) * weight``."""
    _dev(o, weight, gate, out)
    _rows2d(o, "o")
    _rows2d(out, "out")
    T, n = o.shape
    if o.dtype != torch.float32 or tuple(out.shape) != (T, n) or (weight is not None and (weight.numel() != n or not weight.is_contiguous())):
        raise KernelError("gated_group_norm: 32-bit o [T, n], out [T, n] and n weights expected")
    if gate_activation not in ("sigmoid", "silu"):
        raise KernelError(f"gated_group_norm: unknown gate activation {gate_activation!r}")
    if gate is not None:
        _rows2d(gate, "gate")
        if tuple(gate.shape) != (T, n) or gate.dtype != out.dtype:
            raise KernelError("gated_group_norm: gate must be [T, n] in the dtype of out")
    _check(_lib().ri_gated_group_norm(_ptr(o), o.stride(0), T, n, int(group), _ptr(weight),
                                      _dt(weight) if weight is not None else F32, _ptr(gate),
                                      gate.stride(0) if gate is not None else 0, _ptr(out), out.stride(0), _dt(out),
                                      ctypes.c_float(eps), int(gate_activation == "silu"), int(bool(gate_first)), _stream()))


# ---------------------------------------------------------------------------
# what some attention mixers do head by head between their projections and attention
# ---------------------------------------------------------------------------
def _f32_vec(t: Optional[torch.Tensor], n: int, who: str):
    if t is not None and (t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous()):
        raise KernelError(f"{who}: must be contiguous float32 with {n} entries")


def head_norm_kv_write(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], H: int, Hkv: int,
                       dk: int, dv: int, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                       eps: float, positions: torch.Tensor, row_of_token: torch.Tensor, k_cache: torch.Tensor,
                       v_cache: torch.Tensor, block_table: torch.Tensor, page: int, write_kv: bool = True,
                       norm: bool = True, temp_coef: float = 0.0, temp_every: int = 0) -> None:
    """Every head of ``q [T, H dk]`` and ``k [T, Hkv dk]`` divided by its root mean square
    (``norm``), times a 32-bit weight of ``dk`` entries shared by the heads (or None); the query at
    position p also times ``1 + temp_coef ln(floor((p + 1) / temp_every) + 1)`` (``temp_every > 0``).
    q in place; k and ``v [T, Hkv dv]`` go into the token's page (``write_kv``)."""
    _dev(q, k, v, q_weight, k_weight, positions, row_of_token, k_cache, v_cache, block_table)
    _rows2d(q, "q")
    T = q.shape[0]
    if q.shape[1] != H * dk:
        raise KernelError(f"head_norm_kv_write: q must be [T, {H * dk}]")
    _i32(positions, "positions", T)
    _i32(row_of_token, "row_of_token", T)
    _f32_vec(q_weight, dk, "head_norm_kv_write: the query weight")
    _f32_vec(k_weight, dk, "head_norm_kv_write: the key weight")
    if write_kv:
        _rows2d(k, "k")
        _rows2d(v, "v")
        if tuple(k.shape) != (T, Hkv * dk) or tuple(v.shape) != (T, Hkv * dv) or k.dtype != q.dtype or v.dtype != q.dtype:
            raise KernelError(f"head_norm_kv_write: k must be [T, {Hkv * dk}] and v [T, {Hkv * dv}] of {q.dtype}")
        _check_cache_kv(k_cache, v_cache, Hkv, dk, dv, page, q.dtype, "head_norm_kv_write")
        _i32(block_table, "block_table")
        if block_table.dim() != 2:
            raise KernelError("head_norm_kv_write: block_table must be [rows, max_blocks]")
    _check(_lib().ri_head_norm_kv_write(
        _ptr(q), q.stride(0), _ptr(k) if write_kv else ctypes.c_void_p(0), k.stride(0) if write_kv else 0,
        _ptr(v) if write_kv else ctypes.c_void_p(0), v.stride(0) if write_kv else 0, _dt(q), T, H, Hkv, dk, dv,
        _ptr(q_weight), _ptr(k_weight), int(bool(norm)), ctypes.c_float(eps), ctypes.c_float(temp_coef), int(temp_every),
        _ptr(positions), _ptr(row_of_token), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0] if k_cache is not None else 0,
        _ptr(block_table), block_table.shape[1] if block_table is not None and block_table.dim() == 2 else 0, page,
        int(bool(write_kv)), _stream()))


def latent_kv_write(q: torch.Tensor, down: torch.Tensor, q_abs: torch.Tensor, H: int, d: int, r: int, R: int,
                    latent_weight: Optional[torch.Tensor], eps: float, rotary, positions: torch.Tensor,
                    row_of_token: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, page: int, write_kv: bool = True) -> None:
    """Attention through a latent: ``down [T, R + r]`` holds the latent's R features, which are divided
    by their root mean square and multiplied by ``latent_weight`` (32-bit), and one rotated key part of
    r features; the page (one key/value head) takes the key ``[latent, turned part]`` and the value
    ``latent``.  ``q [T, H (d + r)]``: the turned rotated part of every head's query goes to the last r
    columns of that head in ``q_abs [T, H (R + r)]``.  ``rotary = (cos, sin, rot)`` turns the first
    ``rot`` features of a rotated part (feature i with i + rot/2)."""
    _dev(q, down, q_abs, latent_weight, positions, row_of_token, k_cache, v_cache, block_table)
    for t, name in ((q, "q"), (down, "down"), (q_abs, "q_abs")):
        _rows2d(t, name)
    T = q.shape[0]
    if q.shape[1] != H * (d + r) or tuple(down.shape) != (T, R + r) or tuple(q_abs.shape) != (T, H * (R + r)) \
            or down.dtype != q.dtype or q_abs.dtype != q.dtype:
        raise KernelError(f"latent_kv_write: q [T, {H * (d + r)}], down [T, {R + r}] and q_abs [T, {H * (R + r)}] of one dtype expected")
    _i32(positions, "positions", T)
    _i32(row_of_token, "row_of_token", T)
    _f32_vec(latent_weight, R, "latent_kv_write: the latent's weight")
    rot, cos, sin, rows = 0, ctypes.c_void_p(0), ctypes.c_void_p(0), 0
    if rotary is not None:
        rot = int(rotary[2])
        cos, sin, rows = _rot_tables(rotary, rot, "latent_kv_write")
    if write_kv:
        _check_cache_kv(k_cache, v_cache, 1, R + r, R, page, q.dtype, "latent_kv_write")
        _i32(block_table, "block_table")
        if block_table.dim() != 2:
            raise KernelError("latent_kv_write: block_table must be [rows, max_blocks]")
    _check(_lib().ri_latent_kv_write(
        _ptr(q), q.stride(0), _ptr(down), down.stride(0), _ptr(q_abs), q_abs.stride(0), _dt(q), T, H, d, r, R, rot,
        _ptr(latent_weight), ctypes.c_float(eps), cos, sin, rows, _ptr(positions), _ptr(row_of_token),
        _ptr(k_cache), _ptr(v_cache), k_cache.shape[0] if k_cache is not None else 0, _ptr(block_table),
        block_table.shape[1] if block_table is not None and block_table.dim() == 2 else 0, page, int(bool(write_kv)), _stream()))


def head_linear(x: torch.Tensor, x_head: int, w: torch.Tensor, out: torch.Tensor, out_head: int) -> None:
    """``out[t, h * out_head : + N] = w[h] @ x[t, h * x_head : + K]`` for every head h; ``w [H, N, K]``.
    x and out are 2-D with unit column stride (columns of wider buffers allowed); 32-bit sums."""
    _dev(x, w, out)
    _rows2d(x, "x")
    _rows2d(out, "out")
    if w.dim() != 3 or not w.is_contiguous() or w.dtype != x.dtype or out.dtype != x.dtype or out.shape[0] != x.shape[0]:
        raise KernelError("head_linear: w must be contiguous [H, N, K] in the dtype of x and out")
    H, N, K = w.shape
    if x.shape[1] < (H - 1) * x_head + K or out.shape[1] < (H - 1) * out_head + N:
        raise KernelError("head_linear: x or out is narrower than its heads")
    _check(_lib().ri_head_linear(_ptr(x), x.stride(0), int(x_head), _ptr(w), _ptr(out), out.stride(0), int(out_head),
                                 _dt(x), x.shape[0], H, N, K, _stream()))


# ---------------------------------------------------------------------------
# a feed-forward of many experts
# ---------------------------------------------------------------------------
def _score_kind(score: str) -> int:
    if score not in ("softmax", "sigmoid"):
        raise KernelError(f"a router scores with 'softmax' or 'sigmoid', got {score!r}")
    return int(score == "sigmoid")


def _moe_widths(gate_up, act, E: int, F: int, shared: int, who: str):
    """The activations' width: the experts' ``E F`` columns, a shared expert's ``shared`` and zeros up to
    what ``act`` has."""
    T, width = gate_up.shape[0], act.shape[1]
    if gate_up.shape[1] != 2 * E * F + 2 * shared or act.shape[0] != T or width < E * F + shared or act.dtype != gate_up.dtype:
        raise KernelError(f"{who}: gate_up [T, {2 * E * F + 2 * shared}] and act [T, >= {E * F + shared}] of one dtype expected")
    return T, width


def moe_route(logits: torch.Tensor, weights: torch.Tensor, top: int, renormalize: bool = False,
              score: str = "softmax", norm_eps: float = 0.0, scale: float = 1.0) -> None:
    """``weights [T, E]`` (32-bit): ``softmax(logits)`` at the ``top`` largest entries of every row (ties:
    the lower index), 0 elsewhere; ``renormalize`` divides them by their sum (+ ``norm_eps``).
    ``score = "sigmoid"``: the scores are ``sigmoid(logits)``, each on its own; ``scale`` multiplies the weights."""
    _dev(logits, weights)
    _rows2d(logits, "logits")
    T, E = logits.shape
    if logits.dtype != torch.float32 or weights.dtype != torch.float32 or tuple(weights.shape) != (T, E) or not weights.is_contiguous():
        raise KernelError("moe_route: 32-bit logits [T, E] and contiguous 32-bit weights [T, E] expected")
    _check(_lib().ri_moe_route_as(_ptr(logits), logits.stride(0), _ptr(weights), T, E, int(top), int(bool(renormalize)),
                                  _score_kind(score), ctypes.c_float(norm_eps), ctypes.c_float(scale), _stream()))


def moe_swiglu_weighted(gate_up: torch.Tensor, weights: torch.Tensor, act: torch.Tensor, E: int, F: int,
                        shared: int = 0) -> None:
    """``act[t, e F + i] = weights[t, e] * silu(gate_up[t, e 2F + i]) * gate_up[t, e 2F + F + i]``.
    ``shared`` > 0: ``gate_up`` has ``2 shared`` more columns, a shared expert's gate and up, and ``act`` gets
    ``silu(gate) * up`` of them behind the experts' columns (weight 1); wider ``act``: zeros beyond."""
    _dev(gate_up, weights, act)
    _rows2d(gate_up, "gate_up")
    _rows2d(act, "act")
    T, width = _moe_widths(gate_up, act, E, F, shared, "moe_swiglu_weighted")
    if weights.dtype != torch.float32 or tuple(weights.shape) != (T, E) or not weights.is_contiguous():
        raise KernelError("moe_swiglu_weighted: contiguous 32-bit weights [T, E] expected")
    _check(_lib().ri_moe_swiglu_weighted_shared(_ptr(gate_up), gate_up.stride(0), _ptr(weights), _ptr(act), act.stride(0),
                                                _dt(act), T, E, F, int(shared), width, _stream()))


def moe_swiglu_routed(gate_up: torch.Tensor, logits: torch.Tensor, act: torch.Tensor, E: int, F: int, top: int,
                      renormalize: bool = False, score: str = "softmax", norm_eps: float = 0.0, scale: float = 1.0,
                      shared: int = 0) -> None:
    """``moe_route`` and ``moe_swiglu_weighted`` in one launch: the weights are made from the 32-bit
    ``logits [T, E]`` on the way and never stored."""
    _dev(gate_up, logits, act)
    _rows2d(gate_up, "gate_up")
    _rows2d(act, "act")
    _rows2d(logits, "logits")
    T, width = _moe_widths(gate_up, act, E, F, shared, "moe_swiglu_routed")
    if logits.dtype != torch.float32 or tuple(logits.shape) != (T, E):
        raise KernelError("moe_swiglu_routed: 32-bit logits [T, E] expected")
    _check(_lib().ri_moe_swiglu_routed_as(_ptr(gate_up), gate_up.stride(0), _ptr(logits), logits.stride(0), _ptr(act),
                                          act.stride(0), _dt(act), T, E, F, int(top), int(bool(renormalize)),
                                          _score_kind(score), ctypes.c_float(norm_eps), ctypes.c_float(scale),
                                          int(shared), width, _stream()))


# ---------------------------------------------------------------------------
# layer norm around gated sub-layers, a feed-forward that norms powers, a short convolution, the gated delta rule
# ---------------------------------------------------------------------------
def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out: torch.Tensor,
               rows: Optional[torch.Tensor] = None) -> None:
    """``out = (x - mean) / sqrt(var + eps) * weight + bias`` row by row; ``x`` 32-bit ``[T, d]``; with
    ``rows`` (int32) only those rows, in that order."""
    _dev(x, weight, bias, out, rows)
    T, d = x.shape
    n_out = rows.numel() if rows is not None else T
    if rows is not None:
        _i32(rows, "rows")
    if x.dtype != torch.float32 or not x.is_contiguous() or tuple(out.shape) != (n_out, d) or not out.is_contiguous():
        raise KernelError(f"layer_norm: contiguous 32-bit x [T, d] and contiguous out [{n_out}, {d}] expected")
    _f32_vec(weight, d, "layer_norm: the weight")
    _f32_vec(bias, d, "layer_norm: the bias")
    _check(_lib().ri_layer_norm(_ptr(x), _ptr(rows), _ptr(weight), _ptr(bias), ctypes.c_float(eps), _ptr(out), _dt(out),
                                n_out, d, _stream()))


def gated_norm_residual(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
                        gate: Optional[torch.Tensor] = None, gate_bias: Optional[torch.Tensor] = None,
                        delta_bias: Optional[torch.Tensor] = None, next_norm=None,
                        next_out: Optional[torch.Tensor] = None) -> None:
    """``y = (delta + delta_bias) * sigmoid(gate + gate_bias)``; ``x += layer_norm(y) * weight + bias``, in
    place on the 32-bit stream.  ``delta`` is ``[T, d]`` or a 32-bit stack ``[P, T, d]`` of partial sums;
    ``gate [T, d]`` may be columns of a wider buffer.  ``next_norm = (weight, bias)`` with ``next_out``
    ``[T, d]``: the layer norm of the new ``x`` is left there in the same pass."""
    _dev(x, delta, weight, bias, gate, gate_bias, delta_bias, next_out)
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("gated_norm_residual: x must be contiguous float32")
    parts, stride = 1, 0
    if delta.dim() == 3:
        parts, stride = delta.shape[0], delta.stride(0)
    if delta.dim() not in (2, 3) or tuple(delta.shape[-2:]) != (T, d) or delta.stride(-1) != 1 or delta.stride(-2) != d \
            or (delta.dim() == 3 and delta.dtype != torch.float32):
        raise KernelError("gated_norm_residual: delta must be [T, d] or a float32 stack [P, T, d] with contiguous rows")
    for v, name in ((weight, "weight"), (bias, "bias"), (gate_bias, "gate bias"), (delta_bias, "delta bias")):
        _f32_vec(v, d, f"gated_norm_residual: the {name}")
    act_dt = _dt(delta) if delta.dtype != torch.float32 else None
    if gate is not None:
        _rows2d(gate, "gate")
        if tuple(gate.shape) != (T, d):
            raise KernelError(f"gated_norm_residual: gate must be [{T}, {d}]")
        act_dt = _dt(gate)
    nw = nb = None
    if next_out is not None:
        nw, nb = next_norm
        _f32_vec(nw, d, "gated_norm_residual: the next norm's weight")
        _f32_vec(nb, d, "gated_norm_residual: the next norm's bias")
        if tuple(next_out.shape) != (T, d) or not next_out.is_contiguous():
            raise KernelError(f"gated_norm_residual: next_out must be contiguous [{T}, {d}]")
        if gate is not None and next_out.dtype != gate.dtype:
            raise KernelError("gated_norm_residual: gate and next_out must have one dtype")
        act_dt = _dt(next_out)
    if act_dt is None:
        act_dt = F32
    _check(_lib().ri_gated_norm_residual(_ptr(x), _ptr(delta), _dt(delta), parts, ctypes.c_longlong(stride), _ptr(delta_bias),
                                         _ptr(gate), gate.stride(0) if gate is not None else 0, _ptr(gate_bias),
                                         _ptr(weight), _ptr(bias), ctypes.c_float(eps), _ptr(nw), _ptr(nb), _ptr(next_out),
                                         act_dt, T, d, _stream()))


def stream_add(x: torch.Tensor, other: Optional[torch.Tensor] = None, vec: Optional[torch.Tensor] = None) -> None:
    """``x[t] += other[t] + vec`` on the 32-bit stream ``[T, d]``; ``other [T, d]`` contiguous, ``vec [d]`` 32-bit."""
    _dev(x, other, vec)
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or (other is not None and (tuple(other.shape) != (T, d) or not other.is_contiguous())):
        raise KernelError("stream_add: contiguous 32-bit x [T, d] and contiguous other [T, d] expected")
    _f32_vec(vec, d, "stream_add: the vector")
    _check(_lib().ri_stream_add(_ptr(x), _ptr(other), _dt(other) if other is not None else F32, _ptr(vec), T, d, _stream()))


def poly_norm(up: torch.Tensor, bias: Optional[torch.Tensor], coef, eps: float, act: torch.Tensor) -> None:
    """``act = a N(z) + b N(z^2) + c N(z^3) + e`` with ``z = up + bias``, ``coef = (a, b, c, e)`` and
    ``N(v) = v / sqrt(mean(v^2) + eps)`` over each row; ``up``, ``act`` ``[T, n]`` (columns of wider buffers allowed)."""
    _dev(up, bias, act)
    _rows2d(up, "up")
    _rows2d(act, "act")
    T, n = up.shape
    if tuple(act.shape) != (T, n) or act.dtype != up.dtype:
        raise KernelError("poly_norm: up and act must be [T, n] of one dtype")
    _f32_vec(bias, n, "poly_norm: the bias")
    a, b, c, e = (float(v) for v in coef)
    _check(_lib().ri_poly_norm(_ptr(up), up.stride(0), _ptr(bias), ctypes.c_float(a), ctypes.c_float(b), ctypes.c_float(c),
                               ctypes.c_float(e), ctypes.c_float(eps), _ptr(act), act.stride(0), _dt(up), T, n, _stream()))


SHORT_CONV_MAX_TAPS = 8
SHORT_CONV_MAX_SEGMENTS = 4


def short_conv(xs, ws, state: Optional[torch.Tensor], out: torch.Tensor, ctx, taps: int, silu: bool = True,
               biases=None) -> None:
    """A causal convolution over time of ``taps`` taps, channel by channel, through the last ``taps - 1``
    inputs each request keeps in ``state [slots, taps - 1, C]`` (32-bit; a request's first tokens start
    from zeros): ``xs`` are up to four ``[T, n_s]`` inputs (columns of a wider buffer allowed), ``ws`` their
    weights ``[n_s, taps]`` (the last column is the current token's); ``out [T, C]`` (32-bit, ``C`` the sum
    of the ``n_s``) takes the results side by side, through silu if asked.  ``biases``: a 32-bit ``[n_s]``
    (or None) for each input, added before the silu."""
    _dev(state, out, *xs, *ws)
    if biases is not None:
        if len(biases) != len(xs):
            raise KernelError("short_conv: a bias (or None) for each input expected")
        for b, x in zip(biases, xs):
            _f32_vec(b, x.shape[1], "short_conv: a bias")
        _dev(*[b for b in biases if b is not None])
    if not xs or len(xs) != len(ws) or len(xs) > SHORT_CONV_MAX_SEGMENTS:
        raise KernelError(f"short_conv: 1 to {SHORT_CONV_MAX_SEGMENTS} inputs with a weight each expected")
    _rows2d(out, "out")
    T = out.shape[0]
    C = sum(int(x.shape[1]) for x in xs)
    dt = xs[0].dtype
    for x, w in zip(xs, ws):
        _rows2d(x, "x")
        if x.shape[0] != T or x.dtype != dt or w.dtype != dt or tuple(w.shape) != (x.shape[1], taps) or not w.is_contiguous():
            raise KernelError(f"short_conv: inputs [T, n] and contiguous weights [n, {taps}] of one dtype expected")
    if out.dtype != torch.float32 or out.shape[1] != C:
        raise KernelError(f"short_conv: out must be 32-bit [T, {C}]")
    if taps > 1 and (state is None or state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (taps - 1, C)
                     or not state.is_contiguous()):
        raise KernelError(f"short_conv: state must be contiguous float32 [slots, {taps - 1}, {C}]")
    _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
    _i32(ctx.q_start, "q_start", ctx.num_rows)
    _i32(ctx.state_slots, "state_slots", ctx.num_rows)
    n = len(xs)
    ptrs = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
    wptrs = (ctypes.c_void_p * n)(*[w.data_ptr() for w in ws])
    strides = (ctypes.c_int * n)(*[x.stride(0) for x in xs])
    widths = (ctypes.c_int * n)(*[x.shape[1] for x in xs])
    bptrs = None
    if biases is not None:
        bptrs = (ctypes.c_void_p * n)(*[b.data_ptr() if b is not None else None for b in biases])
    _check(_lib().ri_short_conv(n, ptrs, strides, wptrs, bptrs, widths, _dt(xs[0]), int(taps), int(bool(silu)), _ptr(state),
                                state.shape[0] if state is not None else 1, _ptr(out), out.stride(0), _ptr(ctx.cu_q),
                                _ptr(ctx.q_start), _ptr(ctx.state_slots), ctx.num_rows, T, int(ctx.max_q_len), _stream()))


def gated_delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta_in: torch.Tensor, decay_in: torch.Tensor,
                     A: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor, out: torch.Tensor, ctx,
                     H: int, Hk: int, dk: int, dv: int, unit_eps: float = 1e-6, q_scale: float = 1.0) -> None:
    """Walk each request's tokens of the step through ``state[slot] [H, dk, dv]`` (32-bit) by the gated
    delta rule: ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q`` with
    ``beta = sigmoid(beta_in)``, ``g = exp(-A softplus(decay_in + dt_bias))`` (one a head and token), q and k
    divided by ``sqrt(|.|^2 + unit_eps)`` and q times ``q_scale``.  ``q, k [T, Hk dk]``, ``v [T, H dv]`` 32-bit
    (columns allowed); head h reads q/k head ``h // (H // Hk)``; ``beta_in, decay_in [T, H]`` activations;
    ``A, dt_bias [H]`` 32-bit; ``out [T, H dv]`` 32-bit.  A request's first tokens start from zeros."""
    _dev(q, k, v, beta_in, decay_in, A, dt_bias, state, out)
    for t, name in ((q, "q"), (k, "k"), (v, "v"), (out, "out"), (beta_in, "beta_in"), (decay_in, "decay_in")):
        _rows2d(t, name)
    T = q.shape[0]
    if tuple(q.shape) != (T, Hk * dk) or tuple(k.shape) != (T, Hk * dk) or tuple(v.shape) != (T, H * dv) \
            or tuple(out.shape) != (T, H * dv) or any(t.dtype != torch.float32 for t in (q, k, v, out)):
        raise KernelError("gated_delta_scan: 32-bit q, k [T, Hk dk], v [T, H dv] and out [T, H dv] expected")
    if tuple(beta_in.shape) != (T, H) or tuple(decay_in.shape) != (T, H) or beta_in.dtype != decay_in.dtype:
        raise KernelError("gated_delta_scan: beta_in and decay_in must be [T, H] of one dtype")
    if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (H, dk, dv) or not state.is_contiguous():
        raise KernelError(f"gated_delta_scan: state must be contiguous float32 [slots, {H}, {dk}, {dv}]")
    _f32_vec(A, H, "gated_delta_scan: A")
    _f32_vec(dt_bias, H, "gated_delta_scan: dt_bias")
    _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
    _i32(ctx.q_start, "q_start", ctx.num_rows)
    _i32(ctx.state_slots, "state_slots", ctx.num_rows)
    _check(_lib().ri_gated_delta_scan(
        _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(beta_in), beta_in.stride(0),
        _ptr(decay_in), decay_in.stride(0), _dt(beta_in), _ptr(A), _ptr(dt_bias), ctypes.c_float(unit_eps),
        ctypes.c_float(q_scale), _ptr(state), state.shape[0], _ptr(out), out.stride(0), _ptr(ctx.cu_q), _ptr(ctx.q_start),
        _ptr(ctx.state_slots), ctx.num_rows, T, H, Hk, dk, dv, _stream()))


def _scan_common(state, out, ctx, H, dk, dv, T, who):
    if tuple(out.shape) != (T, H * dv) or out.dtype != torch.float32:
        raise KernelError(f"{who}: 32-bit out [T, {H * dv}] expected")
    if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (H, dk, dv) or not state.is_contiguous():
        raise KernelError(f"{who}: state must be contiguous float32 [slots, {H}, {dk}, {dv}]")
    _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
    _i32(ctx.q_start, "q_start", ctx.num_rows)
    _i32(ctx.state_slots, "state_slots", ctx.num_rows)


def channel_delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta_in: torch.Tensor, decay_in: torch.Tensor,
                       A: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor, out: torch.Tensor, ctx,
                       H: int, Hk: int, dk: int, dv: int, unit_eps: float = 1e-6, q_scale: float = 1.0) -> None:
    """``gated_delta_scan`` with a decay for every key channel: ``S <- diag(g) S; u = beta (v - S^T k);
    S <- S + k u^T; out = S^T q`` with ``g = exp(-A_h softplus(decay_in + dt_bias))`` laid out heads x dk
    (``decay_in [T, H dk]`` activations or 32-bit, ``dt_bias [H dk]`` and ``A [H]`` 32-bit) and ``beta = sigmoid(beta_in)``,
    ``beta_in [T, H]``.  q, k ``[T, Hk dk]`` and v ``[T, H dv]`` 32-bit; q and k are divided by
    ``sqrt(|.|^2 + unit_eps)``, q also times ``q_scale``."""
    _dev(q, k, v, beta_in, decay_in, A, dt_bias, state, out)
    for t, name in ((q, "q"), (k, "k"), (v, "v"), (out, "out"), (beta_in, "beta_in"), (decay_in, "decay_in")):
        _rows2d(t, name)
    T = q.shape[0]
    if tuple(q.shape) != (T, Hk * dk) or tuple(k.shape) != (T, Hk * dk) or tuple(v.shape) != (T, H * dv) \
            or any(t.dtype != torch.float32 for t in (q, k, v)):
        raise KernelError("channel_delta_scan: 32-bit q, k [T, Hk dk] and v [T, H dv] expected")
    if tuple(beta_in.shape) != (T, H) or tuple(decay_in.shape) != (T, H * dk):
        raise KernelError("channel_delta_scan: beta_in [T, H] and decay_in [T, H dk] expected")
    _scan_common(state, out, ctx, H, dk, dv, T, "channel_delta_scan")
    _f32_vec(A, H, "channel_delta_scan: A")
    _f32_vec(dt_bias, H * dk, "channel_delta_scan: dt_bias")
    _check(_lib().ri_channel_delta_scan(
        _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(beta_in), beta_in.stride(0),
        _ptr(decay_in), decay_in.stride(0), _dt(beta_in), _dt(decay_in), _ptr(A), _ptr(dt_bias), ctypes.c_float(unit_eps),
        ctypes.c_float(q_scale), _ptr(state), state.shape[0], _ptr(out), out.stride(0), _ptr(ctx.cu_q), _ptr(ctx.q_start),
        _ptr(ctx.state_slots), ctx.num_rows, T, H, Hk, dk, dv, _stream()))


def decay_scan(mode: str, r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay_in: torch.Tensor, bias: torch.Tensor,
               state: torch.Tensor, out: torch.Tensor, ctx, H: int, Hk: int, dk: int, dv: int,
               rate: Optional[torch.Tensor] = None, tau: float = 1.0, q_scale: float = 1.0,
               skip: Optional[torch.Tensor] = None) -> None:
    """Walk each request's tokens of the step through ``state[slot] [H, dk, dv]`` (32-bit):
    ``S <- diag(w) S + k v^T``, ``out = S^T r (+ skip_h v)``, with a decay that depends on the token.
    ``mode = "channel"``: ``w = sigmoid(decay_in + bias)^(1 / tau)`` for every key channel (``decay_in [T, H dk]``,
    ``bias [H dk]``), r times ``q_scale``.  ``mode = "head"``: ``dt = softplus(decay_in + bias)`` (``decay_in [T, H]``,
    ``bias [H]``), ``w = exp(-rate_h dt)`` for the whole head, k times dt; r, k ``[T, Hk dk]``, head h reading
    head ``h // (H // Hk)``.  r, k, v of one dtype; ``decay_in`` an activation; ``bias, rate, skip`` 32-bit."""
    if mode not in ("channel", "head"):
        raise KernelError(f"decay_scan: unknown mode {mode!r}")
    _dev(r, k, v, decay_in, bias, rate, skip, state, out)
    for t, name in ((r, "r"), (k, "k"), (v, "v"), (out, "out"), (decay_in, "decay_in")):
        _rows2d(t, name)
    T = r.shape[0]
    if tuple(r.shape) != (T, Hk * dk) or tuple(k.shape) != (T, Hk * dk) or tuple(v.shape) != (T, H * dv) \
            or k.dtype != r.dtype or v.dtype != r.dtype:
        raise KernelError("decay_scan: r, k [T, Hk dk] and v [T, H dv] of one dtype expected")
    n_dec = H * dk if mode == "channel" else H
    if tuple(decay_in.shape) != (T, n_dec):
        raise KernelError(f"decay_scan: decay_in must be [T, {n_dec}]")
    if mode == "channel" and Hk != H:
        raise KernelError("decay_scan: a decay a key channel goes with a head of r and k for every head")
    _scan_common(state, out, ctx, H, dk, dv, T, "decay_scan")
    _f32_vec(bias, n_dec, "decay_scan: bias")
    _f32_vec(skip, H, "decay_scan: skip")
    if mode == "head":
        if rate is None:
            raise KernelError("decay_scan: a rate for each head expected")
        _f32_vec(rate, H, "decay_scan: rate")
    _check(_lib().ri_decay_scan(
        1 if mode == "channel" else 2, _ptr(r), r.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _dt(r),
        _ptr(decay_in), decay_in.stride(0), _dt(decay_in), _ptr(bias), _ptr(rate), ctypes.c_float(1.0 / tau),
        ctypes.c_float(q_scale), _ptr(skip), _ptr(state), state.shape[0], _ptr(out), out.stride(0), _ptr(ctx.cu_q),
        _ptr(ctx.q_start), _ptr(ctx.state_slots), ctx.num_rows, T, H, Hk, dk, dv, _stream()))


def token_shift(h: torch.Tensor, mix: torch.Tensor, state: torch.Tensor, out: torch.Tensor, ctx) -> None:
    """``out[t] = h[t] + (h[t - 1] - h[t]) * mix`` with ``h[t - 1]`` the same request's previous token (zeros
    before position 0); ``state [slots, d]`` (32-bit) keeps every request's last ``h`` from step to step.
    ``h [T, d]`` contiguous 32-bit, ``mix [d]`` 32-bit, ``out [T, d]`` contiguous in the activations' dtype."""
    _dev(h, mix, state, out)
    T, d = h.shape
    if h.dtype != torch.float32 or not h.is_contiguous() or tuple(out.shape) != (T, d) or not out.is_contiguous():
        raise KernelError("token_shift: contiguous 32-bit h [T, d] and contiguous out [T, d] expected")
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != d or not state.is_contiguous():
        raise KernelError(f"token_shift: state must be contiguous float32 [slots, {d}]")
    _f32_vec(mix, d, "token_shift: the mixing weights")
    _i32(ctx.positions, "positions", T)
    _i32(ctx.row_of_token, "row_of_token", T)
    _i32(ctx.cu_q, "cu_q", ctx.num_rows + 1)
    _i32(ctx.state_slots, "state_slots", ctx.num_rows)
    _check(_lib().ri_token_shift(_ptr(h), _ptr(mix), _ptr(state), state.shape[0], _ptr(out), _dt(out), T, d,
                                 _ptr(ctx.positions), _ptr(ctx.row_of_token), _ptr(ctx.cu_q), _ptr(ctx.state_slots), _stream()))


def stream_pair(x: torch.Tensor, delta: Optional[torch.Tensor], y: torch.Tensor, out: torch.Tensor) -> None:
    """``out[t] = [x[t] + delta[t] | y[t]]`` side by side, rounded to ``out``'s dtype: ``x [T, d]`` 32-bit,
    ``delta`` ``[T, d]`` or a 32-bit stack ``[P, T, d]`` of partial sums (or None), ``y [T, d]`` 32-bit,
    ``out [T, 2 d]``; all contiguous.  ``x`` itself is left as it is."""
    _dev(x, delta, y, out)
    T, d = x.shape
    if x.dtype != torch.float32 or y.dtype != torch.float32 or tuple(y.shape) != (T, d) or tuple(out.shape) != (T, 2 * d) \
            or not (x.is_contiguous() and y.is_contiguous() and out.is_contiguous()):
        raise KernelError("stream_pair: contiguous 32-bit x, y [T, d] and contiguous out [T, 2 d] expected")
    parts, stride, ddt = 1, 0, F32
    if delta is not None:
        if delta.dim() == 3:
            parts, stride = delta.shape[0], delta.stride(0)
        if delta.dim() not in (2, 3) or tuple(delta.shape[-2:]) != (T, d) or delta.stride(-1) != 1 or delta.stride(-2) != d \
                or (delta.dim() == 3 and delta.dtype != torch.float32):
            raise KernelError("stream_pair: delta must be [T, d] or a float32 stack [P, T, d] with contiguous rows")
        ddt = _dt(delta)
    _check(_lib().ri_stream_pair(_ptr(x), _ptr(delta), ddt, parts, ctypes.c_longlong(stride), _ptr(y), F32, _ptr(out),
                                 _dt(out), T, d, _stream()))
