"""Python faces of the HIP kernels: they check shapes, dtypes and contiguity on
the host, then launch on torch's current stream. Tensors are torch tensors on
the GPU; nothing here computes in torch."""
from __future__ import annotations

import torch

from . import kv_layout as layout
from . import lib as _lib
from .profiler import op as _op

F32, BF16, F16 = 0, 1, 2
PAGE_TOKENS = 64

_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise TypeError(f"kernels take float32 or bfloat16 tensors, not {dtype}") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous tensor")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if shape is not None:
        if len(shape) != t.dim() or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


@_op("fill_random")
def fill_random(out, key: int, quantiles, mean: float, std: float) -> None:
    """out (float32 or bfloat16, any shape, contiguous) = seeded normal values, element by
    element what weights.random_init.normal_values gives on the host for the same key."""
    _need(out, "out")
    _need(quantiles, "quantiles", torch.float32, (65536,))
    L = _lib.load()
    _lib.check(L.he_fill_random(out.data_ptr(), out.numel(), dtype_code(out.dtype), key & ((1 << 64) - 1),
                                quantiles.data_ptr(), float(mean), float(std), _stream()))


@_op("fill_random")
def fill_random_integers(out_i32, key: int, high: int) -> None:
    _need(out_i32, "out", torch.int32)
    L = _lib.load()
    _lib.check(L.he_fill_random_integers(out_i32.data_ptr(), out_i32.numel(), key & ((1 << 64) - 1), int(high),
                                         _stream()))


@_op("cast")
def cast(out, src) -> None:
    """out (float32 or bfloat16) = src (float32, bfloat16 or float16) converted, same element count."""
    _need(out, "out")
    _need(src, "src")
    if out.numel() != src.numel():
        raise ValueError("cast: out and src differ in size")
    code = F16 if src.dtype == torch.float16 else dtype_code(src.dtype)
    L = _lib.load()
    _lib.check(L.he_cast(out.data_ptr(), src.data_ptr(), src.numel(), code, dtype_code(out.dtype), _stream()))


@_op("embedding")
def embedding(out_f32, table, ids, rows: int, scale: float = 1.0) -> None:
    """out[t] = table[ids[t]] * scale in fp32."""
    V, D = table.shape
    _need(table, "table")
    _need(out_f32, "out", torch.float32)
    _need(ids, "ids", torch.int32)
    if out_f32.numel() < rows * D or ids.numel() < rows:
        raise ValueError("embedding: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_embedding(out_f32.data_ptr(), table.data_ptr(), ids.data_ptr(), rows, D, V,
                              dtype_code(table.dtype), float(scale), _stream()))


@_op("gather_rows")
def gather_rows_f32(out, src, rows_idx, n_out: int, n_src: int) -> None:
    D = src.shape[-1]
    _need(src, "src", torch.float32)
    _need(out, "out", torch.float32)
    _need(rows_idx, "rows", torch.int32)
    if out.numel() < n_out * D or rows_idx.numel() < n_out or src.numel() < n_src * D:
        raise ValueError("gather_rows: buffers smaller than the row counts")
    L = _lib.load()
    _lib.check(L.he_gather_rows_f32(out.data_ptr(), src.data_ptr(), rows_idx.data_ptr(), n_out, D,
                                    n_src, _stream()))


@_op("residual_add")
def residual_add(resid_f32, delta, rows: int, scale: float = 1.0) -> None:
    """resid += scale * delta."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    _need(delta, "delta")
    if delta.shape[-1] != D or resid_f32.numel() < rows * D or delta.numel() < rows * D:
        raise ValueError("residual_add: shape mismatch")
    L = _lib.load()
    _lib.check(L.he_residual_add(resid_f32.data_ptr(), delta.data_ptr(), rows * D,
                                 dtype_code(delta.dtype), float(scale), _stream()))


@_op("silu_mul")
def silu_mul(out, gate_up, rows: int, interleaved: bool = False, splits: int = 0, *,
             alpha: float = 1.0, limit: float = 0.0, up_shift: float = 0.0) -> None:
    """out[rows, I] = silu(gate) * up. gate_up: [rows, 2I] in out's dtype, or with
    splits > 0 the fp32 K slices [splits, rows, 2I] of the product. Its columns are all
    gates then all ups, or, interleaved, gate i in column 2i and its up in 2i + 1.
    With constants it is the gated activation g' * sigmoid(alpha * g') * (u' + up_shift),
    g' = min(gate, limit), u' = clamp(up, -limit, limit) (limit 0: unbounded)."""
    I = out.shape[-1]
    _need(out, "out")
    _need(gate_up, "gate_up", torch.float32 if splits > 0 else out.dtype)
    if gate_up.shape[-1] != 2 * I or out.numel() < rows * I or \
            gate_up.numel() < max(splits, 1) * rows * 2 * I:
        raise ValueError("silu_mul: gate_up must be [rows, 2*I] for out [rows, I]")
    if splits > 0 and tuple(gate_up.shape) != (splits, rows, 2 * I):
        raise ValueError("silu_mul: split sums must be [splits, rows, 2*I]")
    L = _lib.load()
    _lib.check(L.he_gated_act(out.data_ptr(), gate_up.data_ptr(), rows, I, int(interleaved), splits,
                              dtype_code(out.dtype), float(alpha), float(limit), float(up_shift), _stream()))


@_op("add_dyt")
def add_dyt(resid_f32, delta, weight, bias, alpha, out, rows: int, delta_scale: float = 1.0) -> None:
    """resid += delta_scale * delta (if given); out = tanh(alpha * resid) * weight + bias (if out given).
    alpha: a tensor of one element on the device; weight, bias: [D]; the three share a dtype."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    _need(weight, "weight", shape=(D,))
    _need(bias, "bias", weight.dtype, (D,))
    _need(alpha, "alpha", weight.dtype)
    if alpha.numel() != 1:
        raise ValueError("add_dyt: alpha is one number")
    if resid_f32.numel() < rows * D:
        raise ValueError("add_dyt: resid smaller than the row count")
    act = None
    if out is not None:
        _need(out, "out")
        if out.shape[-1] != D or out.numel() < rows * D:
            raise ValueError(f"add_dyt: out does not match [rows, {D}]")
        act = out.dtype
    if delta is not None:
        _need(delta, "delta")
        if delta.shape[-1] != D or delta.numel() < rows * D:
            raise ValueError(f"add_dyt: delta does not match [rows, {D}]")
        if act is not None and delta.dtype != act:
            raise TypeError("add_dyt: delta and out must share a dtype")
        act = delta.dtype
    L = _lib.load()
    _lib.check(L.he_add_dyt(resid_f32.data_ptr(), _ptr(delta), float(delta_scale), weight.data_ptr(),
                            bias.data_ptr(), alpha.data_ptr(), _ptr(out), rows, D,
                            dtype_code(act or torch.float32), dtype_code(weight.dtype), _stream()))


@_op("add_rmsnorm")
def add_rmsnorm(resid_f32, delta, weight, out, rows: int, eps: float) -> None:
    """resid += delta (if given); out = rmsnorm(resid) * weight (if out given)."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    _need(weight, "weight", shape=(D,))
    if resid_f32.numel() < rows * D:
        raise ValueError("add_rmsnorm: resid smaller than the row count")
    act = None
    if out is not None:
        _need(out, "out")
        if out.shape[-1] != D or out.numel() < rows * D:
            raise ValueError(f"add_rmsnorm: out does not match [rows, {D}]")
        act = out.dtype
    if delta is not None:
        _need(delta, "delta")
        if delta.shape[-1] != D or delta.numel() < rows * D:
            raise ValueError(f"add_rmsnorm: delta does not match [rows, {D}]")
        if act is not None and delta.dtype != act:
            raise TypeError("add_rmsnorm: delta and out must share a dtype")
        act = delta.dtype
    L = _lib.load()
    _lib.check(L.he_add_rmsnorm(resid_f32.data_ptr(), _ptr(delta), weight.data_ptr(), _ptr(out), rows, D,
                                float(eps), dtype_code(act or torch.float32), dtype_code(weight.dtype),
                                _stream()))


@_op("rmsnorm_rows")
def rmsnorm_rows(out, x, weight, rows: int, D: int, x_stride: int, out_stride: int,
                 eps: float) -> None:
    if out.dtype != x.dtype:
        raise TypeError("rmsnorm_rows: out and x must share a dtype")
    if weight is not None:
        _need(weight, "weight", shape=(D,))
    if rows > 0 and (x.numel() < (rows - 1) * x_stride + D or out.numel() < (rows - 1) * out_stride + D):
        raise ValueError("rmsnorm_rows: buffers smaller than rows and strides need")
    L = _lib.load()
    _lib.check(L.he_rmsnorm_rows(out.data_ptr(), x.data_ptr(), _ptr(weight), rows, D, x_stride,
                                 out_stride, float(eps), dtype_code(x.dtype),
                                 dtype_code(weight.dtype) if weight is not None else F32, _stream()))


@_op("rmsnorm_row_pair")
def rmsnorm_row_pair(x, w1, D1: int, w2, D2: int, col2: int, rows: int, eps: float) -> None:
    """x[r, :D1] and x[r, col2:col2 + D2], each by its own root mean square and gain (w1, w2), in place, in one
    launch. x: [rows, wide] with wide >= col2 + D2 (q and k as they lie behind one product)."""
    if not x.is_cuda:
        raise ValueError("x: expected a GPU tensor")
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[0] < rows or x.shape[1] < col2 + D2 or col2 < D1:
        raise ValueError("rmsnorm_row_pair: the stretches do not lie in the rows")
    _need(w1, "w1", shape=(D1,))
    _need(w2, "w2", w1.dtype, (D2,))
    L = _lib.load()
    _lib.check(L.he_rmsnorm_row_pair(x.data_ptr(), w1.data_ptr(), D1, w2.data_ptr(), D2, col2, rows, x.stride(0),
                                     float(eps), dtype_code(x.dtype), dtype_code(w1.dtype), _stream()))


def gemm_plain_workspace_floats(M: int, N: int, K: int) -> int:
    """Floats of workspace with which gemm_plain runs a product of few rows through the kernels made
    for it (0: none needed)."""
    return int(_lib.load().he_gemm_plain_workspace_floats(M, N, K))


@_op("gemm_plain")
def gemm_plain(out, a, w, bias, M: int, workspace=None) -> None:
    """out[M,N] = a[M,K] . w[N,K]^T (+ bias), fixed summation order. workspace: fp32, of
    gemm_plain_workspace_floats(M, N, K) elements or more, for a product of few rows (the result
    is the same bit for bit without it, and slower)."""
    N, K = w.shape
    _need(a, "a")
    _need(w, "w", a.dtype)
    _need(out, "out")
    if a.shape[-1] != K or out.shape[-1] != N or a.numel() < M * K or out.numel() < M * N:
        raise ValueError(f"gemm_plain: shapes a{tuple(a.shape)} w{tuple(w.shape)} out{tuple(out.shape)} M={M}")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    L = _lib.load()
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    _lib.check(L.he_gemm_plain(out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, K,
                               K, N, dtype_code(a.dtype), dtype_code(out.dtype),
                               dtype_code(bias.dtype) if bias is not None else F32,
                               _ptr(workspace), workspace.numel() if workspace is not None else 0, _stream()))


BLOCKSPLIT_MAX_M = 32


PIECES_MAX_M = 64
BLOCKSPLIT_PIECES_MAX_M = 16   # the block-split product reads and writes pieces up to 16 rows
ROWS_MAX_M = 64


def pieces_shape(M: int, D: int) -> tuple[int, int, int]:
    """Shape of a piece-major [M, D] bf16 tensor: 16-byte pieces of 8 columns, the M pieces of
    one column group next to each other: element (m, d) at [d // 8, m, d % 8]. The block-split
    product reads its rows best this way (a wavefront's load of 16 rows x 16 bytes touches two
    cache lines, not sixteen), and writes them so for the next one; at most PIECES_MAX_M rows."""
    if D % 8 != 0 or not 0 < M <= PIECES_MAX_M:
        raise ValueError(f"piece-major rows: D={D} must be a multiple of 8 and 0 < M={M} <= {PIECES_MAX_M}")
    return (D // 8, M, 8)


def gemm_blocksplit_blocks(M: int, N: int, K: int) -> int:
    """Partial sums of squares per row that the residual epilogue of this product gives."""
    return int(_lib.load().he_gemm_blocksplit_blocks(M, N, K))


@_op("gemm_blocksplit")
def gemm_blocksplit(out, a, w, bias, M: int, gated: bool = False, plan=(0, 0, 0), *,
                    row_scale=None, residual=None, x_pieces: bool = False, out_pieces: bool = False,
                    act=(1.0, 0.0, 0.0)) -> None:
    """bf16 MFMA product for M <= 32 with K cut inside the workgroup; one launch, complete
    result (bf16 or fp32), with bias or, gated, as [M, N/2] = silu(gate) * up for a weight
    that alternates gate and up rows (gate i at row 2i, its up at 2i + 1). plan = (R, U, NW),
    zeros = heuristic. act = (alpha, limit, up_shift): the gated epilogue's constants as silu_mul
    takes them.

    row_scale = (partials fp32 [M, count], eps): the rows of `a` are r * gain of an RMS norm
    whose 1/sqrt(mean(r^2) + eps) is applied to the sums here (mean over K).
    residual = (resid fp32 [M, N], gain [N], xg bf16 [M, N], sq fp32 [M, blocks]): instead of
    writing `out` (None), resid += result in place, xg = resid * gain, sq = the sums of resid^2
    per workgroup (blocks = gemm_blocksplit_blocks(M, N, K)).
    The tuple may go on with (scale, dyt_bias, dyt_alpha): resid += scale * result, and with the last two
    (a vector [N] and a one-element tensor of gain's dtype) the rows left are those of a Dynamic Tanh in
    full, xg = tanh(alpha * resid) * gain + dyt_bias, and sq = 0 (with eps 1 nothing is owed).
    x_pieces: `a` is piece-major, shaped pieces_shape(M, K). out_pieces: the bf16 output (`out`,
    or xg of the residual epilogue) is written piece-major, shaped pieces_shape(M, its width)."""
    N, K = w.shape
    NO = N // 2 if gated else N
    _need(a, "a", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    if M > BLOCKSPLIT_MAX_M:
        raise ValueError(f"gemm_blocksplit: M={M} above {BLOCKSPLIT_MAX_M}")
    if (x_pieces or out_pieces) and M > BLOCKSPLIT_PIECES_MAX_M:
        raise ValueError(f"gemm_blocksplit: piece-major rows are for up to {BLOCKSPLIT_PIECES_MAX_M} rows, not {M}")
    if x_pieces:
        _need(a, "a", shape=pieces_shape(M, K))
    elif a.shape[-1] != K or a.numel() < M * K:
        raise ValueError(f"gemm_blocksplit: shapes a{tuple(a.shape)} w{tuple(w.shape)} M={M}")
    if residual is None:
        _need(out, "out")
        if out_pieces:
            _need(out, "out", torch.bfloat16, pieces_shape(M, NO))
        elif out.shape[-1] != NO or out.numel() < M * NO:
            raise ValueError(f"gemm_blocksplit: out{tuple(out.shape)} for M={M} N={NO}")
    elif out is not None or gated or plan != (0, 0, 0):
        raise ValueError("gemm_blocksplit: the residual epilogue writes no `out`, is not gated and plans itself")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    sp, sc, se = None, 0, 0.0
    if row_scale is not None:
        partials, se = row_scale
        _need(partials, "row_scale partials", torch.float32)
        if partials.dim() != 2 or partials.shape[0] < M:
            raise ValueError("gemm_blocksplit: row_scale partials must be [M, count]")
        sp, sc = partials.data_ptr(), partials.shape[1]
    rp = gp = xp = qp = None
    gdt, qc = F32, 0
    rscale, dyt_bias, dyt_alpha = 1.0, None, None
    if residual is not None:
        resid, gain, xg, sq, *more = residual
        rscale = more[0] if more else 1.0
        dyt_bias, dyt_alpha = (more[1], more[2]) if len(more) > 2 else (None, None)
        if dyt_alpha is not None:
            _need(dyt_bias, "dyt bias", gain.dtype, (N,))
            _need(dyt_alpha, "dyt alpha", gain.dtype)
        _need(resid, "resid", torch.float32)
        _need(gain, "gain", shape=(N,))
        _need(xg, "xg", torch.bfloat16)
        _need(sq, "sq", torch.float32)
        if out_pieces:
            _need(xg, "xg", shape=pieces_shape(M, N))
        if resid.shape[-1] != N or resid.numel() < M * N or xg.numel() < M * N \
                or (not out_pieces and xg.shape[-1] != N) or sq.dim() != 2 or sq.shape[0] < M:
            raise ValueError("gemm_blocksplit: residual buffers do not match [M, N]")
        rp, gp, xp, qp = resid.data_ptr(), gain.data_ptr(), xg.data_ptr(), sq.data_ptr()
        gdt, qc = dtype_code(gain.dtype), sq.shape[1]
    L = _lib.load()
    _lib.check(L.he_gemm_blocksplit_fused_bf16(
        _ptr(out), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K,
        dtype_code(out.dtype) if out is not None else BF16,
        dtype_code(bias.dtype) if bias is not None else F32, int(gated),
        int(plan[0]), int(plan[1]), int(plan[2]), sp, sc, float(se), rp, gp, gdt, xp, qp, qc,
        int(x_pieces), int(out_pieces), float(act[0]), float(act[1]), float(act[2]), float(rscale),
        _ptr(dyt_bias), _ptr(dyt_alpha), _stream()))


def gemm_rows_plan(M: int, N: int, K: int) -> tuple[int, int]:
    """(workgroups along N, K slices) of gemm_rows for this product: the count of partial sums of
    squares its residual epilogue gives, and whether it leaves plain sums or partial sums."""
    import ctypes
    g, s = ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.load().he_gemm_rows_plan(M, N, K, ctypes.byref(g), ctypes.byref(s)))
    return g.value, s.value


@_op("gemm_rows")
def gemm_rows(out, partial, a, w, bias, M: int, gated: bool = False, plan=(0, 0, 0), *, row_scale=None,
              residual=None, x_pieces: bool = False, out_pieces: bool = False, act=(1.0, 0.0, 0.0)) -> int:
    """bf16 MFMA product for M <= 64 whose activation rows go through LDS once per workgroup; the
    epilogues of gemm_blocksplit (see there: bias, gated, row_scale, residual, x_pieces, out_pieces).
    plan = (R, NWV, splits), zeros = heuristic. A product cut into several K slices writes its fp32
    sums into `partial` ([slices, M, N], each already scaled by row_scale) and takes no other
    epilogue. Returns the number of slices."""
    import ctypes
    N, K = w.shape
    NO = N // 2 if gated else N
    _need(a, "a", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    if not 0 < M <= ROWS_MAX_M:
        raise ValueError(f"gemm_rows: M={M} outside [1, {ROWS_MAX_M}]")
    if x_pieces:
        _need(a, "a", shape=pieces_shape(M, K))
    elif a.shape[-1] != K or a.numel() < M * K:
        raise ValueError(f"gemm_rows: shapes a{tuple(a.shape)} w{tuple(w.shape)} M={M}")
    if out is not None:
        _need(out, "out")
        if out_pieces:
            _need(out, "out", torch.bfloat16, pieces_shape(M, NO))
        elif out.shape[-1] != NO or out.numel() < M * NO:
            raise ValueError(f"gemm_rows: out{tuple(out.shape)} for M={M} N={NO}")
    pf = 0
    if partial is not None:
        _need(partial, "partial", torch.float32)
        pf = partial.numel()
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    sp, sc, se = None, 0, 0.0
    if row_scale is not None:
        partials, se = row_scale
        _need(partials, "row_scale partials", torch.float32)
        if partials.dim() != 2 or partials.shape[0] < M:
            raise ValueError("gemm_rows: row_scale partials must be [M, count]")
        sp, sc = partials.data_ptr(), partials.shape[1]
    rp = gp = xp = qp = None
    gdt, qc = F32, 0
    rscale, dyt_bias, dyt_alpha = 1.0, None, None
    if residual is not None:
        resid, gain, xg, sq, *more = residual
        rscale = more[0] if more else 1.0
        dyt_bias, dyt_alpha = (more[1], more[2]) if len(more) > 2 else (None, None)
        if dyt_alpha is not None:
            _need(dyt_bias, "dyt bias", gain.dtype, (N,))
            _need(dyt_alpha, "dyt alpha", gain.dtype)
        _need(resid, "resid", torch.float32)
        _need(gain, "gain", shape=(N,))
        _need(xg, "xg", torch.bfloat16)
        _need(sq, "sq", torch.float32)
        if out_pieces:
            _need(xg, "xg", shape=pieces_shape(M, N))
        if resid.shape[-1] != N or resid.numel() < M * N or xg.numel() < M * N \
                or (not out_pieces and xg.shape[-1] != N) or sq.dim() != 2 or sq.shape[0] < M:
            raise ValueError("gemm_rows: residual buffers do not match [M, N]")
        rp, gp, xp, qp = resid.data_ptr(), gain.data_ptr(), xg.data_ptr(), sq.data_ptr()
        gdt, qc = dtype_code(gain.dtype), sq.shape[1]
    used = ctypes.c_int(0)
    L = _lib.load()
    _lib.check(L.he_gemm_rows_bf16(
        _ptr(out), _ptr(partial), pf, a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K,
        dtype_code(out.dtype) if out is not None else BF16,
        dtype_code(bias.dtype) if bias is not None else F32, int(gated),
        int(plan[0]), int(plan[1]), int(plan[2]), sp, sc, float(se), rp, gp, gdt, xp, qp, qc,
        int(x_pieces), int(out_pieces), ctypes.byref(used), float(act[0]), float(act[1]), float(act[2]),
        float(rscale), _ptr(dyt_bias), _ptr(dyt_alpha), _stream()))
    return used.value


def splitk_reduce_residual_blocks(N: int) -> int:
    return int(_lib.load().he_splitk_reduce_residual_blocks(N))


@_op("splitk_reduce_residual")
def splitk_reduce_residual(resid, partial, bias, gain, xg, sq, M: int, splits: int,
                           out_pieces: bool = False, *, scale: float = 1.0, dyt_bias=None, dyt_alpha=None) -> None:
    """resid [M, N] (fp32, in place) += the K slices partial [splits, M, N] in index order (+ bias);
    xg = bf16(resid * gain), piece-major with out_pieces; sq [M, blocks] = sums of resid^2 per block
    of columns (blocks = splitk_reduce_residual_blocks(N))."""
    N = resid.shape[-1]
    _need(resid, "resid", torch.float32)
    _need(partial, "partial", torch.float32)
    _need(gain, "gain", shape=(N,))
    _need(xg, "xg", torch.bfloat16)
    _need(sq, "sq", torch.float32)
    if out_pieces:
        _need(xg, "xg", shape=pieces_shape(M, N))
    if resid.numel() < M * N or partial.numel() < splits * M * N or xg.numel() < M * N \
            or sq.dim() != 2 or sq.shape[0] < M or (not out_pieces and xg.shape[-1] != N):
        raise ValueError("splitk_reduce_residual: buffers do not match [splits, M, N]")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    L = _lib.load()
    _lib.check(L.he_splitk_reduce_residual(
        resid.data_ptr(), partial.data_ptr(), _ptr(bias), dtype_code(bias.dtype) if bias is not None else F32,
        gain.data_ptr(), dtype_code(gain.dtype), xg.data_ptr(), sq.data_ptr(), sq.shape[1], M, N, splits,
        int(out_pieces), float(scale), _ptr(dyt_bias), _ptr(dyt_alpha), _stream()))


@_op("scale_rows")
def scale_rows(out, x, partials, eps: float, rows: int, x_pieces: bool = False) -> None:
    """out = x / sqrt(sum(partials of the row) / D + eps) for rows x = r * gain (bf16). out is
    row-major; x_pieces: x is piece-major, shaped pieces_shape(rows, D)."""
    D = out.shape[-1]
    _need(out, "out", torch.bfloat16)
    _need(x, "x", torch.bfloat16)
    _need(partials, "partials", torch.float32)
    if x_pieces:
        _need(x, "x", shape=pieces_shape(rows, D))
    if out.numel() < rows * D or x.numel() < rows * D or (not x_pieces and x.shape[-1] != D) \
            or partials.dim() != 2 or partials.shape[0] < rows:
        raise ValueError("scale_rows: buffers do not match [rows, D]")
    _lib.check(_lib.load().he_scale_rows_bf16(out.data_ptr(), x.data_ptr(), partials.data_ptr(),
                                              partials.shape[1], rows, D, float(eps), int(x_pieces),
                                              _stream()))


@_op("splitk_reduce")
def splitk_reduce(out, partial, bias, M: int, splits: int) -> None:
    """out[M, N] = sum of partial[s] over the slices in index order (+ bias)."""
    N = out.shape[-1]
    _need(out, "out")
    _need(partial, "partial", torch.float32)
    if partial.numel() < splits * M * N or out.numel() < M * N:
        raise ValueError("splitk_reduce: buffers smaller than [splits, M, N]")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    L = _lib.load()
    _lib.check(L.he_splitk_reduce(out.data_ptr(), partial.data_ptr(), _ptr(bias), M, N, splits,
                                  dtype_code(out.dtype),
                                  dtype_code(bias.dtype) if bias is not None else F32, _stream()))


@_op("qkv_rope_cache")
def qkv_rope_cache(q_out, kpool, vpool, qkv, q_cols: int, kv_cols: int, bias, positions, row_seq,
                   seq_slot, page_table, inv_freq, rotary_dim: int, rows: int, H: int, KVH: int,
                   hd: int, write_kv: bool, *, key_dim: int = 0, value_dim: int = 0,
                   interleaved: bool = False, mscale: float = 1.0, q_temp=None) -> None:
    """qkv: [rows, q_cols + kv_cols + v_cols (+ more)] projected rows without bias; bias (optional)
    covers those columns. Rotated q goes to q_out [rows, H*hd]; k, v go into the pools at
    (slot, position) when write_kv. hd is the head size of q_out and of the cache pages; key_dim and
    value_dim (0: hd) are the head sizes of the q/k and of the v columns, at most hd (q_out is then
    padded with zeros, the pages keep the zeros they were made with). interleaved: frequency i turns
    the dims (2i, 2i + 1) instead of (i, i + rotary_dim / 2); mscale multiplies cos and sin."""
    _need(qkv, "qkv")
    _need(q_out, "q_out")
    if qkv.dtype != q_out.dtype:
        raise TypeError("qkv_rope_cache: qkv and q_out must share a dtype")
    width = qkv.shape[-1]
    kd, vd = key_dim or hd, value_dim or hd
    v_cols = KVH * vd
    if kd > hd or vd > hd or rotary_dim > kd:
        raise ValueError("qkv_rope_cache: the rows' head sizes exceed the pages'")
    if q_cols != H * kd or (write_kv and (kv_cols != KVH * kd or width < q_cols + kv_cols + v_cols)):
        raise ValueError("qkv_rope_cache: column layout does not match the head sizes")
    if not write_kv and width < q_cols:
        raise ValueError("qkv_rope_cache: qkv narrower than the query columns")
    if qkv.numel() < rows * width or q_out.numel() < rows * H * hd:
        raise ValueError("qkv_rope_cache: buffers smaller than the row count")
    _need(positions, "positions", torch.int32)
    _need(row_seq, "row_seq", torch.int32)
    _need(seq_slot, "seq_slot", torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("qkv_rope_cache: metadata shorter than the row count")
    es = qkv.element_size()
    base = qkv.data_ptr()
    k_in = v_in = None
    max_blocks = num_pages = 0
    if write_kv:
        _need(kpool, "kpool", q_out.dtype, (None, KVH, layout.k_page_elems(hd)))
        _need(vpool, "vpool", q_out.dtype, (None, KVH, layout.v_page_elems(hd)))
        _need(page_table, "page_table", torch.int32)
        num_pages = kpool.shape[0]
        max_blocks = page_table.shape[1]
        k_in = base + q_cols * es
        v_in = base + (q_cols + kv_cols) * es
    qb = kb = vb = None
    bias_code = F32
    if bias is not None:
        _need(bias, "bias")
        if bias.numel() < (q_cols + kv_cols + v_cols if write_kv else q_cols):
            raise ValueError("qkv_rope_cache: bias shorter than the columns")
        bias_code = dtype_code(bias.dtype)
        bes = bias.element_size()
        qb = bias.data_ptr()
        if write_kv:
            kb = qb + q_cols * bes
            vb = qb + (q_cols + kv_cols) * bes
    if rotary_dim:
        _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    L = _lib.load()
    _lib.check(L.he_qkv_rope_cache(
        q_out.data_ptr(), _ptr(kpool) if write_kv else None, _ptr(vpool) if write_kv else None,
        base, k_in, v_in, width, qb, kb, vb, bias_code, positions.data_ptr(), row_seq.data_ptr(),
        seq_slot.data_ptr(), _ptr(page_table) if write_kv else None, max_blocks, num_pages,
        _ptr(inv_freq) if rotary_dim else None, rotary_dim, rows, H, KVH if write_kv else 0, hd,
        kd, vd, int(interleaved), float(mscale), float(q_temp[0]) if q_temp else 0.0,
        int(q_temp[1]) if q_temp else 0, dtype_code(q_out.dtype), _stream()))


@_op("conv_state")
def conv_state(out, x, taps, bias, state, positions, row_seq, seq_slot, seq_start, cu_seqlens,
               rows: int, num_seqs: int, all_single: bool, act: bool = True) -> None:
    """out[rows, C] = silu(causal convolution per channel of x + bias) (bias None: none; act False: the
    convolution's sum as it is), the taps' last column on the
    row's own input; the inputs before a step's first row come from the sequence's row of `state`
    (uint8 [slots, bytes], fp32 [K-1][C] at its start), which is then moved on. x: a view [rows, C]
    of wider rows (unit stride along C)."""
    C, K = taps.shape
    _need(out, "out", x.dtype, (None, C))
    _need(taps, "taps")
    if bias is not None:
        _need(bias, "bias", taps.dtype, (C,))
    if x.dim() != 2 or x.shape[1] != C or x.stride(1) != 1 or x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError("conv_state: x must be [rows, C] with unit stride along C")
    if state.dtype != torch.uint8 or state.dim() != 2 or state.stride(1) != 1:
        raise ValueError("conv_state: state must be uint8 [slots, bytes]")
    for name, t, n in (("positions", positions, rows), ("row_seq", row_seq, rows), ("seq_slot", seq_slot, num_seqs),
                       ("seq_start", seq_start, num_seqs), ("cu_seqlens", cu_seqlens, num_seqs + 1)):
        _need(t, name, torch.int32)
        if t.numel() < n:
            raise ValueError(f"conv_state: {name} shorter than the step")
    if state.shape[1] < 4 * (K - 1) * C:
        raise ValueError("conv_state: the state rows are too short")
    L = _lib.load()
    _lib.check(L.he_conv_state(out.data_ptr(), x.data_ptr(), x.stride(0), taps.data_ptr(), _ptr(bias),
                               dtype_code(taps.dtype), state.data_ptr(), state.stride(0), positions.data_ptr(),
                               row_seq.data_ptr(), seq_slot.data_ptr(), seq_start.data_ptr(), cu_seqlens.data_ptr(),
                               rows, num_seqs, C, K, int(all_single), int(act), dtype_code(x.dtype), _stream()))


def ssm_state_floats(R: int, P: int, N: int) -> int:
    """Floats of a sequence's scan state (the state dims padded to the threads' share)."""
    return int(_lib.load().he_ssm_state_floats(R, P, N))


@_op("ssm_scan")
def ssm_scan(y, xbc, dt, dt_bias, a_log, d_skip, state, state_offset: int, cu_seqlens, seq_slot,
             rows: int, num_seqs: int, R: int, Q: int, N: int, P: int, max_q_len: int = 0) -> None:
    """y (fp32 [rows, R P]) = the selective scan of xbc [rows, R P + 2 Q N] (x, then B, then C) with step
    sizes softplus(dt + dt_bias) (dt: a view [rows, R] of wider rows), per head r the decay
    exp(-exp(a_log_r) dt) and the skip d_skip_r; the state [R][P][N'] lives at byte state_offset of a
    sequence's row of `state` and is carried on. max_q_len: a bound on the rows a sequence brings (0: none)."""
    C = R * P + 2 * Q * N
    _need(y, "y", torch.float32, (None, R * P))
    _need(xbc, "xbc", None, (None, C))
    if dt.dtype != xbc.dtype or dt.dim() != 2 or dt.shape[1] != R or dt.stride(1) != 1:
        raise ValueError("ssm_scan: dt must be a [rows, R] view in xbc's dtype")
    for name, t in (("dt_bias", dt_bias), ("a_log", a_log), ("d_skip", d_skip)):
        _need(t, name, dt_bias.dtype, (R,))
    if y.shape[0] < rows or xbc.shape[0] < rows or dt.shape[0] < rows:
        raise ValueError("ssm_scan: buffers smaller than the row count")
    if state.dtype != torch.uint8 or state.dim() != 2 or state.stride(1) != 1 \
            or state.shape[1] < state_offset + 4 * ssm_state_floats(R, P, N):
        raise ValueError("ssm_scan: state must be uint8 [slots, bytes] with room for the scan's state")
    _need(cu_seqlens, "cu_seqlens", torch.int32)
    _need(seq_slot, "seq_slot", torch.int32)
    if cu_seqlens.numel() < num_seqs + 1 or seq_slot.numel() < num_seqs:
        raise ValueError("ssm_scan: metadata shorter than the step")
    L = _lib.load()
    _lib.check(L.he_ssm_scan(y.data_ptr(), xbc.data_ptr(), dt.data_ptr(), dt.stride(0), dt_bias.data_ptr(),
                             a_log.data_ptr(), d_skip.data_ptr(), dtype_code(dt_bias.dtype), state.data_ptr(),
                             state.stride(0), state_offset, cu_seqlens.data_ptr(), seq_slot.data_ptr(), rows,
                             num_seqs, int(max_q_len), R, Q, N, P, dtype_code(xbc.dtype), _stream()))


@_op("gated_group_norm")
def gated_group_norm(out, y, z, weight, rows: int, parts: int, eps: float, gate_after: bool = False,
                     out_scale: float = 1.0) -> None:
    """out[rows, W] = (y * silu(z)), each of `parts` equal stretches of a row divided by its own root mean
    square, times weight. y fp32 [rows, W]; z a view [rows, W] of wider rows in out's dtype. gate_after: each
    stretch of y is divided by its own root mean square as it is, and the result is multiplied by weight,
    sigmoid(z) and out_scale; gate_after "silu": by silu(z) in place of sigmoid(z)."""
    W = weight.shape[0]
    _need(out, "out", None, (None, W))
    _need(y, "y", torch.float32, (None, W))
    _need(weight, "weight")
    if z.dtype != out.dtype or z.dim() != 2 or z.shape[1] != W or z.stride(1) != 1:
        raise ValueError("gated_group_norm: z must be a [rows, W] view in out's dtype")
    if min(out.shape[0], y.shape[0], z.shape[0]) < rows or W % parts:
        raise ValueError("gated_group_norm: buffers smaller than the row count, or parts that do not divide the width")
    L = _lib.load()
    _lib.check(L.he_gated_group_norm(out.data_ptr(), y.data_ptr(), z.data_ptr(), z.stride(0), weight.data_ptr(),
                                     dtype_code(weight.dtype), rows, W, parts, float(eps), 2 if gate_after == "silu" else int(bool(gate_after)),
                                     float(out_scale), dtype_code(out.dtype), _stream()))


ACT_KINDS = {"relu2": 0, "gelu_tanh": 1, "silu": 2, "relu": 3}


def delta_state_floats(H: int, d: int, e: int) -> int:
    """Floats of a sequence's delta-rule state (the key dims padded to the lanes' shares)."""
    return int(_lib.load().he_delta_state_floats(H, d, e))


def delta_workspace_floats(rows: int, H: int, G: int, d: int) -> int:
    """Floats of the rows delta_scan prepares before it walks them (unit vectors, gates)."""
    return int(_lib.load().he_delta_workspace_floats(rows, H, G, d))


@_op("delta_scan")
def delta_scan(y, q, k, v, ba, a_log, dt_bias, state, state_offset: int, cu_seqlens, seq_slot, rows: int,
               num_seqs: int, H: int, G: int, d: int, e: int, q_scale: float, unit_eps: float, workspace=None) -> None:
    """y (fp32 [rows, H e]) = the gated delta rule over q, k [rows, G d] and v [rows, H e] (views of rows of one
    buffer, unit stride along the columns), ba (fp32 [rows, 2 H]: write strengths, then decay inputs, both before
    their sigmoid / softplus) and per head a_log, dt_bias; the state [H][e][d'] lives at byte state_offset of a
    sequence's row of `state` and is carried on. workspace: fp32, delta_workspace_floats elements or more (None: made here)."""
    _need(y, "y", torch.float32, (None, H * e))
    _need(ba, "ba", torch.float32, (None, 2 * H))
    if workspace is None:
        workspace = torch.empty(max(4, delta_workspace_floats(rows, H, G, d)), dtype=torch.float32, device=y.device)
    _need(workspace, "workspace", torch.float32)
    stride = q.stride(0)
    for name, t, width in (("q", q, G * d), ("k", k, G * d), ("v", v, H * e)):
        if not t.is_cuda or t.dtype != q.dtype or t.dim() != 2 or t.shape[1] != width or t.stride(1) != 1 \
                or t.stride(0) != stride or t.shape[0] < rows:
            raise ValueError(f"delta_scan: {name} must be a [rows, {width}] view of rows {stride} elements apart")
    _need(a_log, "a_log", None, (H,))
    _need(dt_bias, "dt_bias", a_log.dtype, (H,))
    if y.shape[0] < rows or ba.shape[0] < rows:
        raise ValueError("delta_scan: buffers smaller than the row count")
    if state.dtype != torch.uint8 or state.dim() != 2 or state.stride(1) != 1 \
            or state.shape[1] < state_offset + 4 * delta_state_floats(H, d, e):
        raise ValueError("delta_scan: state must be uint8 [slots, bytes] with room for the heads' matrices")
    _need(cu_seqlens, "cu_seqlens", torch.int32)
    _need(seq_slot, "seq_slot", torch.int32)
    if cu_seqlens.numel() < num_seqs + 1 or seq_slot.numel() < num_seqs:
        raise ValueError("delta_scan: metadata shorter than the step")
    L = _lib.load()
    _lib.check(L.he_delta_scan(y.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), stride, ba.data_ptr(),
                               a_log.data_ptr(), dt_bias.data_ptr(), dtype_code(a_log.dtype), state.data_ptr(),
                               state.stride(0), state_offset, cu_seqlens.data_ptr(), seq_slot.data_ptr(), rows, num_seqs,
                               H, G, d, e, float(q_scale), float(unit_eps), workspace.data_ptr(), workspace.numel(),
                               dtype_code(q.dtype), _stream()))


@_op("add_group_normed")
def add_group_normed(resid_f32, delta, weight, groups: int, eps: float, delta_scale: float, out, rows: int, *,
                     next_weight=None, next_groups: int = 1, next_eps: float = 0.0) -> None:
    """resid += delta_scale * gn(delta), gn the RMS norm in `groups` equal consecutive parts of the row times weight
    (delta None: nothing is added); then, with out, out = gn'(resid) by (next_weight, next_groups, next_eps), or resid
    itself in out's dtype where next_weight is None."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    if delta is not None:
        _need(delta, "delta", None, (None, D))
        _need(weight, "weight", None, (D,))
    if out is not None:
        _need(out, "out", None, (None, D))
    if next_weight is not None:
        _need(next_weight, "next_weight", weight.dtype if delta is not None else None, (D,))
    if resid_f32.shape[0] < rows or (delta is not None and delta.shape[0] < rows) or (out is not None and out.shape[0] < rows):
        raise ValueError("add_group_normed: buffers smaller than the row count")
    w = weight if delta is not None else next_weight
    L = _lib.load()
    _lib.check(L.he_add_group_normed(resid_f32.data_ptr(), _ptr(delta), dtype_code(delta.dtype) if delta is not None else F32,
                                     _ptr(weight) if delta is not None else None, dtype_code(w.dtype) if w is not None else F32,
                                     int(groups), float(eps), float(delta_scale), _ptr(out),
                                     dtype_code(out.dtype) if out is not None else F32, _ptr(next_weight), int(next_groups),
                                     float(next_eps), rows, D, _stream()))


@_op("polynorm")
def polynorm(out, x, numbers, rows: int, eps: float) -> None:
    """out[r] = a N(z) + b N(z^2) + c N(z^3) + e over row r of x, powers element by element, N the division by the root
    mean square (eps inside the root), numbers = (a, b, c, e). out may be x."""
    W = x.shape[-1]
    _need(x, "x", None, (None, W))
    _need(out, "out", x.dtype, (None, W))
    _need(numbers, "numbers", None, (4,))
    if min(x.shape[0], out.shape[0]) < rows:
        raise ValueError("polynorm: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_polynorm(out.data_ptr(), x.data_ptr(), numbers.data_ptr(), dtype_code(numbers.dtype), rows, W,
                             float(eps), dtype_code(x.dtype), _stream()))


@_op("qk_head_norm")
def qk_head_norm(out, x, q_weight, k_weight, H: int, G: int, d: int, eps: float, rows: int, copy_v: bool = False) -> None:
    """x [rows, (H + G) d or wider]: every q head (the first H stretches of d) and every k head (the next G) is
    divided by its own root mean square and multiplied by q_weight / k_weight [d], into the same columns of out
    (which may be x); copy_v: the k heads as they were before the norm become the G stretches of out behind them (the
    values are the keys)."""
    for name, t, cols in (("x", x, (H + G) * d), ("out", out, (H + G + (G if copy_v else 0)) * d)):
        if not t.is_cuda or t.dtype != x.dtype or t.dim() != 2 or t.stride(1) != 1 or t.shape[0] < rows or t.shape[1] < cols:
            raise ValueError(f"qk_head_norm: {name} must be [rows, {cols} or wider] with unit stride along the columns")
    _need(q_weight, "q_weight", None, (d,))
    _need(k_weight, "k_weight", q_weight.dtype, (d,))
    L = _lib.load()
    _lib.check(L.he_qk_head_norm(out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), q_weight.data_ptr(),
                                 k_weight.data_ptr(), dtype_code(q_weight.dtype), H, G, d, float(eps), int(copy_v), rows,
                                 dtype_code(x.dtype), _stream()))


@_op("depth_mix")
def depth_mix(resid_f32, kept_f32, coeffs, n: int, rows: int) -> None:
    """kept[n - 1] = resid; resid = sum_{j < n} coeffs[j] * kept[j] (fp32, added in ascending j). kept: fp32
    [n or more, rows of the step, D]; resid: fp32 [rows, D]."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    _need(kept_f32, "kept", torch.float32)
    _need(coeffs, "coeffs")
    if kept_f32.dim() != 3 or kept_f32.shape[0] < n or kept_f32.shape[2] != D or kept_f32.shape[1] < rows \
            or resid_f32.shape[0] < rows or coeffs.numel() < n or n < 1:
        raise ValueError("depth_mix: kept must be [n or more, rows, D] and coeffs hold n numbers")
    L = _lib.load()
    _lib.check(L.he_depth_mix(resid_f32.data_ptr(), kept_f32.data_ptr(), kept_f32.stride(0), coeffs.data_ptr(),
                              dtype_code(coeffs.dtype), n, rows * D, _stream()))


@_op("gated_add")
def gated_add(out, a, b, x, gate_weight, rows: int) -> None:
    """out[r] = a[r] + sigmoid(x[r] . gate_weight) * b[r]; the dot product in fp32."""
    D, Dx = a.shape[-1], x.shape[-1]
    _need(a, "a", None, (None, D))
    _need(b, "b", a.dtype, (None, D))
    _need(out, "out", a.dtype, (None, D))
    _need(x, "x", a.dtype, (None, Dx))
    _need(gate_weight, "gate_weight")
    if gate_weight.numel() != Dx or min(a.shape[0], b.shape[0], out.shape[0], x.shape[0]) < rows:
        raise ValueError("gated_add: buffers smaller than the row count, or a gate of another width")
    L = _lib.load()
    _lib.check(L.he_gated_add(out.data_ptr(), a.data_ptr(), b.data_ptr(), x.data_ptr(), gate_weight.data_ptr(),
                              dtype_code(gate_weight.dtype), rows, D, Dx, dtype_code(a.dtype), _stream()))


@_op("head_product")
def head_product(out, x, w, rows: int) -> None:
    """out[r, h, :] = x[r, h, :] @ w[h] for views out [rows, H, N] and x [rows, H, K] (unit stride along the last
    axis, any row and head strides) and w [H, K, N]; fp32 sums in ascending k."""
    H, K, N = w.shape
    _need(w, "w")
    for name, t, last in (("x", x, K), ("out", out, N)):
        if not t.is_cuda or t.dtype != x.dtype or t.dim() != 3 or t.shape[1] != H or t.shape[2] != last \
                or t.stride(2) != 1 or t.shape[0] < rows:
            raise ValueError(f"head_product: {name} must be a [rows, {H}, {last}] view with unit stride along the last axis")
    L = _lib.load()
    _lib.check(L.he_head_product(out.data_ptr(), out.stride(0), out.stride(1), x.data_ptr(), x.stride(0), x.stride(1),
                                 w.data_ptr(), dtype_code(w.dtype), rows, H, K, N, dtype_code(x.dtype), _stream()))


@_op("latent_pack")
def latent_pack(qkv, q, down, rows: int, H: int, d: int, r: int, rank: int) -> None:
    """qkv [rows, H (r + rank) + (r + rank) + rank]: head h's first r columns = the last r of q[row, h] (q [rows, H (d + r)]),
    the key = [down[row, rank:rank + r] | down[row, :rank]], the value = down[row, :rank] (down: a view [rows, rank + r])."""
    hd = r + rank
    _need(qkv, "qkv", None, (None, (H + 1) * hd + rank))
    _need(q, "q", qkv.dtype, (None, H * (d + r)))
    if not down.is_cuda or down.dtype != qkv.dtype or down.dim() != 2 or down.shape[1] != rank + r or down.stride(1) != 1 \
            or min(down.shape[0], q.shape[0], qkv.shape[0]) < rows:
        raise ValueError("latent_pack: down must be a [rows, rank + r] view in qkv's dtype")
    L = _lib.load()
    _lib.check(L.he_latent_pack(qkv.data_ptr(), q.data_ptr(), down.data_ptr(), down.stride(0), rows, H, d, r, rank,
                                dtype_code(qkv.dtype), _stream()))


@_op("add_normed")
def add_normed(resid_f32, delta, post_weight, post_eps: float, next_weight, next_eps: float, out, rows: int) -> None:
    """resid += rmsnorm(delta) * post_weight (post_weight None: += delta; delta None: nothing is added); then,
    with out, out = rmsnorm(resid) * next_weight (next_weight None: out = resid in out's dtype)."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    if resid_f32.numel() < rows * D:
        raise ValueError("add_normed: resid smaller than the row count")
    w_dtype = None
    for name, w in (("post_weight", post_weight), ("next_weight", next_weight)):
        if w is not None:
            _need(w, name, w_dtype, (D,))
            w_dtype = w.dtype
    for name, t in (("delta", delta), ("out", out)):
        if t is not None:
            _need(t, name)
            if t.shape[-1] != D or t.numel() < rows * D:
                raise ValueError(f"add_normed: {name} does not match [rows, {D}]")
    L = _lib.load()
    _lib.check(L.he_add_normed(resid_f32.data_ptr(), _ptr(delta), dtype_code(delta.dtype) if delta is not None else F32,
                               _ptr(post_weight), float(post_eps), _ptr(next_weight), float(next_eps),
                               dtype_code(w_dtype) if w_dtype is not None else F32, _ptr(out),
                               dtype_code(out.dtype) if out is not None else F32, rows, D, _stream()))


@_op("unary_act")
def unary_act(out, x, rows: int, kind: str) -> None:
    """out[rows, W] = act(x[rows, W]); kind: relu2, gelu_tanh, silu, relu. In place when out is x."""
    _need(out, "out", x.dtype)
    _need(x, "x")
    W = x.shape[-1]
    if out.shape[-1] != W or min(out.numel(), x.numel()) < rows * W:
        raise ValueError("unary_act: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_unary_act(out.data_ptr(), x.data_ptr(), rows * W, ACT_KINDS[kind], dtype_code(x.dtype), _stream()))


@_op("token_gate")
def token_gate(out, x, table, ids, rows: int, offset: int, kind: str) -> None:
    """out[r, j] = act(x[r, j]) * table[ids[r], offset + j] for the W columns of x."""
    _need(x, "x")
    W = x.shape[-1]
    _need(out, "out", x.dtype, (None, W))
    _need(table, "table")
    _need(ids, "ids", torch.int32)
    if table.dim() != 2 or offset < 0 or offset + W > table.shape[1]:
        raise ValueError("token_gate: the stretch does not lie inside a row of the table")
    if min(out.shape[0], x.shape[0], ids.numel()) < rows:
        raise ValueError("token_gate: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_token_gate(out.data_ptr(), x.data_ptr(), table.data_ptr(), ids.data_ptr(), rows, W, table.shape[1],
                               offset, table.shape[0], ACT_KINDS[kind], dtype_code(x.dtype), dtype_code(table.dtype),
                               _stream()))


@_op("sigmoid_gate")
def sigmoid_gate(x, gate, rows: int, H: int, hd: int, vd: int, scale: float = 1.0) -> None:
    """x[r, h, d] *= sigmoid(gate[r, h * vd + d]) * scale for d < vd; x [rows, H * hd], gate a view [rows, H * vd]
    of wider rows."""
    _need(x, "x", None, (None, H * hd))
    if gate.dtype != x.dtype or gate.dim() != 2 or gate.shape[1] != H * vd or gate.stride(1) != 1:
        raise ValueError("sigmoid_gate: gate must be a [rows, H * vd] view in x's dtype")
    if min(x.shape[0], gate.shape[0]) < rows or hd < vd:
        raise ValueError("sigmoid_gate: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_sigmoid_gate(x.data_ptr(), gate.data_ptr(), gate.stride(0), rows, H, hd, vd, float(scale),
                                 dtype_code(x.dtype), _stream()))


@_op("scaled_sum")
def scaled_sum(out, a, b, rows: int, sa: float, sb: float) -> None:
    """out = sa * a + sb * b over [rows, D]."""
    _need(a, "a")
    D = a.shape[-1]
    _need(b, "b", a.dtype, (None, D))
    _need(out, "out", a.dtype, (None, D))
    if min(out.shape[0], a.shape[0], b.shape[0]) < rows:
        raise ValueError("scaled_sum: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_scaled_sum(out.data_ptr(), a.data_ptr(), b.data_ptr(), rows * D, float(sa), float(sb),
                               dtype_code(a.dtype), _stream()))


def mlstm_state_floats(H: int, dk: int, dv: int) -> int:
    """Floats of a sequence's matrix memory (S with padded key dims, and n and m once a workgroup)."""
    return int(_lib.load().he_mlstm_state_floats(H, dk, dv))


@_op("mlstm_gates")
def mlstm_gates(out, x, bias, rows: int, H: int, cap: float) -> None:
    """out fp32 [rows, 2 H] = the logarithms of the input gates and of the forget gates from x fp32 [rows, 2 H]."""
    _need(out, "out", torch.float32, (None, 2 * H))
    _need(x, "x", torch.float32, (None, 2 * H))
    if bias is not None:
        _need(bias, "bias", None, (2 * H,))
    if min(out.shape[0], x.shape[0]) < rows:
        raise ValueError("mlstm_gates: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_mlstm_gates(out.data_ptr(), x.data_ptr(), _ptr(bias), dtype_code(bias.dtype) if bias is not None else F32,
                                rows, H, float(cap), _stream()))


@_op("mlstm_scan")
def mlstm_scan(y, q, k, v, gates, state, state_offset: int, cu_seqlens, seq_slot, rows: int, num_seqs: int,
               H: int, dk: int, dv: int, q_scale: float, raw_gates: bool = False, gate_bias=None, cap: float = 0.0) -> None:
    """y (fp32 [rows, H dv]) = the matrix memory's answers to q, after each row's k and v went in under the
    row's gates (gates: fp32 [rows, 2 H], the logarithms). q, k [rows, H dk] and v [rows, H dv] are views of
    the same wider rows; the memory lives at byte state_offset of a sequence's row of `state` and is carried on.
    raw_gates: `gates` holds the pre-activations, and the kernel forms the logarithms itself from them, gate_bias
    ([2 H] or None) and cap, with mlstm_gates' arithmetic."""
    _need(y, "y", torch.float32, (None, H * dv))
    _need(gates, "gates", torch.float32, (None, 2 * H))
    stride = q.stride(0)
    for name, t, w in (("q", q, H * dk), ("k", k, H * dk), ("v", v, H * dv)):
        if t.dtype != q.dtype or t.dim() != 2 or t.shape[1] != w or t.stride(1) != 1 or t.stride(0) != stride \
                or t.shape[0] < rows:
            raise ValueError(f"mlstm_scan: {name} must be a [rows, {w}] view of the rows q lies in")
    if y.shape[0] < rows or gates.shape[0] < rows:
        raise ValueError("mlstm_scan: buffers smaller than the row count")
    if state.dtype != torch.uint8 or state.dim() != 2 or state.stride(1) != 1 \
            or state.shape[1] < state_offset + 4 * mlstm_state_floats(H, dk, dv):
        raise ValueError("mlstm_scan: state must be uint8 [slots, bytes] with room for the memory")
    _need(cu_seqlens, "cu_seqlens", torch.int32)
    _need(seq_slot, "seq_slot", torch.int32)
    if cu_seqlens.numel() < num_seqs + 1 or seq_slot.numel() < num_seqs:
        raise ValueError("mlstm_scan: metadata shorter than the step")
    if gate_bias is not None:
        _need(gate_bias, "gate_bias", None, (2 * H,))
    L = _lib.load()
    _lib.check(L.he_mlstm_scan(y.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), stride, gates.data_ptr(),
                               state.data_ptr(), state.stride(0), state_offset, cu_seqlens.data_ptr(),
                               seq_slot.data_ptr(), rows, num_seqs, H, dk, dv, float(q_scale), dtype_code(q.dtype),
                               int(raw_gates), _ptr(gate_bias), dtype_code(gate_bias.dtype) if gate_bias is not None else F32,
                               float(cap), _stream()))


@_op("route_tokens")
def route_tokens(dense, ids, weights, logits, correction, rows: int, real: int, groups: int, keep: int,
                 top: int, scale: float, *, x=None, router=None, normalize: bool = False) -> None:
    """The choice of `top` of E router outputs per row (logits fp32 [rows, E]; or logits None and the kernel
    forms them in fp32 from the rows x [rows, D] and the router's matrix, fp32 [E, D]): softmax scores s, the
    choice on s + correction inside the `keep` best of `groups` equal groups, weights s * scale. dense (fp32
    [rows, real + 1]): each expert's weight or 0, the outputs from `real` on added up in the last column;
    ids (int32) and weights (fp32) [rows, top]: the chosen outputs. normalize: the chosen outputs' weights are divided
    by their sum (times scale): the softmax over the chosen logits alone."""
    if logits is None:
        E, D = router.shape
        _need(router, "router", torch.float32)
        _need(x, "x", None, (None, D))
        if x.shape[0] < rows:
            raise ValueError("route_tokens: x has fewer rows than the step")
        return _route(dense, ids, weights, None, x, router, correction, rows, E, real, groups, keep, top, scale, normalize)
    E = logits.shape[-1]
    _need(logits, "logits", torch.float32, (None, E))
    if logits.shape[0] < rows:
        raise ValueError("route_tokens: buffers smaller than the row count")
    _route(dense, ids, weights, logits, None, None, correction, rows, E, real, groups, keep, top, scale, normalize)


def _route(dense, ids, weights, logits, x, router, correction, rows, E, real, groups, keep, top, scale, normalize=False) -> None:
    _need(dense, "dense", torch.float32, (None, real + 1))
    _need(ids, "ids", torch.int32, (None, top))
    _need(weights, "weights", torch.float32, (None, top))
    if correction is not None:
        _need(correction, "correction", None, (E,))
    if min(dense.shape[0], ids.shape[0], weights.shape[0]) < rows:
        raise ValueError("route_tokens: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_route_tokens(dense.data_ptr(), ids.data_ptr(), weights.data_ptr(), _ptr(logits),
                                 _ptr(x), dtype_code(x.dtype) if x is not None else F32, _ptr(router),
                                 router.shape[1] if router is not None else 0,
                                 _ptr(correction), dtype_code(correction.dtype) if correction is not None else F32,
                                 rows, E, real, groups, keep, top, float(scale), int(normalize), _stream()))


@_op("routed_act")
def routed_act(out, gate_up, dense, h, rows: int, real: int, inter: int, *, alpha: float = 1.0,
               limit: float = 0.0, up_shift: float = 0.0) -> None:
    """out[rows, real * inter + extra]: the experts' gated activations (gate_up [rows, 2 real inter], gate and
    up alternating) times their weights dense[row, e]; the last extra = h.shape[1] columns (h None: none)
    are dense[row, real] * h."""
    extra = 0 if h is None else h.shape[1]
    _need(out, "out", None, (None, real * inter + extra))
    _need(gate_up, "gate_up", out.dtype, (None, 2 * real * inter))
    _need(dense, "dense", torch.float32, (None, real + 1))
    if h is not None:
        _need(h, "h", out.dtype)
    if min(out.shape[0], gate_up.shape[0], dense.shape[0], rows if h is None else h.shape[0]) < rows:
        raise ValueError("routed_act: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_routed_act(out.data_ptr(), gate_up.data_ptr(), dense.data_ptr(), _ptr(h), rows, real, inter,
                               extra, dtype_code(out.dtype), float(alpha), float(limit), float(up_shift), _stream()))


@_op("chosen_experts")
def chosen_experts(out, h_scratch, x, gate_up, down, ids, weights, dense, rows: int, real: int, inter: int, *,
                   alpha: float = 1.0, limit: float = 0.0, up_shift: float = 0.0) -> None:
    """For a step of very few bf16 rows: out[rows, D] = the weighted sum of the chosen experts' results alone
    (ids, weights [rows, top] and dense [rows, real + 1] as route_tokens leaves them), read from the fused matrices
    of the products over all experts: gate_up [2 real inter, D] (gate and up alternating), down [D, real inter (+ D)].
    The identity experts' share dense[row, real] * x is added. h_scratch: bf16 [rows * top, inter]."""
    D = x.shape[1]
    top = ids.shape[1]
    for name, t in (("out", out), ("h_scratch", h_scratch), ("x", x), ("gate_up", gate_up), ("down", down)):
        _need(t, name, torch.bfloat16)
    _need(ids, "ids", torch.int32, (None, top))
    _need(weights, "weights", torch.float32, (None, top))
    _need(dense, "dense", torch.float32, (None, real + 1))
    if tuple(gate_up.shape) != (2 * real * inter, D) or down.shape[0] != D or down.shape[1] < real * inter:
        raise ValueError("chosen_experts: the fused matrices do not match the sizes")
    if min(out.shape[0], x.shape[0], ids.shape[0], weights.shape[0], dense.shape[0]) < rows or out.shape[1] != D \
            or h_scratch.numel() < rows * top * inter:
        raise ValueError("chosen_experts: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_chosen_experts(out.data_ptr(), h_scratch.data_ptr(), x.data_ptr(), gate_up.data_ptr(), down.data_ptr(),
                                   down.stride(0), ids.data_ptr(), weights.data_ptr(), dense.data_ptr(), rows, top, real,
                                   inter, D, float(alpha), float(limit), float(up_shift), _stream()))


@_op("diff_heads")
def diff_heads(out, attn, rows: int, H: int, G: int, hd: int, vd: int, lam: float, post: float, eps: float) -> None:
    """out[rows, H, vd] = rms(a1 - lam * a2) * post per head, a1 and a2 the outputs of the two score maps in
    attn [rows, 2 H, hd] (head order [kv head][map][query head of the group])."""
    _need(attn, "attn")
    _need(out, "out", attn.dtype)
    if attn.numel() < rows * 2 * H * hd or out.numel() < rows * H * vd:
        raise ValueError("diff_heads: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_diff_heads(out.data_ptr(), attn.data_ptr(), rows, H, G, hd, vd, float(lam), float(post),
                               float(eps), dtype_code(out.dtype), _stream()))


def _check_attention(out, q, kpool, vpool, page_table, rows, H, KVH, hd):
    _need(q, "q")
    _need(out, "out", q.dtype)
    _need(kpool, "kpool", q.dtype, (None, KVH, layout.k_page_elems(hd)))
    _need(vpool, "vpool", q.dtype, (None, KVH, layout.v_page_elems(hd)))
    _need(page_table, "page_table", torch.int32)
    if page_table.dim() != 2:
        raise ValueError("attention: page_table must be [slots, blocks]")
    if q.numel() < rows * H * hd or out.numel() < rows * H * hd:
        raise ValueError("attention: q/out smaller than the row count")


@_op("attention_plain")
def attention_plain(out, q, kpool, vpool, positions, row_seq, seq_slot, page_table, rows: int,
                    H: int, KVH: int, hd: int, window: int, scale: float, most_keys: int = 0,
                    workspace=None, *, chunk: int = 0, sinks=None, gate=None, slopes=None) -> None:
    """most_keys: a bound on the keys any sequence holds after the step, and workspace: fp32, of
    attention_plain_workspace_floats elements or more: the pages of a query then run in parallel
    (a step of few queries over many keys); the result is the same bit for bit without them.
    chunk > 0: a query sees the keys of its own chunk of so many positions only (counted from
    position 0). sinks [H]: a number a head that joins the softmax's denominator as exp(sink).
    gate: a view [rows, H] of q's dtype (unit stride along heads, any row stride): the head's output
    is multiplied by sigmoid(gate). slopes (fp32 [H]): the score of key j for the query at p loses
    slopes[h] * (p - j)."""
    _check_attention(out, q, kpool, vpool, page_table, rows, H, KVH, hd)
    gate_ptr, gate_stride = _gate_view(gate, q, rows, H)
    if sinks is not None:
        _need(sinks, "sinks", shape=(H,))
    if slopes is not None:
        _need(slopes, "slopes", torch.float32, (H,))
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    for name, t in (("positions", positions), ("row_seq", row_seq), ("seq_slot", seq_slot)):
        _need(t, name, torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("attention: metadata shorter than the row count")
    L = _lib.load()
    _lib.check(L.he_attention_plain(
        out.data_ptr(), q.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), positions.data_ptr(),
        row_seq.data_ptr(), seq_slot.data_ptr(), page_table.data_ptr(), page_table.shape[1],
        kpool.shape[0], rows, H, KVH, hd, window, int(chunk), float(scale), _ptr(sinks),
        dtype_code(sinks.dtype) if sinks is not None else F32, gate_ptr, gate_stride,
        dtype_code(q.dtype), int(most_keys),
        _ptr(workspace), workspace.numel() if workspace is not None else 0, _ptr(slopes), _stream()))


def _gate_view(gate, q, rows: int, H: int):
    """(pointer, row stride in elements) of a gate view [rows or more, H], or (None, 0)."""
    if gate is None:
        return None, 0
    if not gate.is_cuda or gate.dtype != q.dtype or gate.dim() != 2 or gate.shape[1] != H \
            or gate.shape[0] < rows or gate.stride(1) != 1:
        raise ValueError(f"attention: gate must be a view [rows, {H}] of {q.dtype} with unit stride along heads")
    return gate.data_ptr(), gate.stride(0)


def attention_plain_workspace_floats(rows: int, H: int, hd: int, most_keys: int, window: int,
                                     chunk: int = 0) -> int:
    return int(_lib.load().he_attention_plain_workspace_floats(rows, H, hd, most_keys, window, chunk))


def attention_decode_workspace_floats(rows: int, H: int, KVH: int, hd: int, max_keys: int) -> int:
    return int(_lib.load().he_attention_decode_workspace_floats(rows, H, KVH, hd, max_keys))


@_op("attention_decode")
def attention_decode(out, q, kpool, vpool, positions, row_seq, seq_slot, page_table, rows: int,
                     H: int, KVH: int, hd: int, window: int, scale: float, max_keys: int,
                     workspace, *, chunk: int = 0, sinks=None, gate=None, slopes=None) -> None:
    """chunk, sinks, gate, slopes: as attention_plain takes them."""
    _check_attention(out, q, kpool, vpool, page_table, rows, H, KVH, hd)
    _need(q, "q", torch.bfloat16)
    gate_ptr, gate_stride = _gate_view(gate, q, rows, H)
    if sinks is not None:
        _need(sinks, "sinks", shape=(H,))
    if slopes is not None:
        _need(slopes, "slopes", torch.float32, (H,))
    for name, t in (("positions", positions), ("row_seq", row_seq), ("seq_slot", seq_slot)):
        _need(t, name, torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("attention: metadata shorter than the row count")
    _need(workspace, "workspace", torch.float32)
    L = _lib.load()
    _lib.check(L.he_attention_decode_bf16(
        out.data_ptr(), q.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), positions.data_ptr(),
        row_seq.data_ptr(), seq_slot.data_ptr(), page_table.data_ptr(), page_table.shape[1],
        kpool.shape[0], rows, H, KVH, hd, window, float(scale), max_keys, workspace.data_ptr(),
        workspace.numel(), int(chunk), _ptr(sinks), dtype_code(sinks.dtype) if sinks is not None else F32,
        gate_ptr, gate_stride, _ptr(slopes), _stream()))


def attention_decode_fused_ok(H: int, KVH: int, hd: int, rotary_dim: int) -> bool:
    return int(_lib.load().he_attention_decode_fused_ok(H, KVH, hd, rotary_dim)) > 0


def attention_decode_fused_workspace_floats(rows: int, H: int, KVH: int, hd: int, max_keys: int,
                                           spread: bool = False) -> int:
    return int(_lib.load().he_attention_decode_fused_workspace_floats(rows, H, KVH, hd, max_keys, int(spread)))


@_op("attention_decode_fused")
def attention_decode_fused(out, qkv, bias, kpool, vpool, positions, row_seq, seq_slot, page_table,
                           inv_freq, rotary_dim: int, rows: int, H: int, KVH: int, hd: int,
                           window: int, scale: float, max_keys: int, write_kv: bool,
                           workspace, out_pieces: bool = False, spread: bool = False) -> None:
    """One-token steps in one launch: bias, rotation of q and of the new key, cache write,
    attention over the cache, merge. spread: one sequence has several times the keys of the
    others (every sequence's keys are then cut across more workgroups; the workspace is asked for
    with the same flag). qkv: bf16 [rows, (H + 2 KVH) hd] without bias, or fp32 [slices, rows, width]:
    the sums of the projection's K slices as gemm_rows leaves them; q columns
    alone where the run reads another run's cache (write_kv False). out_pieces: out is written
    piece-major for exactly `rows` rows (see :func:`to_pieces`). seq_slot None: page_table has a row
    per row of the step ([rows or more, blocks]: the page numbers of the row's sequence), not a
    row per slot; the kernel then asks for them at its start, without the chain through the slot."""
    width = (H + 2 * KVH) * hd if write_kv else H * hd
    _need(out, "out", torch.bfloat16)
    slices, slice_stride = 0, 0
    if qkv.dtype == torch.float32:
        # the fp32 sums of the projection's K slices, [slices, rows of the product, width] (gemm_rows):
        # the kernel adds them itself, in slice order, and rounds as splitk_reduce would have
        _need(qkv, "qkv (K slices)", torch.float32)
        if qkv.dim() != 3 or qkv.shape[2] != width or qkv.shape[1] < rows:
            raise ValueError("attention_decode_fused: K slices [slices, rows, width] do not match the head sizes and row count")
        slices, slice_stride = qkv.shape[0], qkv.shape[1] * width
    else:
        _need(qkv, "qkv", torch.bfloat16)
        if qkv.dim() != 2 or qkv.shape[1] != width or qkv.shape[0] < rows:
            raise ValueError("attention_decode_fused: qkv does not match the head sizes and row count")
    if out.numel() < rows * H * hd:
        raise ValueError("attention_decode_fused: out does not match the head sizes and row count")
    if out_pieces:
        _need(out, "out", shape=pieces_shape(rows, H * hd))
    _need(kpool, "kpool", torch.bfloat16, (None, KVH, layout.k_page_elems(hd)))
    _need(vpool, "vpool", torch.bfloat16, (None, KVH, layout.v_page_elems(hd)))
    _need(page_table, "page_table", torch.int32)
    for name, t in (("positions", positions), ("row_seq", row_seq)) + ((("seq_slot", seq_slot),) if seq_slot is not None else ()):
        _need(t, name, torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows or page_table.dim() != 2:
        raise ValueError("attention_decode_fused: metadata shorter than the row count")
    if seq_slot is None and page_table.shape[0] < rows:
        raise ValueError("attention_decode_fused: a page table by rows needs a row per row of the step")
    if bias is not None:
        _need(bias, "bias", shape=(width,))
    _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    L = _lib.load()
    _lib.check(L.he_attention_decode_fused_bf16(
        out.data_ptr(), qkv.data_ptr() if not slices else None, qkv.data_ptr() if slices else None, slices,
        slice_stride, width, _ptr(bias),
        dtype_code(bias.dtype) if bias is not None else F32, kpool.data_ptr(), vpool.data_ptr(),
        positions.data_ptr(), row_seq.data_ptr(), _ptr(seq_slot), page_table.data_ptr(),
        page_table.shape[1], kpool.shape[0], inv_freq.data_ptr(), rotary_dim, rows, H, KVH, hd,
        window, float(scale), max_keys, int(spread), int(write_kv), int(out_pieces), _ptr(workspace),
        workspace.numel() if workspace is not None else 0, _stream()))


def attention_prefill_parts(num_seqs: int, max_q_len: int, H: int, hd: int, most_keys: int) -> int:
    """Parts the library would cut the keys of this prompt step into (1: none): more than one
    for a step of few queries against many keys, which would otherwise leave most of the chip idle."""
    return int(_lib.load().he_attention_prefill_parts(num_seqs, max_q_len, H, hd, most_keys))


def attention_prefill_workspace_floats(total_rows: int, H: int, hd: int, parts: int) -> int:
    return int(_lib.load().he_attention_prefill_workspace_floats(total_rows, H, hd, parts))


@_op("attention_prefill")
def attention_prefill(out, q, kpool, vpool, cu_seqlens, seq_slot, seq_start, page_table,
                      num_seqs: int, max_q_len: int, total_rows: int, H: int, KVH: int, hd: int,
                      window: int, scale: float, kernel: int = 0, parts: int = 1, workspace=None, *,
                      chunk: int = 0, sinks=None, gate=None, slopes=None) -> None:
    """kernel: 0 leaves the choice to the library (by head size and prompt length); 1 or 2
    name it: 16 queries a wavefront with operands from global memory, or 32 queries a
    wavefront with the pages shared through LDS (head sizes up to 128). parts > 1 (kernel 2):
    the keys in that many parts side by side, joined by a second launch; the workspace holds
    attention_prefill_workspace_floats() floats. chunk, sinks, gate, slopes: as attention_plain takes them."""
    _check_attention(out, q, kpool, vpool, page_table, total_rows, H, KVH, hd)
    _need(q, "q", torch.bfloat16)
    gate_ptr, gate_stride = _gate_view(gate, q, total_rows, H)
    if sinks is not None:
        _need(sinks, "sinks", shape=(H,))
    if slopes is not None:
        _need(slopes, "slopes", torch.float32, (H,))
    for name, t in (("cu_seqlens", cu_seqlens), ("seq_slot", seq_slot), ("seq_start", seq_start)):
        _need(t, name, torch.int32)
    if cu_seqlens.numel() < num_seqs + 1 or seq_slot.numel() < num_seqs or seq_start.numel() < num_seqs:
        raise ValueError("attention_prefill: metadata shorter than the sequence count")
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    L = _lib.load()
    _lib.check(L.he_attention_prefill_bf16(
        out.data_ptr(), q.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), cu_seqlens.data_ptr(),
        seq_slot.data_ptr(), seq_start.data_ptr(), page_table.data_ptr(), page_table.shape[1],
        kpool.shape[0], num_seqs, max_q_len, H, KVH, hd, window, float(scale), int(kernel),
        total_rows, int(parts), _ptr(workspace), workspace.numel() if workspace is not None else 0,
        int(chunk), _ptr(sinks), dtype_code(sinks.dtype) if sinks is not None else F32, gate_ptr, gate_stride,
        _ptr(slopes), _stream()))


@_op("argmax_rows")
def argmax_rows(out_i32, logits, rows: int) -> None:
    _need(logits, "logits", torch.float32)
    _need(out_i32, "out", torch.int32)
    V = logits.shape[-1]
    if logits.numel() < rows * V or out_i32.numel() < rows:
        raise ValueError("argmax_rows: buffers smaller than the row count")
    L = _lib.load()
    need = int(L.he_argmax_workspace_bytes(rows, V))
    ws = torch.empty(need, dtype=torch.uint8, device=logits.device) if need else None
    _lib.check(L.he_argmax_rows(out_i32.data_ptr(), logits.data_ptr(), rows, V, V, _ptr(ws), need, _stream()))


@_op("apply_penalties")
def apply_penalties(logits, rows: int, ids, counts, offsets, rep: float, freq: float,
                    pres: float) -> None:
    _need(logits, "logits", torch.float32)
    for name, t in (("ids", ids), ("counts", counts), ("offsets", offsets)):
        _need(t, name, torch.int32)
    V = logits.shape[-1]
    if logits.numel() < rows * V or offsets.numel() < rows + 1 or ids.numel() != counts.numel():
        raise ValueError("apply_penalties: buffers do not match the row count")
    L = _lib.load()
    _lib.check(L.he_apply_penalties(logits.data_ptr(), rows, V, V, ids.data_ptr(),
                                    counts.data_ptr(), offsets.data_ptr(), float(rep), float(freq),
                                    float(pres), _stream()))


PENALTY_WINDOW_MAX = 4096


@_op("apply_penalties_window")
def apply_penalties_window(logits, rows: int, window, appended, last_ids, rep: float, freq: float,
                           pres: float) -> None:
    """The penalties of apply_penalties from a ring of recent tokens on the device: window int32
    [rows, W] (token number n at n % W), appended int32 [rows] (tokens ever appended). last_ids
    (int32 [rows] or None) are appended first. Changes logits in place."""
    _need(logits, "logits", torch.float32)
    _need(window, "window", torch.int32)
    _need(appended, "appended", torch.int32)
    V = logits.shape[-1]
    if window.dim() != 2 or window.shape[0] < rows or appended.numel() < rows or logits.numel() < rows * V:
        raise ValueError("apply_penalties_window: buffers smaller than the row count")
    if last_ids is not None:
        _need(last_ids, "last_ids", torch.int32)
        if last_ids.numel() < rows:
            raise ValueError("apply_penalties_window: fewer ids than rows")
    L = _lib.load()
    _lib.check(L.he_apply_penalties_window(logits.data_ptr(), rows, V, V, window.data_ptr(),
                                           appended.data_ptr(), window.shape[1], _ptr(last_ids),
                                           float(rep), float(freq), float(pres), _stream()))


@_op("sample_rows")
def sample_rows(out_i32, logits, rows: int, uniforms_u32, temperature: float, top_k: int,
                top_p: float) -> None:
    _need(logits, "logits", torch.float32)
    _need(out_i32, "out", torch.int32)
    _need(uniforms_u32, "uniforms")
    if uniforms_u32.element_size() != 4 or uniforms_u32.numel() < rows:
        raise ValueError("sample_rows: uniforms must be one 32-bit word per row")
    V = logits.shape[-1]
    if logits.numel() < rows * V or out_i32.numel() < rows:
        raise ValueError("sample_rows: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_sample_rows(out_i32.data_ptr(), logits.data_ptr(), rows, V, V,
                                uniforms_u32.data_ptr(), float(temperature), int(top_k),
                                float(top_p), _stream()))
