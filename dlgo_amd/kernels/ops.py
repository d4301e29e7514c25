"""Python faces of the HIP kernels: each checks on the host what its kernel and
grid assume (device, dtype, contiguity, shapes), then launches on torch's current
stream.  There is no other implementation behind these: on a machine without the
GPU or the compiler they raise.
"""
from __future__ import annotations

import ctypes
import functools
import math
from typing import Dict, List, Optional, Sequence

import torch

from . import build

PAGE = 64   # tokens per cache page; the kernels are compiled with the same number

EPI_STORE, EPI_ACCUM_F32, EPI_SWIGLU, EPI_STORE_F32 = 0, 1, 2, 3
GEMM_AUTO, GEMM_STREAM, GEMM_TILE128, GEMM_TILE64, GEMM_TILE32, GEMM_ROWS16 = 0, 1, 2, 3, 4, 5
GEMM_FEW_ROWS = 64      # up to this many rows of x the weight-streaming kernels can be chosen
GEMM_SPLIT_FLOATS = 1 << 22   # scratch that lets gemm() share the inner size of a product out over blocks
GEMM_VERY_WIDE = 65536   # from this many weight rows on (a vocabulary: 16 blocks of 16 rows for each of 256 compute units) the tiled kernel is faster for any number of rows of x
GEMM_FEW_ROWS_WIDE = 16  # ... and up to this many when the weight has very many rows (there the tiled kernel is faster)

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels run in float32 or bfloat16, not {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)    # the handle without a Stream object around it


_raw_device = getattr(torch._C, "_cuda_getDevice", None)              # the current device without torch.cuda's start-up check


def _stream() -> ctypes.c_void_p:
    """torch's current stream on the current device, as the launches take it (asked at every launch: a recording has
    a stream of its own)."""
    if _raw_stream is not None and _raw_device is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _need(t: torch.Tensor, name: str, dtype: Optional[torch.dtype] = None, dims: Optional[int] = None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a tensor on the GPU")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, found {t.dtype}")
    if dims is not None and t.dim() != dims:
        raise KernelError(f"{name}: expected {dims} dimensions, found shape {tuple(t.shape)}")


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride (elements) of a 2-d tensor whose rows are contiguous."""
    strides = t.stride()
    if len(strides) != 2 or (strides[1] != 1 and t.shape[1] > 1):
        raise KernelError(f"{name}: expected rows that are contiguous in memory, found shape {tuple(t.shape)} strides {strides}")
    return strides[0] if t.shape[0] > 1 else max(strides[0], t.shape[1])


def _check(err: Optional[bytes]) -> None:
    if err:
        raise KernelError(err.decode())


_libs: dict = {}      # (module, defines) -> loaded library with its return types set; looked up at every launch


def _lib(module: str, defines=()):
    key = (module, tuple(defines))
    lib = _libs.get(key)
    if lib is None:
        lib = build.load(module, defines)
        for name in ("dlgo_embed", "dlgo_copy_rows", "dlgo_rmsnorm", "dlgo_rope_kv", "dlgo_gemm", "dlgo_gemm_accum_norm", "dlgo_gemm_parts", "dlgo_gemm_rows", "dlgo_gemm_rmsnorm", "dlgo_gemm_rows_leave_parts", "dlgo_gemm_rows_scaled", "dlgo_gemm_tile_leave", "dlgo_gemm_tile_scaled", "dlgo_attention_rows",
                     "dlgo_attention_prefill", "dlgo_attention_prefill_f32", "dlgo_attention_decode", "dlgo_attention_decode_f32", "dlgo_argmax", "dlgo_sample", "dlgo_bias_add", "dlgo_head_rmsnorm"):
            if hasattr(lib, name):
                getattr(lib, name).restype = ctypes.c_char_p
        _libs[key] = lib
    return lib


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] as float32."""
    _need(table, "embed table", dims=2)
    _need(ids, "token ids", torch.int32, 1)
    _need(out, "embed output", torch.float32, 2)
    n, d = ids.shape[0], table.shape[1]
    if not table.is_contiguous() or not out.is_contiguous() or tuple(out.shape) != (n, d):
        raise KernelError(f"embed: output {tuple(out.shape)} does not fit {n} tokens of width {d}")
    _check(_lib("embed").dlgo_embed(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(out), n, d, table.shape[0], _stream()))
    return out


def copy_rows(src: torch.Tensor, dst: torch.Tensor, src_rows: Optional[torch.Tensor] = None,
              dst_rows: Optional[torch.Tensor] = None, n: Optional[int] = None) -> torch.Tensor:
    """dst[dst_rows[i]] = src[src_rows[i]] for i < n (a missing list stands for i itself; n defaults to the lists'
    length, or to src's rows).  Rows of any element type whose bytes are a multiple of 4; 1-d tensors are rows of one
    element.  The lists are int32 on the device and hold row numbers inside the two tensors (the caller's duty: they
    are not read here); source and destination rows must not overlap."""
    given = dst
    if src.dim() == 1:
        src = src.unsqueeze(1)
    if dst.dim() == 1:
        dst = dst.unsqueeze(1)
    _need(src, "rows to copy", dims=2)
    _need(dst, "copied rows", src.dtype, 2)
    for name, r in (("source rows", src_rows), ("destination rows", dst_rows)):
        if r is not None:
            _need(r, name, torch.int32, 1)
    if n is None:
        n = src_rows.shape[0] if src_rows is not None else (dst_rows.shape[0] if dst_rows is not None else src.shape[0])
    es = src.element_size()
    if src.shape[1] != dst.shape[1] or (src.shape[1] * es) % 4 or n < 0 \
            or any(r is not None and r.shape[0] < n for r in (src_rows, dst_rows)) \
            or (src_rows is None and src.shape[0] < n) or (dst_rows is None and dst.shape[0] < n):
        raise KernelError(f"copy_rows: {n} rows of {tuple(src.shape)} into {tuple(dst.shape)} (rows of equal width, a multiple of 4 bytes)")
    _check(_lib("embed").dlgo_copy_rows(_ptr(src), _ptr(src_rows), _ptr(dst), _ptr(dst_rows), n, ctypes.c_longlong(src.shape[1] * es),
                                        ctypes.c_longlong(_rows(src, "rows to copy") * es), ctypes.c_longlong(_rows(dst, "copied rows") * es),
                                        _stream()))
    return given


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = rmsnorm(x[rows[r]] if rows is given else x[r]) * weight; x float32, out in its own dtype."""
    _need(x, "rmsnorm input", torch.float32, 2)
    _need(weight, "rmsnorm weight", torch.float32, 1)
    _need(out, "rmsnorm output", dims=2)
    d = x.shape[1]
    n = out.shape[0]
    if rows is not None:
        _need(rows, "rmsnorm rows", torch.int32, 1)
        if rows.shape[0] != n:
            raise KernelError("rmsnorm: one output row per gathered row")
    elif x.shape[0] != n:
        raise KernelError(f"rmsnorm: {x.shape[0]} input rows, {n} output rows")
    if weight.shape[0] != d or out.shape[1] != d or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"rmsnorm: width mismatch or strided operands (x {tuple(x.shape)}, w {tuple(weight.shape)}, out {tuple(out.shape)})")
    _check(_lib("rmsnorm").dlgo_rmsnorm(_ptr(x), _ptr(rows), _ptr(weight), _ptr(out), dtype_code(out.dtype), n, d,
                                        ctypes.c_float(eps), _stream()))
    return out


def bias_add(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y[t, n] += bias[n]; y rows in float32 or bfloat16 (row stride free), bias float32."""
    _need(y, "rows", dims=2)
    _need(bias, "bias", torch.float32, 1)
    if bias.shape[0] != y.shape[1] or not bias.is_contiguous():
        raise KernelError(f"bias_add: bias {tuple(bias.shape)} does not fit rows {tuple(y.shape)}")
    _check(_lib("rowwise").dlgo_bias_add(_ptr(y), dtype_code(y.dtype), y.shape[0], y.shape[1], _rows(y, "rows"), _ptr(bias), _stream()))
    return y


def head_rmsnorm(x: torch.Tensor, first_col: int, n_heads: int, head_dim: int, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Each of n_heads heads of head_dim consecutive elements, from column first_col on, of every row of x is RMS-normalised
    in place over its own elements and multiplied by weight [head_dim] (float32)."""
    _need(x, "rows", dims=2)
    _need(weight, "head norm weight", torch.float32, 1)
    if weight.shape[0] != head_dim or not weight.is_contiguous() or first_col < 0 or first_col + n_heads * head_dim > x.shape[1]:
        raise KernelError(f"head_rmsnorm: {n_heads} heads of {head_dim} from column {first_col} and weight {tuple(weight.shape)} do not fit rows {tuple(x.shape)}")
    _check(_lib("rowwise").dlgo_head_rmsnorm(_ptr(x), dtype_code(x.dtype), x.shape[0], _rows(x, "rows"), first_col, n_heads, head_dim,
                                             _ptr(weight), ctypes.c_float(eps), _stream()))
    return x


_cus: dict = {}


def compute_units(device=None) -> int:
    """Compute units of the device (256 on an MI355X): what the rules below count blocks against."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    if index not in _cus:
        _cus[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _cus[index]


def stream_plan(weight: torch.Tensor, t: int):
    """(waves a block, kilobytes of a row a wave takes in turn, groups of 16 weight rows a block works through) of the
    streamed products for this weight and t rows of x, or None if they do not take it."""
    if weight.dim() != 2 or weight.stride(1) != 1 or not (1 <= t <= 16):
        return None
    lib = _lib("gemm_rows", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    lib.dlgo_gemm_rows_stream_plan.restype = ctypes.c_int
    waves, turns, groups = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    ok = lib.dlgo_gemm_rows_stream_plan(dtype_code(weight.dtype), weight.shape[0], t, weight.shape[1], weight.stride(0),
                                        ctypes.byref(waves), ctypes.byref(turns), ctypes.byref(groups))
    return (waves.value, turns.value, groups.value) if ok else None


def _streams_rows(weight: torch.Tensor, t: int, kind: int, has_scratch: bool, splits: int) -> bool:
    """Whether a product of t rows with this weight goes to the kernels that stream W against a few rows of x (else to
    the tiled ones).  The rules count bytes, blocks and rows, not the sizes of a model:

      row_bytes  what a block reads of one weight row; in 128-byte pieces the tiles can load it straight into LDS, and
                 from 32 pieces (4 KB) on they can share k out over blocks, given scratch (`can_split`);
      blocks16   blocks of the streamed kernels (16 weight rows each), tiles64 those of the small tiles (64 rows each),
                 both against the device's compute units.

    Up to 16 rows stream, except: (a) so few blocks that compute units stay idle and rows long enough to share out
    (the split tiles use every unit); (b) rows that a wave takes in several turns, from 8 rows of x on, where k can be
    shared out (the streamed kernel for such rows has one group of weight rows a block, and every block reads all of
    x again: with 10 KB rows and 8 rows of x the split tiles are 10 to 30% faster, with 40 KB rows also for one row);
    (c) a matrix with 16 and more blocks a unit (a vocabulary), which streams only with up to 8 rows and a wave per
    kilobyte of a row, or when the tiles cannot load its rows.  17 to 64 rows go to the kernel that reads W into
    registers only where the tiles are few and cannot split."""
    n, k = weight.shape
    es = weight.element_size()
    row_bytes = k * es
    pieces = row_bytes // 128 if row_bytes % 128 == 0 else 0
    can_split = has_scratch and splits != 1 and pieces >= 32
    if kind != GEMM_AUTO or splits > 1:
        return kind in (GEMM_STREAM, 5, 6, 7, 8, 9, 10, 11, 15, 16, 17, 18, 19)
    cus = compute_units(weight.device)
    blocks16, tiles64 = (n + 15) // 16, (n + 63) // 64
    very_wide = blocks16 >= 16 * cus
    if t <= GEMM_FEW_ROWS_WIDE:
        plan = stream_plan(weight, t)
        waves, turns, groups = plan if plan is not None else (0, 1, 1)
        if very_wide:                                                                       # (c)
            return pieces == 0 or (t <= 8 and plan is not None and turns == 1 and waves not in (5, 7))
        if can_split and blocks16 <= cus and pieces >= 64:                                  # (a)
            return False
        if can_split and plan is not None and turns > 1 and (t >= 8 or pieces >= 256):      # (b)
            return False
        return True
    if t <= GEMM_FEW_ROWS:
        return blocks16 < 4 * cus and not (can_split and tiles64 <= cus // 2 and (pieces >= 48 or t >= 24)) and (t <= 40 or pieces == 0)
    return False


def gemm_streams(weight: torch.Tensor, rows: int, has_scratch: bool = True) -> bool:
    """Which family gemm() gives a product of `rows` rows of x with this weight when the choice is its own: the kernels
    that stream W against a few rows (True) or the tiled ones (False).  The rules are _streams_rows'."""
    return _streams_rows(weight, rows, GEMM_AUTO, has_scratch, 0)


def gemm_accum_then_norm(weight: torch.Tensor, x: torch.Tensor, residual: torch.Tensor, scratch: Optional[torch.Tensor],
                         norm_weight: torch.Tensor, eps: float, normed: torch.Tensor) -> bool:
    """residual += x @ weight.T and, beside it, normed = rmsnorm(residual) * norm_weight of the new rows, if this
    product is one whose inner size gemm() would share out over blocks (then the sum of the runs gives the norm for
    nothing).  Returns False, having done nothing, if it is not: the caller then runs gemm() and the norm."""
    _need(weight, "gemm weight", dims=2)
    _need(x, "gemm input", weight.dtype, 2)
    n, k = weight.shape
    t = x.shape[0]
    if scratch is None or t == 0 or n % 4 or n > 8192 or _streams_rows(weight, t, GEMM_AUTO, True, 0):
        return False
    _need(scratch, "gemm scratch", torch.float32, 1)
    lib = _lib("gemm", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    ldw, ldx = _rows(weight, "gemm weight"), _rows(x, "gemm input")
    splits = lib.dlgo_gemm_auto_splits(dtype_code(weight.dtype), n, t, k, ldw, ldx, ctypes.c_longlong(scratch.numel()))
    if splits <= 1:
        return False
    _need(residual, "residual rows", torch.float32, 2)
    _need(norm_weight, "norm weight", torch.float32, 1)
    _need(normed, "normed rows", weight.dtype, 2)
    if x.shape[1] != k or tuple(residual.shape) != (t, n) or tuple(normed.shape) != (t, n) or norm_weight.shape[0] != n:
        raise KernelError(f"gemm_accum_then_norm: x {tuple(x.shape)}, residual {tuple(residual.shape)}, normed {tuple(normed.shape)} "
                          f"and norm weight {tuple(norm_weight.shape)} do not fit weight {tuple(weight.shape)}")
    _check(lib.dlgo_gemm_accum_norm(_ptr(weight), _ptr(x), _ptr(residual), dtype_code(weight.dtype), n, t, k, ldw, ldx,
                                    _rows(residual, "residual rows"), splits, _ptr(scratch), ctypes.c_longlong(scratch.numel()),
                                    _ptr(norm_weight), ctypes.c_float(eps), _ptr(normed), _rows(normed, "normed rows"), _stream()))
    return True


class UnsummedRows:
    """The rows x @ weight.T as gemm_runs leaves them: `runs` float32 planes [T, N] one after the other in `scratch`, each
    the sum over one run of k; the rows themselves are the planes added in order.  A kernel that reads the rows once
    can do that sum as it reads (rope_kv does) and save the pass that would write them out."""
    __slots__ = ("scratch", "runs", "rows", "cols")

    def __init__(self, scratch, runs, rows, cols):
        self.scratch, self.runs, self.rows, self.cols = scratch, runs, rows, cols


def gemm_runs(weight: torch.Tensor, x: torch.Tensor, scratch: Optional[torch.Tensor]) -> Optional[UnsummedRows]:
    """x @ weight.T left as unsummed runs of k in `scratch`, if this product is one whose inner size gemm() would share
    out over blocks; None, having done nothing, if it is not (the caller then runs gemm())."""
    _need(weight, "gemm weight", dims=2)
    _need(x, "gemm input", weight.dtype, 2)
    n, k = weight.shape
    t = x.shape[0]
    if scratch is None or t == 0 or n % 4 or _streams_rows(weight, t, GEMM_AUTO, True, 0):
        return None
    _need(scratch, "gemm scratch", torch.float32, 1)
    if x.shape[1] != k:
        raise KernelError(f"gemm_runs: x {tuple(x.shape)} does not fit weight {tuple(weight.shape)}")
    lib = _lib("gemm", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    ldw, ldx = _rows(weight, "gemm weight"), _rows(x, "gemm input")
    splits = lib.dlgo_gemm_auto_splits(dtype_code(weight.dtype), n, t, k, ldw, ldx, ctypes.c_longlong(scratch.numel()))
    if splits <= 1:
        return None
    runs = ctypes.c_int(0)
    _check(lib.dlgo_gemm_parts(_ptr(weight), _ptr(x), dtype_code(weight.dtype), n, t, k, ldw, ldx, splits, _ptr(scratch),
                               ctypes.c_longlong(scratch.numel()), ctypes.byref(runs), _stream()))
    return UnsummedRows(scratch, runs.value, t, n)


def gemm(weight: torch.Tensor, x: torch.Tensor, out: torch.Tensor, epilogue: int = EPI_STORE,
         kind: int = GEMM_AUTO, scratch: Optional[torch.Tensor] = None, splits: int = 0) -> torch.Tensor:
    """out (epilogue)= x @ weight.T with weight [N, K], x [T, K].

    scratch: float32 of GEMM_SPLIT_FLOATS elements (optional).  With it, a product of few rows with a long inner
    size may share k out over several blocks (splits: 0 = let the kernel choose, 1 = never, n = n runs of k).

    EPI_STORE: out [T, N] in the run dtype.  EPI_ACCUM_F32: out float32 [T, N], added to.
    EPI_SWIGLU: weight rows are (gate_0, up_0, gate_1, up_1, ...), out [T, N/2] = silu(gate) * up.
    EPI_STORE_F32: out float32 [T, N].
    """
    _need(weight, "gemm weight", dims=2)
    _need(x, "gemm input", weight.dtype, 2)
    n, k = weight.shape
    t = x.shape[0]
    if x.shape[1] != k:
        raise KernelError(f"gemm: input width {x.shape[1]} does not match weight {tuple(weight.shape)}")
    want_dtype = torch.float32 if epilogue in (EPI_ACCUM_F32, EPI_STORE_F32) else weight.dtype
    _need(out, "gemm output", want_dtype, 2)
    cols = n // 2 if epilogue == EPI_SWIGLU else n
    if tuple(out.shape) != (t, cols):
        raise KernelError(f"gemm: output {tuple(out.shape)}, expected {(t, cols)}")
    if scratch is not None:
        _need(scratch, "gemm scratch", torch.float32, 1)
    elif splits > 1:
        raise KernelError("gemm: a split product needs scratch")
    rows_kernel = _streams_rows(weight, t, kind, scratch is not None, splits)
    args = (_ptr(weight), _ptr(x), _ptr(out), dtype_code(weight.dtype), n, t, k, _rows(weight, "gemm weight"),
            _rows(x, "gemm input"), _rows(out, "gemm output"), epilogue)
    if rows_kernel:
        fn = _lib("gemm_rows", (("DLGO_ELEM", dtype_code(weight.dtype)),)).dlgo_gemm_rows
        _check(fn(*args, 0 if kind in (GEMM_AUTO, GEMM_ROWS16) else kind, _stream()))
    else:
        fn = _lib("gemm", (("DLGO_ELEM", dtype_code(weight.dtype)),)).dlgo_gemm
        _check(fn(*args, kind, splits, _ptr(scratch), ctypes.c_longlong(scratch.numel() if scratch is not None else 0), _stream()))
    return out


FUSED_NORM_ROWS = 64   # most rows of the residual stream that gemm_rmsnorm takes
FUSED_NORM_PAYS = 16   # up to this many rows the fused norm is faster than a norm kernel and a plain product


def fused_norm_pays(weight: torch.Tensor, rows: int) -> bool:
    """Whether gemm_rmsnorm beats a norm kernel followed by gemm for this weight and this many rows."""
    tiled = weight.shape[0] >= GEMM_VERY_WIDE and weight.shape[1] % (128 // weight.element_size()) == 0
    return rows <= FUSED_NORM_PAYS and not tiled


def gemm_rmsnorm(weight: torch.Tensor, x: torch.Tensor, norm_weight: torch.Tensor, eps: float, out: torch.Tensor,
                 epilogue: int = EPI_STORE, kind: int = GEMM_AUTO) -> torch.Tensor:
    """out (epilogue)= (rmsnorm(x) * norm_weight) @ weight.T for up to 64 rows x of the float32 residual stream,
    without writing the normed rows.  Epilogues as gemm().  kind: 0 = chosen by the shape, 10 = the weights go through
    LDS in whole 1 KB runs wherever that kernel applies (up to 16 rows, weight rows of 2 to 16 whole KB), 11 = never."""
    _need(weight, "gemm weight", dims=2)
    _need(x, "residual rows", torch.float32, 2)
    _need(norm_weight, "norm weight", torch.float32, 1)
    n, k = weight.shape
    t = x.shape[0]
    if x.shape[1] != k or norm_weight.shape[0] != k or t > FUSED_NORM_ROWS:
        raise KernelError(f"gemm_rmsnorm: rows {tuple(x.shape)} and norm weight {tuple(norm_weight.shape)} do not fit weight {tuple(weight.shape)} (at most {FUSED_NORM_ROWS} rows)")
    want_dtype = torch.float32 if epilogue in (EPI_ACCUM_F32, EPI_STORE_F32) else weight.dtype
    _need(out, "gemm output", want_dtype, 2)
    cols = n // 2 if epilogue == EPI_SWIGLU else n
    if tuple(out.shape) != (t, cols):
        raise KernelError(f"gemm_rmsnorm: output {tuple(out.shape)}, expected {(t, cols)}")
    _check(_lib("gemm_rows", (("DLGO_ELEM", dtype_code(weight.dtype)),)).dlgo_gemm_rmsnorm(_ptr(weight), _ptr(x), _ptr(norm_weight), ctypes.c_float(eps), _ptr(out),
                                          dtype_code(weight.dtype), n, t, k, _rows(weight, "gemm weight"),
                                          _rows(x, "residual rows"), _rows(out, "gemm output"), epilogue, kind, _stream()))
    return out


class UnscaledNorm:
    """What gemm_accum_leave_norm leaves of rmsnorm(residual) * norm_weight: the rows it wrote hold residual * norm_weight,
    and `parts` [T, n_parts] (float32) each row's sum of squares in n_parts shares; rmsnorm's factor of row t is
    1 / sqrt(sum(parts[t]) / width + eps).  It is a scalar per row, so a product of the rows can apply it to its sums:
    gemm_scaled does."""
    __slots__ = ("rows", "parts", "n_parts", "width", "eps")

    def __init__(self, rows, parts, n_parts, width, eps):
        self.rows, self.parts, self.n_parts, self.width, self.eps = rows, parts, n_parts, width, eps


ROLE_PLAIN, ROLE_LEAVES_NORM, ROLE_APPLIES_NORM = 0, 1, 2


def streams_few_rows(weight: torch.Tensor, rows: int, role: int = ROLE_PLAIN) -> bool:
    """Whether the streamed products take this weight with this many rows of x: up to 16 rows and weight rows of whole
    KB; as the product that leaves a norm (ROLE_LEAVES_NORM) or applies one left to it (ROLE_APPLIES_NORM) also a
    normed width that its shares of the sums of squares cover."""
    if weight.dim() != 2 or weight.stride(1) != 1 or not (1 <= rows <= 16):
        return False
    lib = _lib("gemm_rows", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    lib.dlgo_gemm_rows_streams.restype = ctypes.c_int
    return bool(lib.dlgo_gemm_rows_streams(dtype_code(weight.dtype), weight.shape[0], rows, weight.shape[1], weight.stride(0), int(role)))


def _tiles_take_norm(weight: torch.Tensor, rows: int, role: int) -> bool:
    """Whether the tiled products leave (role 1) or apply (role 2) a norm for this weight and this many rows: steps of
    many rows whose product gemm() would give to tiles that sum the whole of k."""
    if weight.dim() != 2 or weight.stride(1) != 1 or rows <= 16:
        return False
    lib = _lib("gemm", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    lib.dlgo_gemm_tile_norm_takes.restype = ctypes.c_int
    return bool(lib.dlgo_gemm_tile_norm_takes(dtype_code(weight.dtype), weight.shape[0], rows, weight.shape[1], weight.stride(0),
                                              weight.shape[1], role, ctypes.c_longlong(GEMM_SPLIT_FLOATS)))


def can_leave_unscaled(weight: torch.Tensor, rows: int) -> bool:
    """Whether gemm_accum_leave_norm takes this weight with this many rows of x (contiguous rows of x assumed)."""
    return streams_few_rows(weight, rows, ROLE_LEAVES_NORM) or _tiles_take_norm(weight, rows, 1)


def can_take_unscaled(weight: torch.Tensor, rows: int) -> bool:
    """Whether gemm_scaled takes this weight with this many rows (contiguous rows assumed)."""
    return streams_few_rows(weight, rows, ROLE_APPLIES_NORM) or _tiles_take_norm(weight, rows, 2)


def gemm_accum_leave_norm(weight: torch.Tensor, x: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                          unscaled: torch.Tensor, parts: torch.Tensor) -> UnscaledNorm:
    """residual += x @ weight.T, and of rmsnorm(residual) * norm_weight of the new rows what UnscaledNorm describes
    (unscaled: [T, N] in the run dtype; parts: float32 scratch of at least T * ceil(N / 8) elements).  For weights
    and rows that can_leave_unscaled accepts: few rows go to the streamed product, many to tiles."""
    _need(weight, "gemm weight", dims=2)
    _need(x, "gemm input", weight.dtype, 2)
    _need(residual, "residual rows", torch.float32, 2)
    _need(norm_weight, "norm weight", torch.float32, 1)
    _need(unscaled, "unscaled rows", weight.dtype, 2)
    _need(parts, "norm parts", torch.float32, 1)
    n, k = weight.shape
    t = x.shape[0]
    if x.shape[1] != k or tuple(residual.shape) != (t, n) or tuple(unscaled.shape) != (t, n) or norm_weight.shape[0] != n:
        raise KernelError(f"gemm_accum_leave_norm: x {tuple(x.shape)}, residual {tuple(residual.shape)}, unscaled {tuple(unscaled.shape)} "
                          f"and norm weight {tuple(norm_weight.shape)} do not fit weight {tuple(weight.shape)}")
    n_parts = ctypes.c_int(0)
    tiled = t > 16
    lib = _lib("gemm" if tiled else "gemm_rows", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    fn = lib.dlgo_gemm_tile_leave if tiled else lib.dlgo_gemm_rows_leave_parts
    _check(fn(_ptr(weight), _ptr(x), _ptr(residual), dtype_code(weight.dtype), n, t, k,
              _rows(weight, "gemm weight"), _rows(x, "gemm input"), _rows(residual, "residual rows"),
              _ptr(norm_weight), _ptr(unscaled), _rows(unscaled, "unscaled rows"), _ptr(parts),
              ctypes.c_longlong(parts.numel()), ctypes.byref(n_parts), _stream()))
    return UnscaledNorm(unscaled, parts, n_parts.value, n, eps)


def gemm_scaled(weight: torch.Tensor, left: UnscaledNorm, out: torch.Tensor, epilogue: int = EPI_STORE) -> torch.Tensor:
    """out (epilogue)= rmsnorm's factor of each row * (left.rows @ weight.T): the product of the normed rows that `left`
    describes.  Epilogues as gemm() for few rows, store and SwiGLU for many; for weights and rows that can_take_unscaled
    accepts."""
    _need(weight, "gemm weight", dims=2)
    x = left.rows
    _need(x, "unscaled rows", weight.dtype, 2)
    n, k = weight.shape
    t = x.shape[0]
    if x.shape[1] != k or left.width != k or left.parts.numel() < t * left.n_parts:
        raise KernelError(f"gemm_scaled: rows {tuple(x.shape)} of a norm over {left.width} with {left.n_parts} parts do not fit weight {tuple(weight.shape)}")
    want_dtype = torch.float32 if epilogue in (EPI_ACCUM_F32, EPI_STORE_F32) else weight.dtype
    _need(out, "gemm output", want_dtype, 2)
    cols = n // 2 if epilogue == EPI_SWIGLU else n
    if tuple(out.shape) != (t, cols):
        raise KernelError(f"gemm_scaled: output {tuple(out.shape)}, expected {(t, cols)}")
    tiled = t > 16
    lib = _lib("gemm" if tiled else "gemm_rows", (("DLGO_ELEM", dtype_code(weight.dtype)),))
    fn = lib.dlgo_gemm_tile_scaled if tiled else lib.dlgo_gemm_rows_scaled
    _check(fn(_ptr(weight), _ptr(x), _ptr(out), dtype_code(weight.dtype), n, t, k, _rows(weight, "gemm weight"),
              _rows(x, "unscaled rows"), _rows(out, "gemm output"), epilogue, _ptr(left.parts), left.n_parts,
              left.width, ctypes.c_float(left.eps), _stream()))
    return out


def rope_kv(qkv: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, rot: int, interleaved: bool,
            cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
            tok_seq: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
            cache: Optional[torch.Tensor], page_stride: int, v_off: int, write_kv: bool = True,
            unsummed: Optional[UnsummedRows] = None, single_tokens: bool = False,
            seq_pages: Optional[torch.Tensor] = None) -> None:
    """Rotate the query heads of qkv [T, (H+2KV)*hd] in place; rotate the key heads and copy the value heads
    into the cache page of each token (cache: the first element of this layer's pages).  unsummed: the rows are not
    in qkv yet but in the runs that gemm_runs left (see rope_takes_unsummed); the rotated queries are written to qkv.
    single_tokens: every row is a sequence of its own (a hint for how the transposed values are best stored; the
    result is the same).  seq_pages: for such a step, the sequences' page-table rows in the order of the rows
    ([>= T, the table's width], row i = page_table[slots[tok_seq[i]]]); the kernel then reads a row's page from there
    without going through its sequence and slot."""
    _need(qkv, "qkv rows", dims=2)
    _need(positions, "positions", torch.int32, 1)
    t = qkv.shape[0]
    if positions.shape[0] != t:
        raise KernelError("rope_kv: one position per row")
    table_rows = 0
    if cos is not None:
        _need(cos, "cos table", torch.float32, 2)
        _need(sin, "sin table", torch.float32, 2)
        if cos.shape != sin.shape or cos.shape[1] != rot // 2 or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError(f"rope_kv: tables {tuple(cos.shape)} do not fit a rotated width of {rot}")
        table_rows = cos.shape[0]
    max_pages = 0
    if write_kv:
        _need(tok_seq, "token->sequence", torch.int32, 1)
        _need(slots, "slots", torch.int32, 1)
        _need(page_table, "page table", torch.int32, 2)
        _need(cache, "cache", qkv.dtype)
        if tok_seq.shape[0] != t or not page_table.is_contiguous():
            raise KernelError("rope_kv: one sequence index per row and a contiguous page table")
        max_pages = page_table.shape[1]
    by_row = write_kv and seq_pages is not None
    if by_row:
        _need(seq_pages, "pages by sequence", torch.int32, 2)
        if not single_tokens or seq_pages.shape[0] < t or seq_pages.shape[1] != max_pages or not seq_pages.is_contiguous():
            raise KernelError(f"rope_kv: pages by sequence {tuple(seq_pages.shape)} do not fit {t} single-token rows "
                              f"and a table {max_pages} wide")
        page_table = seq_pages
    part = (_ptr(None), 0, ctypes.c_longlong(0), 0)
    if unsummed is not None:
        if unsummed.rows != t or unsummed.cols < (n_heads + (2 * n_kv if write_kv else 0)) * head_dim:
            raise KernelError(f"rope_kv: unsummed rows [{unsummed.rows}, {unsummed.cols}] do not fit {t} rows of qkv")
        part = (_ptr(unsummed.scratch), unsummed.runs, ctypes.c_longlong(unsummed.rows * unsummed.cols), unsummed.cols)
    _check(_lib("rope_kv").dlgo_rope_kv(_ptr(qkv), dtype_code(qkv.dtype), t, _rows(qkv, "qkv rows"), n_heads, n_kv, head_dim,
                                        rot, int(interleaved), _ptr(cos), _ptr(sin), table_rows, _ptr(positions),
                                        _ptr(tok_seq), _ptr(slots), _ptr(page_table), max_pages, _ptr(cache),
                                        ctypes.c_longlong(page_stride), ctypes.c_longlong(v_off), int(write_kv), *part,
                                        int(single_tokens), int(by_row), _stream()))


def rope_takes_unsummed(dtype: torch.dtype, head_dim: int, rot: int) -> bool:
    """Whether rope_kv can read rows that gemm_runs left unsummed: it does so in whole 16-byte pieces."""
    epc = 4 if dtype == torch.float32 else 8
    return head_dim % epc == 0 and rot % (2 * epc) == 0


def attention_rows(q: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                   positions: torch.Tensor, tok_seq: torch.Tensor, slots: torch.Tensor, page_table: torch.Tensor,
                   cache: torch.Tensor, page_stride: int, v_off: int, window: int = 0,
                   scale: Optional[float] = None, n_splits: int = 1, scratch=None) -> torch.Tensor:
    """One wave per (row, head): the general kernel, every dtype, every step shape.  n_splits > 1 deals each row's
    pages to that many waves, whose partial results (in scratch(n): float32, n elements) a second kernel merges."""
    _need(q, "query rows", dims=2)
    _need(out, "attention output", q.dtype, 2)
    for name, v in (("positions", positions), ("token->sequence", tok_seq), ("slots", slots)):
        _need(v, name, torch.int32, 1)
    _need(page_table, "page table", torch.int32, 2)
    _need(cache, "cache", q.dtype)
    t = q.shape[0]
    if out.shape[0] != t or positions.shape[0] != t or tok_seq.shape[0] != t or not page_table.is_contiguous():
        raise KernelError("attention: one position, sequence index and output row per query row")
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    lib = _lib("attention", (("HEAD_DIM", head_dim),))
    part = None
    if n_splits > 1:
        need = t * n_heads * n_splits * (head_dim + 4)
        part = scratch(need) if scratch is not None else torch.empty(need, dtype=torch.float32, device=q.device)
        _need(part, "attention scratch", torch.float32, 1)
    _check(lib.dlgo_attention_rows(_ptr(q), _rows(q, "query rows"), _ptr(out), _rows(out, "attention output"),
                                   dtype_code(q.dtype), t, n_heads, n_kv, head_dim, _ptr(positions), _ptr(tok_seq),
                                   _ptr(slots), _ptr(page_table), page_table.shape[1], _ptr(cache),
                                   ctypes.c_longlong(page_stride), ctypes.c_longlong(v_off), int(window),
                                   ctypes.c_float(scale), int(n_splits), _ptr(part),
                                   ctypes.c_longlong(part.numel() if part is not None else 0), _stream()))
    return out


def attention_fuses_rotation(dtype: torch.dtype, head_dim: int, group: int, max_q_len: int, rot_width: int,
                             n_seq: int = 1, n_kv: int = 8) -> bool:
    """True if attention() should rotate the queries and take in the new keys and values itself for such a step:
    one row per sequence, bfloat16, a rotated width that is a multiple of 16 or no rotation at all; at most one
    (sequence, kv head) pair for every compute unit, so that a kernel launch costs more than the rotation repeated in
    every wave (with 8 kv heads on 256 units: up to 32 sequences; measured at 64: 62 against 9 + 52 us), and no more
    than 32 sequences whatever the heads (the largest step the fused variant is tested with); and heads small enough
    that eight waves of a block each keep a page (keys and values of 64 tokens) in 128 KB of LDS (at a head size of 128
    the kernel of its own is faster)."""
    page_bytes = 2 * PAGE * head_dim * 2
    return (dtype == torch.bfloat16 and 8 * page_bytes <= 128 * 1024 and group <= 128 and max_q_len == 1 and rot_width % 16 == 0
            and n_seq * n_kv * ((group + 15) // 16) <= compute_units() and n_seq <= 32)


def attention(q: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, positions: torch.Tensor,
              tok_seq: torch.Tensor, slots: torch.Tensor, page_table: torch.Tensor, cache: torch.Tensor, page_stride: int,
              v_off: int, q_lens: Sequence[int], start_pos: Sequence[int], window: int = 0,
              scale: Optional[float] = None, cu_q: Optional[torch.Tensor] = None,
              start_pos_dev: Optional[torch.Tensor] = None, scratch=None,
              max_pages_used: Optional[int] = None, kernel: str = "auto", rotation=None, new_kv: bool = False,
              split_variant: int = 0, seq_pages: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of a step's query rows over the cache, with the kernel chosen by the step's shape and dtype.

    q_lens, start_pos: per sequence, on the host (rows of the step, and the length before it).  cu_q and
    start_pos_dev are the same numbers on the device (built here if not given).  scratch(n) returns a
    float32 buffer of at least n elements (partials of long sequences in decode).  max_pages_used bounds the pages any sequence
    of the step holds (default: from q_lens and start_pos; a captured step passes the context's bound).
    kernel: "auto", "rows", "tiled" (prefill) or "split" (decode).  All kernels compute the same thing.
    rotation = (cos, sin, width, interleaved) and new_kv: only where attention_fuses_rotation() says so; then q
    holds the step's unrotated [q | k | v] rows, which the kernel rotates, and with new_kv it also takes each
    token's own key and value from its row and writes them to the cache (what rope_kv() does otherwise).
    split_variant (bfloat16 split kernel): 0 or 2 = a page goes through LDS in whole 1 KB runs, 1 = it is read straight
    into the operands' registers.
    seq_pages (steps of single tokens): the sequences' rows of page_table in the order of the step, [>= n_seq, the table's
    width]: row i holds what row slots[i] of page_table holds.  The bfloat16 split kernel then finds a sequence's pages
    without waiting for its slot, and asks for its first page's number together with the position.
    """
    n_seq = len(q_lens)
    max_q = int(max(q_lens)) if n_seq else 0
    group = n_heads // n_kv
    fast_ok = q.dtype == torch.bfloat16 and head_dim <= 256 and group <= 128
    tiled_f32 = q.dtype == torch.float32 and head_dim <= 128 and group <= 128       # prompts in float32: a kernel of their own
    split_f32 = q.dtype == torch.float32 and head_dim <= 128 and group <= 128      # and so have steps of single tokens
    if kernel == "auto":
        if fast_ok:
            kernel = "split" if max_q == 1 else "tiled"
        else:
            kernel = "split" if split_f32 and max_q == 1 else ("tiled" if tiled_f32 and max_q > 1 else "rows")
    if (rotation is not None or new_kv) and not (kernel == "split" and fast_ok and max_q == 1):
        raise KernelError("attention: only the bfloat16 split kernel rotates and stores by itself")
    if kernel == "rows" or n_seq == 0:
        # a few rows with long histories (a decode step off the fast kernels): each row's pages go to several waves
        n_splits = 1
        if max_q == 1 and n_seq > 0:
            pages = max_pages_used if max_pages_used is not None else (int(max(start_pos)) + PAGE) // PAGE
            n_splits = max(1, min(pages // 2, 2048 // max(1, n_seq * n_heads)))
        return attention_rows(q, out, n_heads, n_kv, head_dim, positions, tok_seq, slots, page_table, cache, page_stride,
                              v_off, window, scale, n_splits, scratch)
    if not fast_ok and not (tiled_f32 and kernel == "tiled") and not (split_f32 and kernel == "split"):
        raise KernelError("attention: the tiled and split kernels take bfloat16, head sizes up to 256 and up to 128 heads per kv head "
                          "(and float32 with head sizes up to 128)")
    _need(q, "query rows", q.dtype, 2)
    _need(out, "attention output", q.dtype, 2)
    _need(slots, "slots", torch.int32, 1)
    _need(page_table, "page table", torch.int32, 2)
    _need(cache, "cache", q.dtype)
    if slots.shape[0] != n_seq or out.shape[0] != q.shape[0] or q.shape[0] != int(sum(q_lens)) or not page_table.is_contiguous():
        raise KernelError("attention: rows, sequences and slots do not match")
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    lib = _lib("attention", (("HEAD_DIM", head_dim),))
    if kernel == "split":
        if max_q != 1:
            raise KernelError("attention: the split kernel takes one row per sequence")
        _need(positions, "positions", torch.int32, 1)
        if positions.shape[0] != n_seq:
            raise KernelError("attention: one position per sequence")
        max_pages = page_table.shape[1]
        if max_pages_used is None:
            max_pages_used = (int(max(start_pos)) + 1 + PAGE - 1) // PAGE
        max_pages_used = max(1, min(max_pages_used, max_pages))
        cos = sin = None
        rot_width, interleaved = 0, False
        if rotation is not None:
            cos, sin, rot_width, interleaved = rotation
            _need(cos, "cos table", torch.float32, 2)
            _need(sin, "sin table", torch.float32, 2)
            if cos.shape != sin.shape or cos.shape[1] != rot_width // 2 or not cos.is_contiguous() or not sin.is_contiguous():
                raise KernelError(f"attention: tables {tuple(cos.shape)} do not fit a rotated width of {rot_width}")
        if seq_pages is not None:
            _need(seq_pages, "pages by sequence", torch.int32, 2)
            if seq_pages.shape[0] < n_seq or seq_pages.shape[1] != max_pages or not seq_pages.is_contiguous():
                raise KernelError(f"attention: pages by sequence {tuple(seq_pages.shape)} do not fit {n_seq} sequences and a table {max_pages} wide")
        lib.dlgo_attention_decode_splits.restype = ctypes.c_int
        variant = split_variant if q.dtype == torch.bfloat16 else 1
        n_splits = lib.dlgo_attention_decode_splits(n_seq, n_heads, n_kv, max_pages_used, int(rotation is not None or new_kv), variant)
        part = None
        if n_splits > 1:
            need = n_seq * n_heads * n_splits * (head_dim + 4)
            part = scratch(need) if scratch is not None else torch.empty(need, dtype=torch.float32, device=q.device)
            _need(part, "attention scratch", torch.float32, 1)
        if q.dtype == torch.float32:
            _check(lib.dlgo_attention_decode_f32(_ptr(q), _rows(q, "query rows"), _ptr(out), _rows(out, "attention output"), _ptr(part),
                                                 ctypes.c_longlong(part.numel() if part is not None else 0), n_seq, n_heads, n_kv,
                                                 head_dim, _ptr(positions), _ptr(slots), _ptr(page_table), max_pages, max_pages_used,
                                                 _ptr(cache), ctypes.c_longlong(page_stride), ctypes.c_longlong(v_off), int(window),
                                                 ctypes.c_float(scale), _stream()))
            return out
        _check(lib.dlgo_attention_decode(_ptr(q), _rows(q, "query rows"), _ptr(out), _rows(out, "attention output"), _ptr(part),
                                         ctypes.c_longlong(part.numel() if part is not None else 0), n_seq, n_heads, n_kv,
                                         head_dim, _ptr(positions), _ptr(slots), _ptr(page_table), max_pages, max_pages_used,
                                         _ptr(cache), ctypes.c_longlong(page_stride), ctypes.c_longlong(v_off), int(window),
                                         ctypes.c_float(scale), _ptr(cos), _ptr(sin), cos.shape[0] if cos is not None else 0,
                                         int(rot_width), int(interleaved), int(new_kv), int(variant), _ptr(seq_pages), _stream()))
        return out
    if kernel != "tiled":
        raise KernelError(f"attention: unknown kernel {kernel!r}")
    if cu_q is None:
        import numpy as np
        cu = np.concatenate([[0], np.cumsum(np.asarray(q_lens, dtype=np.int64))]).astype(np.int32)
        cu_q = torch.from_numpy(cu).to(q.device)
        start_pos_dev = torch.as_tensor(list(start_pos), dtype=torch.int32).to(q.device)
    _need(cu_q, "row offsets", torch.int32, 1)
    _need(start_pos_dev, "start positions", torch.int32, 1)
    if cu_q.shape[0] != n_seq + 1 or start_pos_dev.shape[0] != n_seq:
        raise KernelError("attention: row offsets and start positions do not match the sequences")
    entry = lib.dlgo_attention_prefill_f32 if q.dtype == torch.float32 else lib.dlgo_attention_prefill
    _check(entry(_ptr(q), _rows(q, "query rows"), _ptr(out), _rows(out, "attention output"), n_seq, max_q,
                                      n_heads, n_kv, head_dim, _ptr(cu_q), _ptr(start_pos_dev), _ptr(slots), _ptr(page_table),
                                      page_table.shape[1], _ptr(cache), ctypes.c_longlong(page_stride),
                                      ctypes.c_longlong(v_off), int(window), ctypes.c_float(scale), _stream()))
    return out


_argmax_scratch: dict = {}


def argmax(logits: torch.Tensor, out: torch.Tensor, scratch: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = index of the first maximum of row r.  scratch: 512 bytes per row (kept here per device if not given)."""
    _need(logits, "logits", torch.float32, 2)
    _need(out, "argmax output", torch.int32, 1)
    n = logits.shape[0]
    if out.shape[0] != n:
        raise KernelError("argmax: one output per row")
    if scratch is None:
        scratch = _argmax_scratch.get(logits.device)
        if scratch is None or scratch.numel() < n * 512:
            scratch = torch.empty(max(n, 256) * 512, dtype=torch.uint8, device=logits.device)
            _argmax_scratch[logits.device] = scratch
    _check(_lib("sampling").dlgo_argmax(_ptr(logits), _rows(logits, "logits"), n, logits.shape[1], _ptr(scratch),
                                        ctypes.c_longlong(scratch.numel() * scratch.element_size()), _ptr(out), _stream()))
    return out


def sample(logits: torch.Tensor, work: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, min_p: torch.Tensor, penalty: torch.Tensor, recent: Optional[torch.Tensor],
           uniform: torch.Tensor, out: torch.Tensor, recent_rows: Optional[torch.Tensor] = None,
           counts: Optional[torch.Tensor] = None, dealt_rows: bool = True) -> torch.Tensor:
    """One token per row of float32 logits, each row with its own options.  work: float32 scratch [rows, vocab].  recent [rows, w]: the row's recent tokens
    (-1 where empty) for the repetition penalty.  With recent_rows [rows] and counts: recent is a table of rings, row
    recent_rows[r] of it belongs to row r and holds its last min(counts, w) tokens; the chosen token is added to it.
    dealt_rows=False: the caller, who has the options on the host, knows that no row is of a kind that several blocks
    share over a wide vocabulary (a top-k of 1 to 1,024, or neither top-k nor top-p); the kernels for those are
    then not launched."""
    _need(logits, "logits", torch.float32, 2)
    n, v = logits.shape
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32),
                        ("penalty", penalty, torch.float32), ("uniform", uniform, torch.float32),
                        ("sample output", out, torch.int32)):
        _need(t, name, dt, 1)
        if t.shape[0] != n:
            raise KernelError(f"sample: {name} has {t.shape[0]} entries for {n} rows")
    _need(work, "work", torch.float32, 2)
    if work.shape[0] < n or work.shape[1] != v or not work.is_contiguous():
        raise KernelError(f"sample: scratch {tuple(work.shape)} too small for {(n, v)}")
    n_recent = 0
    if (recent_rows is None) != (counts is None):
        raise KernelError("sample: a table of rings needs both recent_rows and counts")
    if recent is not None:
        _need(recent, "recent tokens", torch.int32, 2)
        if not recent.is_contiguous() or (counts is None and recent.shape[0] != n):
            raise KernelError("sample: one row of recent tokens per row of logits")
        n_recent = recent.shape[1]
    if counts is not None:
        _need(recent_rows, "rows of the recent tokens", torch.int32, 1)
        _need(counts, "counts of recent tokens", torch.int32, 1)
        if recent is None or recent_rows.shape[0] != n or counts.shape[0] != recent.shape[0]:
            raise KernelError("sample: recent_rows has one entry per row of logits, counts one per row of the table")
    _check(_lib("sampling").dlgo_sample(_ptr(logits), _rows(logits, "logits"), n, v, _ptr(work), _ptr(temperature),
                                        _ptr(top_k), _ptr(top_p), _ptr(min_p), _ptr(penalty), _ptr(recent), n_recent,
                                        _ptr(recent_rows), _ptr(counts), _ptr(uniform), _ptr(out), int(bool(dealt_rows)),
                                        _stream()))
    return out


# ---------------------------------------------------------------------------
# Timing the launches one by one (what computerex/dlgo's gpu_timing_main.go:73-119 does for its operations): inside a
# `with Timings() as t:` block every face above that launches something is bracketed by two events on the current
# stream; t.microseconds() then gives, per label, the time between them summed over the block.  A product's label
# carries its weight's shape, which is what tells the products of a layer apart.  The steps inside the block must run
# as they are (a replayed recording calls no face).  Outside such a block a face costs one comparison more.
_recorder: Optional[list] = None


class Timings:
    def __enter__(self) -> "Timings":
        global _recorder
        self.events: List[tuple] = []
        self._outer, _recorder = _recorder, self.events
        return self

    def __exit__(self, *exc) -> None:
        global _recorder
        _recorder = self._outer

    def microseconds(self) -> Dict[str, float]:
        torch.cuda.synchronize()
        out: Dict[str, float] = {}
        for label, start, end in self.events:
            out[label] = out.get(label, 0.0) + start.elapsed_time(end) * 1000.0
        return out

    def launches(self) -> Dict[str, int]:
        out: Dict[str, int] = {}
        for label, _, _ in self.events:
            out[label] = out.get(label, 0) + 1
        return out


def _timed(fn):
    name = fn.__name__
    by_weight = name.startswith("gemm")

    @functools.wraps(fn)
    def face(*args, **kwargs):
        rec = _recorder
        if rec is None:
            return fn(*args, **kwargs)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        result = fn(*args, **kwargs)
        end.record()
        if result is False or (result is None and name == "gemm_runs"):
            return result                # it declined: nothing was launched
        label = name
        if by_weight and args and isinstance(args[0], torch.Tensor):
            label = f"{name}[{args[0].shape[0]}x{args[0].shape[1]}]"
        rec.append((label, start, end))
        return result
    return face


for _name in ("embed", "copy_rows", "rmsnorm", "bias_add", "head_rmsnorm", "gemm_accum_then_norm", "gemm_runs", "gemm", "gemm_rmsnorm",
              "gemm_accum_leave_norm", "gemm_scaled", "rope_kv", "attention", "argmax", "sample"):
    globals()[_name] = _timed(globals()[_name])
del _name
