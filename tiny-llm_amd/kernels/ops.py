"""Python face of the HIP kernels: one function per kernel entry point.

Every function checks on the host that device, dtype, contiguity, alignment and
shapes are what the kernel and its grid assume, then hands raw pointers and the
current stream to the library.  A refused size raises `KernelError`; nothing is
computed on the CPU or by a library op.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import library

c_void_p = ctypes.c_void_p
c_int = ctypes.c_int
c_int64 = ctypes.c_int64
c_float = ctypes.c_float

_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _lib():
    return library.load()


try:                                        # the raw handle without building a Stream object
    from torch._C import _cuda_getCurrentRawStream as _raw_stream
except ImportError:                          # pragma: no cover
    _raw_stream = None


def _stream():
    """The current stream of the current device (also while a graph is being captured)."""
    if _raw_stream is not None:
        return c_void_p(_raw_stream(torch.cuda.current_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not float32 or bfloat16") from None


def _fail(msg: str) -> None:
    raise KernelError(msg)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None:
            if not (t.is_cuda):
                _fail("kernel operands must live on the GPU (there is no CPU path)")


def _ptr(t: Optional[torch.Tensor], align: int = 1) -> c_void_p:
    if t is None:
        return c_void_p(0)
    p = t.data_ptr()
    if not (p % align == 0):
        _fail(f"operand is not {align}-byte aligned")
    return c_void_p(p)


def _check(code: int, what: str) -> None:
    if code == 1:
        raise KernelError(f"{what}: the kernel refuses these sizes")
    if code != 0:
        raise KernelError(f"{what}: launch failed (status {code})")


def _rows_2d(t: torch.Tensor, name: str) -> None:
    if not (t.dim() == 2 and t.stride(1) == 1):
        _fail(f"{name} must be 2-D with unit inner stride")


# ------------------------------------------------------------- step workspace
class Workspace:
    """The buffers a step's kernels pass intermediates through, by name: allocated once at the
    size of the largest step (`max_rows` rows for row-shaped buffers) and used again by every
    layer and every step, eager or captured.  A buffer is never freed or moved while the workspace
    lives (a captured graph holds its address); one that turns out too small is retired, not freed.

    `rotate=n` hands out n buffers in turn under one name, for values that are still read while
    their successor is written (the norm hand-off between consecutive products)."""

    FIRST_ROWS = 4096       # rows the buffers are first made for when steps may be larger still

    def __init__(self, device, max_rows: int):
        self.device = torch.device(device)
        self.max_rows = min(int(max_rows), self.FIRST_ROWS)
        self._bufs: dict = {}
        self._turn: dict = {}
        self._retired: list = []

    def take(self, name: str, shape, dtype: torch.dtype, rotate: int = 1) -> torch.Tensor:
        shape = tuple(int(s) for s in shape)
        if rotate > 1:
            i = self._turn.get(name, 0)
            self._turn[name] = (i + 1) % rotate
            name = f"{name}#{i}"
        n = 1
        for s in shape:
            n *= s
        key = (name, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            if buf is not None:
                self._retired.append(buf)
            cap = n
            if len(shape) == 2 and shape[0] <= self.max_rows:
                cap = self.max_rows * shape[1]
            elif buf is not None:
                # sizes that depend on the batch and on how a context is split creep up in a
                # serving run: at least double, so that few retired buffers stay behind
                cap = max(n, 2 * buf.numel())
            buf = self._bufs[key] = torch.empty(cap, dtype=dtype, device=self.device)
        return buf[:n].view(shape)

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in list(self._bufs.values()) + self._retired)


_workspace: Optional[Workspace] = None


class use_workspace:
    """`with use_workspace(ws):` intermediates of the ops and parts inside come from `ws`."""

    def __init__(self, ws: Optional[Workspace]):
        self.ws = ws

    def __enter__(self):
        global _workspace
        self.prev, _workspace = _workspace, self.ws
        return self.ws

    def __exit__(self, *exc):
        global _workspace
        _workspace = self.prev


def scratch(name: str, shape, dtype: torch.dtype, device, rotate: int = 1) -> torch.Tensor:
    """An uninitialised intermediate: from the step's workspace when one is in use, else fresh."""
    if _workspace is not None and torch.device(device) == _workspace.device:
        return _workspace.take(name, shape, dtype, rotate)
    return torch.empty(tuple(shape), dtype=dtype, device=device)


# ------------------------------------------------- sizes, checked when parts are built
MAX_HEAD_DIM = 256      # the general attention kernel keeps a head's row in one wave's registers


def check_linear_sizes(dtype: torch.dtype, inner: int, what: str = "inner size") -> None:
    """Raises KernelError if no product kernel takes rows of `inner` elements in `dtype`
    (the bfloat16 kernels move 16-byte vectors: multiples of 8)."""
    if dtype == torch.bfloat16 and inner % 8:
        _fail(f"{what} = {inner}: the bfloat16 products need a multiple of 8 (float32 takes any size)")
    if inner <= 0:
        _fail(f"{what} = {inner} must be positive")


def check_attention_sizes(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Raises KernelError for head shapes no attention kernel takes."""
    if head_dim > MAX_HEAD_DIM or head_dim <= 0:
        _fail(f"head_dim {head_dim} is outside the attention kernels' range of 1 to {MAX_HEAD_DIM}")
    if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads or num_heads > 65535:
        _fail(f"{num_heads} heads over {num_kv_heads} kv heads: heads must be a multiple of kv heads, at most 65535")


# --------------------------------------------------------------------------- ops
def embedding(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t, :] = table[tokens[t], :] * scale as float32."""
    _dev(tokens, table, out)
    T = tokens.numel()
    V, H = table.shape
    if not (tokens.dtype == torch.int32 and tokens.is_contiguous()):
        _fail("tokens must be contiguous int32")
    if not (table.is_contiguous()):
        _fail("embedding table must be contiguous")
    if not (out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, H)):
        _fail(f"embedding output must be float32 [{T}, {H}]")
    _check(_lib().tl_embedding(_ptr(tokens), _ptr(table), _ptr(out), c_int(T), c_int(H), c_int(V), c_float(scale),
                               c_int(_dt(table)), _stream()), "embedding")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i] = weight * x[rows[i] or i] / sqrt(mean(x^2) + eps); x is float32."""
    _dev(x, weight, out, rows)
    if not (x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()):
        _fail("norm input must be contiguous float32 [T, H]")
    H = x.shape[1]
    n = out.shape[0]
    if not (weight.is_contiguous() and weight.numel() == H):
        _fail(f"norm weight must have {H} elements")
    if not (out.dim() == 2 and out.is_contiguous() and out.shape[1] == H):
        _fail("norm output must be contiguous [n, H]")
    if rows is None:
        if not (n == x.shape[0]):
            _fail("norm output rows must match input rows")
    else:
        if not (rows.dtype == torch.int32 and rows.is_contiguous() and rows.numel() == n):
            _fail("row index must be contiguous int32, one per output row")
    _check(_lib().tl_rmsnorm(_ptr(x), _ptr(weight), _ptr(rows), _ptr(out), c_int(n), c_int(H),
                             c_float(eps), c_int(_dt(weight)), c_int(_dt(out)), _stream()), "rmsnorm")
    return out


def linear(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, residual: Optional[torch.Tensor] = None,
           epilogue: Optional[str] = None, row_scale: Optional[torch.Tensor] = None, tile: int = 0) -> torch.Tensor:
    """out = a @ w.T (+ residual).  a [M, K], w [N, K] share an element type; out [M, N] is that
    type or float32; residual float32 with out's strides.  epilogue="swiglu": the N columns are
    interleaved (gate_j, up_j) pairs and out [M, N/2] = silu(gate) * up, computed from the float32
    accumulators.  row_scale [M] (float32) multiplies the rows of the product first.
    tile: 0 lets the sizes choose the tile of the bfloat16 product for more than 64 rows; 1 to 4
    force 256x256, 256x128, 128x128, 64x128 (tests and tuning)."""
    _dev(a, w, out, residual, row_scale)
    _rows_2d(a, "linear input")
    _rows_2d(out, "linear output")
    M, K = a.shape
    N = w.shape[0]
    swiglu = _epilogue(epilogue)
    if not (w.dim() == 2 and w.is_contiguous() and w.shape[1] == K):
        _fail(f"weight must be contiguous [N, {K}]")
    if not (a.dtype == w.dtype):
        _fail("input and weight must share an element type")
    dt, odt = _dt(a), _dt(out)
    if swiglu:
        if not (N % 2 == 0 and tuple(out.shape) == (M, N // 2) and odt == dt and residual is None):
            _fail(f"the SiLU-gate epilogue writes [{M}, {N // 2}] of the input's type and takes no residual")
    else:
        if not (tuple(out.shape) == (M, N)):
            _fail(f"linear output must be [{M}, {N}]")
        if not (odt == dt or odt == 0):
            _fail("linear output must have the input's type or float32")
    if residual is not None:
        if not (residual.dtype == torch.float32 and residual.shape == out.shape
                and residual.stride() == out.stride()):
            _fail("residual must be float32 with the output's layout")
    if dt == 1:
        if not (K % 8 == 0 and a.stride(0) % 8 == 0):
            _fail(f"bfloat16 linear needs an inner size that is a multiple of 8, got K={K}")
    al = 16 if dt == 1 else 4      # the bfloat16 kernel moves 16-byte vectors
    ao = 16 if (dt == 1 and not swiglu and M > 64) else 4
    if row_scale is not None:
        if not (row_scale.dtype == torch.float32 and row_scale.is_contiguous() and row_scale.numel() == M):
            _fail("row scales are float32, one per row")
    if not (0 <= tile <= 4):
        _fail("tile is 0 (by size) or 1 to 4")
    if dt == 1 and tile == 0 and M > 16:
        splits = split_k(M, N, K)
        if splits > 1:
            return _linear_split(a, w, out, residual, swiglu, row_scale, None, 0, 0.0, 0, None, splits)
    _check(_lib().tl_linear_tile(_ptr(a, al), _ptr(w, al), _ptr(out, ao), _ptr(residual, ao), _ptr(row_scale),
                                 c_int(M), c_int(N), c_int(K), c_int64(a.stride(0)), c_int64(out.stride(0)), c_int(dt),
                                 c_int(odt), c_int(swiglu), c_int(tile), _stream()), "linear")
    return out


def _epilogue(name: Optional[str]) -> int:
    if name is None:
        return 0
    if not (name == "swiglu"):
        _fail(f"unknown epilogue {name!r}")
    return 1

FUSED_MAX_ROWS = 16    # most rows for which the few-row product kernel normalises its input itself
FUSED_MAX_COLS = 4096  # most columns for which the fused norm prologue pays


def linear_norm(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor,
                residual: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
                epilogue: Optional[str] = None) -> torch.Tensor:
    """out = rmsnorm(x[rows] or x; norm_weight, eps) @ w.T, then the epilogue of `linear`, for float32
    x and bfloat16 w.  The norm is evaluated as (bf16(norm_weight * x) @ w.T) / rms: the row factor
    1 / rms is applied to the product, so the operand does not wait for the row statistics.  Few
    rows and few columns run in ONE kernel (every workgroup prepares the operand itself, which pays
    while one round of workgroups covers the columns); otherwise a pre-scale kernel writes the
    operand and the row factors once and the plain product applies them."""
    _dev(x, norm_weight, w, out, residual, rows)
    if not (x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1):
        _fail("norm input must be float32 [T, K]")
    K = x.shape[1]
    M = x.shape[0] if rows is None else rows.numel()
    N = w.shape[0]
    swiglu = _epilogue(epilogue)
    if not (M > 0):
        _fail("the product needs at least one row")
    if not (w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous() and w.shape[1] == K):
        _fail(f"weight must be contiguous bfloat16 [N, {K}]")
    if not (norm_weight.is_contiguous() and norm_weight.numel() == K):
        _fail(f"norm weight must have {K} elements")
    if not (K % 8 == 0 and x.stride(0) % 8 == 0):
        _fail("inner size must be a multiple of 8")
    if rows is not None:
        if not (rows.dtype == torch.int32 and rows.is_contiguous()):
            _fail("row index must be contiguous int32")
    if M > FUSED_MAX_ROWS or N > FUSED_MAX_COLS:
        if not (x.is_contiguous()):
            _fail("norm input must be contiguous")
        h = scratch("norm_operand", (M, K), torch.bfloat16, x.device)
        inv_rms = scratch("norm_row_factor", (M,), torch.float32, x.device)
        _check(_lib().tl_norm_prescale(_ptr(x), _ptr(norm_weight), _ptr(rows), _ptr(h), _ptr(inv_rms), c_int(M),
                                       c_int(K), c_float(eps), c_int(_dt(norm_weight)), _stream()), "norm_prescale")
        return linear(h, w, out, residual, epilogue, row_scale=inv_rms)
    _rows_2d(out, "linear output")
    if swiglu:
        if not (N % 2 == 0 and tuple(out.shape) == (M, N // 2) and out.dtype == torch.bfloat16 and residual is None):
            _fail(f"the SiLU-gate epilogue writes bfloat16 [{M}, {N // 2}] and takes no residual")
    else:
        if not (tuple(out.shape) == (M, N)):
            _fail(f"linear output must be [{M}, {N}]")
    if residual is not None:
        if not (residual.dtype == torch.float32 and residual.shape == out.shape
                and residual.stride() == out.stride()):
            _fail("residual must be float32 with the output's layout")
    _check(_lib().tl_linear_norm(_ptr(x, 16), _ptr(w, 16), _ptr(out), _ptr(residual), _ptr(norm_weight, 16),
                                 _ptr(rows), c_float(eps), c_int(_dt(norm_weight)), c_int(M), c_int(N), c_int(K),
                                 c_int64(x.stride(0)), c_int64(out.stride(0)), c_int(_dt(out)), c_int(swiglu),
                                 _stream()), "linear_norm")
    return out

def linear_norm_f32_ok(rows: int, cols: int, inner: int, row_stride: int) -> bool:
    """Whether `linear_norm_f32` takes these sizes (few rows, an inner size in whole vectors)."""
    return bool(_lib().tl_linear_norm_f32_ok(c_int(rows), c_int(cols), c_int(inner), c_int64(row_stride)))


def linear_f32_col_tiles(rows: int, cols: int, inner: int) -> int:
    """Column tiles a workgroup of the float32 few-row product owns at these sizes (more than one: a
    wide product, in front of which a norm is cheaper as `norm_prescale_f32` than inside `linear_norm_f32`)."""
    return int(_lib().tl_linear_f32_col_tiles(c_int(rows), c_int(cols), c_int(inner)))


def linear_norm_f32(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor,
                    residual: Optional[torch.Tensor] = None, epilogue: Optional[str] = None) -> torch.Tensor:
    """out = rmsnorm(x; norm_weight, eps) @ w.T, then the epilogue of `linear`, all float32 and for few
    rows (`linear_norm_f32_ok`): the norm rides in the product's kernel, evaluated as
    ((norm_weight * x) @ w.T) / rms with the squares added up in one fixed order per row."""
    _dev(x, norm_weight, w, out, residual)
    for t, what in ((x, "norm input"), (w, "weight"), (out, "output"), (norm_weight, "norm weight")):
        if t.dtype != torch.float32:
            _fail(f"{what} must be float32")
    if not (x.dim() == 2 and x.stride(1) == 1):
        _fail("norm input must be [T, K] with contiguous rows")
    M, K = x.shape
    N = w.shape[0]
    swiglu = _epilogue(epilogue)
    if not (w.dim() == 2 and w.is_contiguous() and w.shape[1] == K):
        _fail(f"weight must be contiguous [N, {K}]")
    if not (norm_weight.is_contiguous() and norm_weight.numel() == K):
        _fail(f"norm weight must have {K} elements")
    if not linear_norm_f32_ok(M, N, K, x.stride(0)):
        _fail(f"the float32 product with a norm takes at most {FEW_ROWS} rows and an inner size in whole vectors")
    _rows_2d(out, "linear output")
    if swiglu:
        if not (N % 2 == 0 and tuple(out.shape) == (M, N // 2) and residual is None):
            _fail(f"the SiLU-gate epilogue writes [{M}, {N // 2}] and takes no residual")
    elif tuple(out.shape) != (M, N):
        _fail(f"linear output must be [{M}, {N}]")
    if residual is not None:
        if not (residual.dtype == torch.float32 and residual.shape == out.shape and residual.stride() == out.stride()):
            _fail("residual must be float32 with the output's layout")
    _check(_lib().tl_linear_norm_f32(_ptr(x, 16), _ptr(norm_weight, 16), c_float(eps), _ptr(w, 16), _ptr(out),
                                     _ptr(residual), c_int(M), c_int(N), c_int(K), c_int64(x.stride(0)),
                                     c_int64(out.stride(0)), c_int(swiglu), _stream()), "linear_norm_f32")
    return out


def norm_prescale_f32(x: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                      rows: Optional[torch.Tensor] = None):
    """(h, inv_rms) for float32 x: h = norm_weight * x[rows or all] and the rows' factors 1 / rms, so that
    linear(h, w, out, row_scale=inv_rms) is rmsnorm(x) @ w.T with the very bits of `linear_norm_f32`
    (one order of addition for the squares in both): a row's result does not depend on the number of
    rows in its step, which decides between the two routes."""
    _dev(x, norm_weight, rows)
    if not (x.dtype == torch.float32 and norm_weight.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1):
        _fail("norm input and weight must be float32, the input [T, K] with contiguous rows")
    K = x.shape[1]
    M = x.shape[0] if rows is None else rows.numel()
    if not (norm_weight.is_contiguous() and norm_weight.numel() == K):
        _fail(f"norm weight must have {K} elements")
    if rows is not None and not (rows.dtype == torch.int32 and rows.is_contiguous()):
        _fail("row index must be contiguous int32")
    h = scratch("norm_operand_f32", (M, K), torch.float32, x.device)
    inv_rms = scratch("norm_row_factor", (M,), torch.float32, x.device)
    _check(_lib().tl_norm_prescale_f32(_ptr(x), _ptr(norm_weight), _ptr(rows), _ptr(h), _ptr(inv_rms), c_int(M),
                                       c_int(K), c_int64(x.stride(0)), c_float(eps), _stream()), "norm_prescale_f32")
    return h, inv_rms


FEW_ROWS = 64   # most rows the few-row product takes


def split_k(rows: int, cols: int, inner: int) -> int:
    """Into how many parts the bfloat16 product [rows, inner] x [cols, inner]^T has its inner size
    split over workgroups (1: not at all): products with few output tiles and more rows than the
    few-row kernel likes."""
    if inner % 8:
        return 1
    key = (rows, cols, inner)
    n = _SPLITS.get(key)
    if n is None:
        n = _SPLITS[key] = int(_lib().tl_splitk_plan(c_int(rows), c_int(cols), c_int(inner)))
    return n


_SPLITS: dict = {}      # the plan is a pure function of the sizes


def can_hand_off(rows: int, width: int, inner: int, dtype: torch.dtype) -> bool:
    """Whether `linear_handoff` can prepare a norm over `width` columns for `rows` rows, as the
    epilogue of the product with inner size `inner`: the few-row kernel, a product whose inner
    size is split, or the tiled kernel where the width is a multiple of 64."""
    if dtype != torch.bfloat16 or rows <= 0 or width % 8 or inner % 8:
        return False
    return rows <= FEW_ROWS or split_k(rows, width, inner) > 1 or width % 64 == 0


def handoff_parts(rows: int, width: int, inner: int) -> int:
    """How many partial sums of squares per row the product [rows, inner] x [width, inner]^T writes
    when it prepares a norm: one per workgroup in the few-row kernel (16 or 8 columns), per 1024
    after a split inner size, per 64 in the tiled kernel."""
    if split_k(rows, width, inner) > 1:
        return (width + 1023) // 1024
    if not (rows <= FEW_ROWS or width % 64 == 0):
        _fail(f"a norm is prepared for at most {FEW_ROWS} rows, with a split inner size or over a multiple of 64 columns")
    key = (rows, width, inner)
    n = _PARTS.get(key)
    if n is None:
        n = _PARTS[key] = int(_lib().tl_handoff_parts(c_int(rows), c_int(width), c_int(inner)))
    return n


_PARTS: dict = {}


def _linear_split(a, w, out, residual, swiglu, row_scale, sumsq_in, parts, eps, width, emit, splits) -> torch.Tensor:
    """Partial products into a workspace, then one kernel that adds them and applies the epilogue."""
    M, K = a.shape
    N = w.shape[0]
    work = scratch("splitk_partials", (splits * M * N,), torch.float32, a.device)
    emit_w, emit_op, emit_sq = emit if emit is not None else (None, None, None)
    _check(_lib().tl_linear_splitk(
        _ptr(a, 16), _ptr(w, 16), _ptr(out), _ptr(residual), _ptr(row_scale), _ptr(sumsq_in), c_int(parts),
        c_float(eps), c_int(width), _ptr(emit_w), c_int(_dt(emit_w) if emit_w is not None else 0), _ptr(emit_op),
        _ptr(emit_sq), c_int(M), c_int(N), c_int(K), c_int64(a.stride(0)), c_int64(out.stride(0)), c_int(_dt(out)),
        c_int(swiglu), _ptr(work, 16), _stream()), "linear_splitk")
    return out


def linear_handoff(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, residual: Optional[torch.Tensor] = None,
                   epilogue: Optional[str] = None, rows: Optional[torch.Tensor] = None, prepared=None,
                   emit=None) -> torch.Tensor:
    """The bfloat16 product with a norm handed over between products.

    emit = (norm_weight [N], operand [M, N] bfloat16, sumsq [M, handoff_parts(M, N, K)] float32):
    besides out = a @ w.T + residual (float32) the kernel writes operand = bf16(norm_weight * out)
    and the sums of out^2 over groups of columns.  prepared = (sumsq [R, P], eps, width): `a` is
    such an operand ([R, K]; `rows` picks rows of both) and the product is multiplied by
    1 / sqrt(sum(sumsq[row]) / width + eps): together the two are rmsnorm(out) @ w.T.
    At most 64 rows go to the few-row kernel, a product whose inner size is split (`split_k`) to
    its two kernels, any other to the tiled kernel (no `rows` then; emitting needs N % 64 == 0)."""
    _dev(a, w, out, residual, rows)
    _rows_2d(a, "linear input")
    _rows_2d(out, "linear output")
    K = a.shape[1]
    M = a.shape[0] if rows is None else rows.numel()
    N = w.shape[0]
    swiglu = _epilogue(epilogue)
    splits = split_k(M, N, K) if rows is None and M > 16 else 1
    if not (M > 0):
        _fail("no rows")
    if M > FEW_ROWS and splits == 1 and rows is not None:
        _fail(f"rows are gathered for at most {FEW_ROWS} of them")
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
            and w.shape[1] == K):
        _fail(f"input and weight must be bfloat16, weight contiguous [N, {K}]")
    if not (K % 8 == 0 and a.stride(0) % 8 == 0):
        _fail("inner size must be a multiple of 8")
    if rows is not None:
        if not (rows.dtype == torch.int32 and rows.is_contiguous()):
            _fail("row index must be contiguous int32")
    if swiglu:
        if not (N % 2 == 0 and tuple(out.shape) == (M, N // 2) and out.dtype == torch.bfloat16 and residual is None):
            _fail(f"the SiLU-gate epilogue writes bfloat16 [{M}, {N // 2}] and takes no residual")
    else:
        if not (tuple(out.shape) == (M, N) and out.dtype in (torch.float32, torch.bfloat16)):
            _fail(f"linear output must be [{M}, {N}], float32 or bfloat16")
    if residual is not None:
        if not (residual.dtype == torch.float32 and residual.shape == out.shape
                and residual.stride() == out.stride()):
            _fail("residual must be float32 with the output's layout")
    sumsq_in, parts, eps, width = None, 0, 0.0, 0
    if prepared is not None:
        sumsq_in, eps, width = prepared
        _dev(sumsq_in)
        if not (sumsq_in.dtype == torch.float32 and sumsq_in.dim() == 2 and sumsq_in.is_contiguous()
                and sumsq_in.shape[0] == a.shape[0] and width > 0):
            _fail("sums of squares must be contiguous float32 [rows of the input, parts]")
        parts = sumsq_in.shape[1]
    emit_w = emit_op = emit_sq = None
    if emit is not None:
        emit_w, emit_op, emit_sq = emit
        _dev(emit_w, emit_op, emit_sq)
        if not (not swiglu and out.dtype == torch.float32):
            _fail("only a float32 product without SiLU-gate prepares a norm")
        if not (emit_w.is_contiguous() and emit_w.numel() == N and emit_w.dtype in (torch.float32, torch.bfloat16)):
            _fail(f"norm weight must have {N} elements, float32 or bfloat16")
        if not (emit_op.dtype == torch.bfloat16 and emit_op.is_contiguous() and tuple(emit_op.shape) == (M, N)):
            _fail(f"operand must be contiguous bfloat16 [{M}, {N}]")
        if not (emit_sq.dtype == torch.float32 and emit_sq.is_contiguous()
                and tuple(emit_sq.shape) == (M, handoff_parts(M, N, K))):
            _fail(f"sums of squares must be float32 [{M}, {handoff_parts(M, N, K)}]")
    if splits > 1:
        return _linear_split(a, w, out, residual, swiglu, None, sumsq_in, parts, eps, width, emit, splits)
    _check(_lib().tl_linear_handoff(
        _ptr(a, 16), _ptr(w, 16), _ptr(out), _ptr(residual), _ptr(rows), _ptr(sumsq_in), c_int(parts), c_float(eps),
        c_int(width), _ptr(emit_w), c_int(_dt(emit_w) if emit_w is not None else 0), _ptr(emit_op), _ptr(emit_sq),
        c_int(M), c_int(N), c_int(K), c_int64(a.stride(0)), c_int64(out.stride(0)), c_int(_dt(out)), c_int(swiglu),
        _stream()), "linear_handoff")
    return out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor, pairs: bool = False) -> torch.Tensor:
    """out[t, j] = silu(gate_up[t, j]) * gate_up[t, I + j]; pairs: the rows hold (gate_j, up_j) side by side and
    out[t, j] = silu(gate_up[t, 2j]) * gate_up[t, 2j + 1]."""
    _dev(gate_up, out)
    T, I2 = gate_up.shape
    if not (I2 % 2 == 0 and gate_up.is_contiguous()):
        _fail("gate_up must be contiguous [T, 2I]")
    if not (out.dtype == gate_up.dtype and out.is_contiguous() and tuple(out.shape) == (T, I2 // 2)):
        _fail("silu_mul output must be contiguous [T, I] of the input's type")
    _check(_lib().tl_silu_mul(_ptr(gate_up), _ptr(out), c_int(T), c_int(I2 // 2), c_int(1 if pairs else 0),
                              c_int(_dt(gate_up)), _stream()), "silu_mul")
    return out


def add_residual(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """x += y with x float32."""
    _dev(x, y)
    if not (x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.shape == y.shape):
        _fail("residual add needs contiguous operands of one shape, the sum in float32")
    _check(_lib().tl_add_residual(_ptr(x), _ptr(y), c_int64(x.numel()), c_int(_dt(y)), _stream()), "add_residual")
    return x


def rope_store(qkv: torch.Tensor, positions: torch.Tensor, cos: Optional[torch.Tensor],
               sin: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor],
               k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
               num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int, pairing: str = "half") -> None:
    """Rotate q and k of every row of qkv in place by the row's position and
    store k, v at the row's cache slot.  Caches: [blocks, kv_heads, block, head_dim].
    pairing: which dims of a head make the i-th rotated pair: "half" (i, i + rotary_dim / 2) or
    "interleaved" (2i, 2i + 1)."""
    if pairing not in ROPE_PAIRINGS:
        _fail(f"rotary pairing {pairing!r} is not built; known: {', '.join(ROPE_PAIRINGS)}")
    _dev(qkv, positions, cos, sin, slot_mapping, k_cache, v_cache)
    _rows_2d(qkv, "qkv")
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if not (qkv.shape[1] == width):
        _fail(f"qkv rows must be {width} wide")
    if not (positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() == T):
        _fail("positions must be contiguous int32, one per row")
    block_size = 1
    if rotary_dim:
        if not (cos is not None and sin is not None and cos.dtype == torch.float32
                and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
                and cos.shape == sin.shape and cos.shape[1] == rotary_dim // 2):
            _fail("angle tables must be float32 [positions, rotary_dim/2]")
    if slot_mapping is not None:
        if not (slot_mapping.dtype == torch.int32 and slot_mapping.is_contiguous() and slot_mapping.numel() == T):
            _fail("slot mapping must be contiguous int32, one per row")
        for c in (k_cache, v_cache):
            if not (c is not None and c.dtype == qkv.dtype and c.is_contiguous() and c.dim() == 4
                    and c.shape[1] == num_kv_heads and c.shape[3] == head_dim):
                _fail("cache must be contiguous [blocks, kv_heads, block, head_dim] of the activations' type")
        if not (k_cache.shape == v_cache.shape):
            _fail("key and value caches must have one shape")
        block_size = k_cache.shape[2]
    _check(_lib().tl_rope_store(_ptr(qkv), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
                                _ptr(k_cache), _ptr(v_cache), c_int(T), c_int(num_heads), c_int(num_kv_heads),
                                c_int(head_dim), c_int(rotary_dim), c_int(block_size), c_int64(qkv.stride(0)),
                                c_int(_dt(qkv)), c_int(ROPE_PAIRINGS.index(pairing)), _stream()), "rope_store")


ROPE_PAIRINGS = ("half", "interleaved")     # the rotation kernel's pairings, by the number it takes


def _attn_flags(sink: bool, q: torch.Tensor, out: torch.Tensor) -> int:
    """The flags the attention kernels take in their `sink` argument: bit 0 the sink term, bit 1 a float32 result
    from operands of another type (the general kernel and the bfloat16 kernels)."""
    return (1 if sink else 0) | (2 if (out.dtype == torch.float32 and q.dtype != torch.float32) else 0)


def _attn_types_ok(q, k_cache, v_cache, out) -> bool:
    return q.dtype == k_cache.dtype == v_cache.dtype and out.dtype in (q.dtype, torch.float32)


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_tables: torch.Tensor, req_of_token: torch.Tensor, positions: torch.Tensor,
                    out: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                    window: int = 0, sink: bool = False) -> torch.Tensor:
    """Causal attention of every row of q (at its absolute position) over its
    request's cached keys 0..position (the last `window` of them if window > 0).
    sink: the softmax's denominator has one more term, exp(0), that carries no value."""
    _dev(q, k_cache, v_cache, block_tables, req_of_token, positions, out)
    _rows_2d(q, "q")
    _rows_2d(out, "attention output")
    T = q.shape[0]
    if not (q.shape[1] == num_heads * head_dim and tuple(out.shape) == (T, num_heads * head_dim)):
        _fail("q and the attention output must be [T, heads * head_dim]")
    if not _attn_types_ok(q, k_cache, v_cache, out):
        _fail("q and caches must share an element type; the output has it too or is float32")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dim() == 4
            and k_cache.shape == v_cache.shape and k_cache.shape[1] == num_kv_heads
            and k_cache.shape[3] == head_dim):
        _fail("cache must be contiguous [blocks, kv_heads, block, head_dim]")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()):
        _fail("block tables must be contiguous int32 [requests, max_blocks]")
    for t in (req_of_token, positions):
        if not (t.dtype == torch.int32 and t.is_contiguous() and t.numel() == T):
            _fail("per-token request ids and positions must be contiguous int32")
    if not (num_kv_heads > 0 and num_heads % num_kv_heads == 0):
        _fail("heads must be a multiple of kv heads")
    if not (head_dim <= MAX_HEAD_DIM):
        _fail(f"head_dim {head_dim} exceeds the attention kernel's limit of {MAX_HEAD_DIM}")
    _check(_lib().tl_paged_attention(
        _ptr(q), c_int64(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
        c_int(block_tables.shape[1]), _ptr(req_of_token), _ptr(positions), _ptr(out), c_int64(out.stride(0)),
        c_int(T), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_int(k_cache.shape[2]),
        c_float(scale), c_int(window), c_int(_attn_flags(sink, q, out)), c_int(_dt(q)), _stream()), "paged_attention")
    return out


F32_CHUNK_KEYS = 256     # keys per chunk of the float32 attention kernel's fixed merge tree


def attention_f32_supported(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Sizes the float32 matrix-core attention kernel takes; everything else goes to `paged_attention`."""
    return (dtype == torch.float32 and head_dim % 16 == 0 and head_dim <= 128 and num_kv_heads > 0
            and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16)


def attention_f32(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                  tiles, positions: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                  head_dim: int, scale: float, window: int = 0, n_chunks: int = 1,
                  scratch: Optional[torch.Tensor] = None, sink: bool = False) -> torch.Tensor:
    """The same function as `paged_attention` in true float32 on the matrix cores.  `tiles` as for
    `flash_attention` (None: row i is the one new token of request i).  n_chunks == 1: one
    workgroup per tile and kv head walks all keys; n_chunks > 1 (at least ceil(longest context /
    256)): the chunks of 256 keys go to workgroups of their own and float32 `scratch` of
    n_chunks * T * heads * (head_dim + 2) elements holds their results.  The bits of a row's result
    do not depend on n_chunks, on the tiles or on the rest of the batch."""
    tile_req, tile_tok0, tile_ntok = tiles if tiles is not None else (None, None, None)
    _dev(q, k_cache, v_cache, block_tables, tile_req, tile_tok0, tile_ntok, positions, out, scratch)
    _rows_2d(q, "q")
    _rows_2d(out, "attention output")
    T = q.shape[0]
    if not attention_f32_supported(q.dtype, num_heads, num_kv_heads, head_dim):
        _fail("the float32 matrix-core attention kernel takes float32, head sizes in steps of 16 up to 128, up "
              "to 16 heads per kv head")
    if not (q.shape[1] == num_heads * head_dim and tuple(out.shape) == (T, num_heads * head_dim)):
        _fail("q and the attention output must be [T, heads * head_dim]")
    if not (k_cache.dtype == v_cache.dtype == out.dtype == torch.float32):
        _fail("q, caches and output must be float32")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dim() == 4
            and k_cache.shape == v_cache.shape and k_cache.shape[1] == num_kv_heads
            and k_cache.shape[3] == head_dim):
        _fail("cache must be contiguous [blocks, kv_heads, block, head_dim]")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()):
        _fail("block tables must be contiguous int32 [requests, max_blocks]")
    if not (positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() == T):
        _fail("positions must be contiguous int32, one per row")
    if tiles is None:
        n_tiles = T
        if not (block_tables.shape[0] >= T):
            _fail("without tile arrays every row is a request of its own and needs a block table row")
    else:
        n_tiles = tile_req.numel()
        for t in (tile_req, tile_tok0, tile_ntok):
            if not (t.dtype == torch.int32 and t.is_contiguous() and t.numel() == n_tiles):
                _fail("tile arrays must be int32 [tiles]")
    if not (q.stride(0) % 4 == 0 and n_chunks >= 1):
        _fail("q rows must be 16-byte aligned and n_chunks positive")
    if n_chunks > 1:
        need = n_chunks * T * num_heads * (head_dim + 2)
        if not (scratch is not None and scratch.dtype == torch.float32 and scratch.is_contiguous()
                and scratch.numel() >= need):
            _fail(f"chunked attention needs {need} float32 of scratch")
    _check(_lib().tl_attention_f32(
        _ptr(q, 16), c_int64(q.stride(0)), _ptr(k_cache, 16), _ptr(v_cache, 16), _ptr(block_tables),
        c_int(block_tables.shape[1]), _ptr(tile_req), _ptr(tile_tok0), _ptr(tile_ntok), _ptr(positions),
        _ptr(out), c_int64(out.stride(0)), _ptr(scratch), c_int(n_tiles), c_int(T), c_int(num_heads),
        c_int(num_kv_heads), c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale), c_int(window), c_int(1 if sink else 0),
        c_int(n_chunks), _stream()), "attention_f32")
    return out


def flash_attention_supported(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Sizes the MFMA attention kernel takes; everything else goes to `paged_attention`."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 128 and num_kv_heads > 0
            and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16)


def flash_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    tiles, positions: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                    head_dim: int, scale: float, window: int = 0, n_splits: int = 1,
                    scratch: Optional[torch.Tensor] = None, fused_rope=None, static_scratch: bool = False,
                    sink: bool = False) -> torch.Tensor:
    """The same function as `paged_attention` on the matrix cores (bfloat16).  `tiles` =
    (tile_req, tile_tok0, tile_ntok): groups of at most 16 // (heads / kv_heads) consecutive
    tokens of one request; None for a decode step, where row i is the one new token of request i
    (the kernel then starts without waiting for the tile arrays).  n_splits > 1 needs float32 `scratch` of at least
    n_splits * T * heads * (head_dim + 2) elements.

    fused_rope=(cos, sin), for steps of ONE new token per request: `q` is the first slice of the
    unrotated rows [q heads | k heads | v heads]; the kernel rotates q and the new key over the
    whole head and writes the new key and value into the caches itself (no `rope_store` before).

    static_scratch=True: the partial results go to the device array the library holds itself
    (`tl_flash_attention_static`: no `scratch` is taken; sizes beyond that array are refused)."""
    tile_req, tile_tok0, tile_ntok = tiles if tiles is not None else (None, None, None)
    _dev(q, k_cache, v_cache, block_tables, tile_req, tile_tok0, tile_ntok, positions, out, scratch)
    _rows_2d(q, "q")
    _rows_2d(out, "attention output")
    T = q.shape[0]
    if not (flash_attention_supported(q.dtype, num_heads, num_kv_heads, head_dim)):
        _fail("the MFMA attention kernel takes bfloat16, head sizes in steps of 16 up to 128, up to 16 "
              "heads per kv head")
    if not (q.shape[1] == num_heads * head_dim and tuple(out.shape) == (T, num_heads * head_dim)):
        _fail("q and the attention output must be [T, heads * head_dim]")
    if not _attn_types_ok(q, k_cache, v_cache, out):
        _fail("q and caches must share an element type; the output has it too or is float32")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dim() == 4
            and k_cache.shape == v_cache.shape and k_cache.shape[1] == num_kv_heads
            and k_cache.shape[3] == head_dim):
        _fail("cache must be contiguous [blocks, kv_heads, block, head_dim]")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()):
        _fail("block tables must be contiguous int32 [requests, max_blocks]")
    if not (positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() == T):
        _fail("positions must be contiguous int32, one per row")
    if tiles is None:        # a decode step: row i is the one new token of request i
        n_tiles = T
        if not (block_tables.shape[0] >= T):
            _fail("without tile arrays every row is a request of its own and needs a block table row")
    else:
        n_tiles = tile_req.numel()
        for t in (tile_req, tile_tok0, tile_ntok):
            if not (t.dtype == torch.int32 and t.is_contiguous() and t.numel() == n_tiles):
                _fail("tile arrays must be int32 [tiles]")
    if not (q.stride(0) % 8 == 0):
        _fail("q rows must be 16-byte aligned")
    if not (k_cache.shape[0] * k_cache.shape[1] * k_cache.shape[2] < 2 ** 31):
        _fail("the attention kernel counts the rows of a cache in 32 bits")
    part_o = part_ml = None
    if n_splits > 1 and not static_scratch:
        need = n_splits * T * num_heads * (head_dim + 2)
        if not (scratch is not None and scratch.dtype == torch.float32 and scratch.is_contiguous()
                and scratch.numel() >= need):
            _fail(f"split attention needs {need} float32 of scratch")
        part_o = scratch[:n_splits * T * num_heads * head_dim]
        part_ml = scratch[n_splits * T * num_heads * head_dim:]
    cos = sin = None
    if fused_rope is not None:
        cos, sin = fused_rope
        _dev(cos, sin)
        if not (n_tiles == T):
            _fail("the fused rotation and cache write take one token per tile")
        if not (cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous()
                and sin.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == head_dim // 2):
            _fail("angle tables must be float32 [positions, head_dim / 2]")
        # q must be the head of a [q | k | v] row
        if not (q.stride(0) >= (num_heads + 2 * num_kv_heads) * head_dim):
            _fail("fused mode needs q inside its qkv rows")
    if static_scratch:
        code = _lib().tl_flash_attention_static(
            _ptr(q, 16), c_int64(q.stride(0)), _ptr(k_cache, 16), _ptr(v_cache, 16), _ptr(block_tables),
            c_int(block_tables.shape[1]), _ptr(tile_req), _ptr(tile_tok0), _ptr(tile_ntok), _ptr(positions),
            _ptr(out, 8), c_int64(out.stride(0)), c_int(n_tiles), c_int(T), c_int(num_heads), c_int(num_kv_heads),
            c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale), c_int(window), c_int(_attn_flags(sink, q, out)), c_int(n_splits), _ptr(cos),
            _ptr(sin), c_int(1 if fused_rope is not None else 0), _stream())
        if code == 3:
            _fail(f"split attention over the library's static scratch: {n_splits} splits x {T} tokens x {num_heads} "
                  f"heads x {head_dim + 2} floats exceed its {STATIC_SCRATCH_FLOATS} floats")
        _check(code, "flash_attention_static")
        return out
    _check(_lib().tl_flash_attention(
        _ptr(q, 16), c_int64(q.stride(0)), _ptr(k_cache, 16), _ptr(v_cache, 16), _ptr(block_tables),
        c_int(block_tables.shape[1]), _ptr(tile_req), _ptr(tile_tok0), _ptr(tile_ntok), _ptr(positions),
        _ptr(out, 8), c_int64(out.stride(0)), _ptr(part_o), _ptr(part_ml), c_int(n_tiles), c_int(T),
        c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale),
        c_int(window), c_int(_attn_flags(sink, q, out)), c_int(n_splits), _ptr(cos), _ptr(sin),
        c_int(1 if fused_rope is not None else 0), _stream()), "flash_attention")
    return out


STATIC_SCRATCH_FLOATS = 1 << 20     # capacity of the library's own scratch array (csrc/no_alloc.h)


def flash_waves(head_dim: int, groups: int = 1 << 20) -> int:
    """Waves of a `flash_attention` workgroup in a launch of `groups` query tiles x kv heads: each
    takes one 64-key tile per round trip to memory."""
    key = (head_dim, min(groups, 1 << 20))
    n = _WAVES.get(key)
    if n is None:
        n = _WAVES[key] = int(_lib().tl_flash_waves(c_int(head_dim), c_int(key[1])))
    return n


_WAVES: dict = {}


def decode_key_splits(num_tokens: int, max_seq_len: int, num_kv_heads: int, head_dim: int) -> int:
    """Over how many workgroups `flash_attention` shares one query tile's keys out in a decode step of
    `num_tokens` rows.  The waves of a workgroup take a 64-key tile each per round trip to memory (the
    next one is on its way while a tile is worked on).  Up to two tiles a wave nothing is split: the
    partial results of a split are merged by a second kernel, which costs more than a wave's second
    tile (measured on whole decode steps at contexts of 9 to 16 key tiles: 1.5 % of the step).  Longer
    contexts are split until a wave has one tile (at 17 to 32 key tiles two tiles a wave with a merge
    are 3 to 5 % of the step slower than one), as far as that keeps the launch within about 256
    workgroups (beyond that the splits only queue up) and within the kernel's 64.  One request at
    131,072 tokens: 36 us with 64 splits, 79 with 16, 1,090 with none (heads of 64, 4 kv heads).
    A launch of more workgroups than compute units runs in rounds, and a last round that is mostly empty
    takes as long as a full one (320 workgroups: two rounds for the work of 1.25); where the contexts
    are long (eight key tiles a wave and more even after it) the keys are split further, 2, 4 or 8 ways,
    if that fills the rounds better (8 requests x 40 kv heads at 32,768 tokens: 912 us with 4 splits,
    1,174 with none)."""
    groups = max(1, num_tokens * num_kv_heads)
    key_tiles = -(-max_seq_len // 64)
    room = max(1, 256 // groups)
    per_wave = -(-key_tiles // flash_waves(head_dim, groups))       # key tiles a wave, unsplit
    if per_wave <= 2:
        return 1
    n_splits = max(1, min(per_wave, room, 64))
    if groups * n_splits > 256:
        def rounds_per_split(s):
            return -(-groups * s // 256) / s
        best = n_splits
        for more in (2, 4, 8):
            s = n_splits * more
            if s <= 64 and per_wave >= 8 * s and rounds_per_split(s) < 0.95 * rounds_per_split(best):
                best = s
        n_splits = best
    return n_splits


PREFILL_TILES = 8     # query tiles (of 16 rows) one workgroup of the prefill attention kernel owns


def prefill_key_splits(num_tokens: int, max_seq_len: int, num_heads: int, num_kv_heads: int, tile_waves: int) -> int:
    """Over how many workgroups `flash_prefill` shares the key tiles of a query tile out: 1 unless the
    step has few query tiles (fewer than two workgroups a compute unit) and contexts of 16 key tiles and
    more; then one split per 8 key tiles of the longest context, at most 4 (8 from 32,768 tokens of
    context on: a portion of 512 tokens at 131,072 takes 1.30 ms with 8, 1.42 with 4, 2.29 with none).
    (Chosen by the time of whole steps: timed alone, with keys and values in the caches, fewer and larger
    workgroups look faster than they are in a model.  A whole prompt of 2,048 tokens has two workgroups a
    compute unit without any split: 7.4 -> 7.05 ms.)"""
    tiles = -(-num_tokens // (tile_waves * (16 // (num_heads // num_kv_heads))))
    key_tiles = -(-max_seq_len // 64)
    if key_tiles < 16:
        return 1
    if tiles * num_kv_heads >= 512:
        # Portions of thousands of tokens at the end of 65,536 tokens and more: four splits although the
        # launch is several rounds long already; the workgroups that run together then read the same
        # quarter of the keys (a layer's keys and values of one request are hundreds of megabytes there).
        # 8,192 rows at 131,072: 32.1 ms against 36.2 (heads of 128, 8 kv heads), 15.2 either way (64, 4).
        return 4 if key_tiles >= 1024 and tiles * num_kv_heads * 4 <= 16384 else 1
    most, launch = (8, 2048) if key_tiles >= 512 else (4, 1024)      # splits, workgroups of the launch
    return max(1, min(most, key_tiles // 8, launch // max(1, tiles * num_kv_heads)))


def prefill_tile_waves(num_tokens: int, num_heads: int, num_kv_heads: int) -> int:
    """Waves (query tiles of 16 rows) per workgroup of `flash_prefill` for a step of `num_tokens`:
    eight, or four where eight would give fewer workgroups than the chip has compute units."""
    per_tile = PREFILL_TILES * (16 // (num_heads // num_kv_heads))
    return 8 if -(-num_tokens // per_tile) * num_kv_heads >= 256 else 4


def flash_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                  tiles, positions: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                  head_dim: int, scale: float, window: int = 0, tile_waves: int = 8, n_splits: int = 1,
                  scratch: Optional[torch.Tensor] = None, sink: bool = False) -> torch.Tensor:
    """`flash_attention` arranged for prompt portions: `tiles` are groups of at most
    tile_waves * (16 // (heads / kv_heads)) consecutive tokens of one request, and a key or value
    row is staged once per such group.  tile_waves is PREFILL_TILES (8), or 4 for steps with few
    tokens, where workgroups of eight waves would leave compute units without work
    (`prefill_tile_waves`).  n_splits > 1 shares a group's key tiles out over that many workgroups
    (few query rows over long contexts: a portion late in a long prompt) and needs float32 `scratch`
    of n_splits * T * heads * (head_dim + 2) elements for their results, which a second kernel merges."""
    tile_req, tile_tok0, tile_ntok = tiles
    _dev(q, k_cache, v_cache, block_tables, tile_req, tile_tok0, tile_ntok, positions, out)
    _rows_2d(q, "q")
    _rows_2d(out, "attention output")
    T = q.shape[0]
    if not (flash_attention_supported(q.dtype, num_heads, num_kv_heads, head_dim)):
        _fail("the MFMA attention kernel takes bfloat16, head sizes in steps of 16 up to 128, up to 16 "
              "heads per kv head")
    if not (q.shape[1] == num_heads * head_dim and tuple(out.shape) == (T, num_heads * head_dim)):
        _fail("q and the attention output must be [T, heads * head_dim]")
    if not _attn_types_ok(q, k_cache, v_cache, out):
        _fail("q and caches must share an element type; the output has it too or is float32")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dim() == 4
            and k_cache.shape == v_cache.shape and k_cache.shape[1] == num_kv_heads
            and k_cache.shape[3] == head_dim):
        _fail("cache must be contiguous [blocks, kv_heads, block, head_dim]")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()):
        _fail("block tables must be contiguous int32 [requests, max_blocks]")
    if not (positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() == T):
        _fail("positions must be contiguous int32, one per row")
    n_tiles = tile_req.numel()
    for t in (tile_req, tile_tok0, tile_ntok):
        if not (t.dtype == torch.int32 and t.is_contiguous() and t.numel() == n_tiles):
            _fail("tile arrays must be int32 [tiles]")
    if not (q.stride(0) % 8 == 0 and out.stride(0) % 4 == 0):
        _fail("q and output rows must be vector aligned")
    if not (k_cache.shape[0] * k_cache.shape[1] * k_cache.shape[2] < 2 ** 31):
        _fail("the prefill attention kernel counts the rows of a cache in 32 bits")
    part_o = part_ml = None
    if n_splits > 1:
        need = n_splits * T * num_heads * (head_dim + 2)
        _dev(scratch)
        if not (scratch is not None and scratch.dtype == torch.float32 and scratch.is_contiguous()
                and scratch.numel() >= need):
            _fail(f"split attention needs {need} float32 of scratch")
        part_o = scratch[:n_splits * T * num_heads * head_dim]
        part_ml = scratch[n_splits * T * num_heads * head_dim:]
    _check(_lib().tl_flash_prefill(
        _ptr(q, 16), c_int64(q.stride(0)), _ptr(k_cache, 16), _ptr(v_cache, 16), _ptr(block_tables),
        c_int(block_tables.shape[1]), _ptr(tile_req), _ptr(tile_tok0), _ptr(tile_ntok), _ptr(positions),
        _ptr(out, 16 if out.dtype == torch.float32 else 8), c_int64(out.stride(0)), _ptr(part_o, 16), _ptr(part_ml), c_int(n_tiles), c_int(T),
        c_int(num_heads), c_int(num_kv_heads),
        c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale), c_int(window), c_int(_attn_flags(sink, q, out)), c_int(tile_waves), c_int(n_splits),
        _stream()), "flash_prefill")
    return out


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           seeds: Optional[torch.Tensor] = None, counters: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of float32 logits.  temperature <= 0 (or None): first
    maximum.  Otherwise temperature -> top-k -> top-p -> multinomial with the
    uniform number drawn from (seeds[row], counters[row])."""
    _dev(logits, out, temperature, top_k, top_p, seeds, counters)
    _rows_2d(logits, "logits")
    n, V = logits.shape
    if not (logits.dtype == torch.float32):
        _fail("logits must be float32")
    if not (out.dtype == torch.int32 and out.is_contiguous() and out.numel() == n):
        _fail("token output must be int32 [rows]")
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p"), (seeds, torch.int64, "seeds"),
                        (counters, torch.int32, "counters")):
        if t is not None:
            if not (t.dtype == dt and t.is_contiguous() and t.numel() == n):
                _fail(f"{name} must be contiguous {dt} [rows]")
    _check(_lib().tl_sample(_ptr(logits), c_int64(logits.stride(0)), c_int(n), c_int(V), _ptr(temperature),
                            _ptr(top_k), _ptr(top_p), _ptr(seeds), _ptr(counters), _ptr(out), _stream()), "sample")
    return out


def random_normal(out: torch.Tensor, table: torch.Tensor, key: int, scale: float, shift: float) -> torch.Tensor:
    """out.flat[i] = shift + scale * table[hash(key, i)], a pure function of (key, i): the numbers of
    random-weights mode (weights/loader.py gives the formula).  table: float32, a power of two long."""
    _dev(out, table)
    n = table.numel()
    if not (table.dtype == torch.float32 and table.is_contiguous() and n >= 2 and n & (n - 1) == 0):
        _fail("the quantile table must be contiguous float32 with a power-of-two length")
    if not out.is_contiguous():
        _fail("the output must be contiguous")
    _check(_lib().tl_random_normal(_ptr(out), c_int64(out.numel()), ctypes.c_uint64(key & ((1 << 64) - 1)), _ptr(table),
                                   c_int(n.bit_length() - 1), c_float(scale), c_float(shift), c_int(_dt(out)),
                                   _stream()), "random_normal")
    return out


# ------------------------------------------------------------- measured peaks
def peak_stream(src: torch.Tensor, dst: Optional[torch.Tensor], sink: torch.Tensor, blocks: int = 2048) -> None:
    """Streams through `src` (and copies it to `dst` if given): the kernel the measurement
    program times for the memory bandwidth the machine gives."""
    _dev(src, dst, sink)
    nbytes = src.numel() * src.element_size()
    if not (src.is_contiguous() and nbytes % 16 == 0 and sink.dtype == torch.float32 and sink.numel() >= 1):
        _fail("the source must be contiguous with a multiple of 16 bytes, the sink float32")
    if dst is not None and not (dst.is_contiguous() and dst.numel() * dst.element_size() >= nbytes):
        _fail("the destination must be contiguous and at least as large as the source")
    _check(_lib().tl_peak_stream(_ptr(src, 16), _ptr(dst, 16), _ptr(sink), c_int64(nbytes), c_int(0 if dst is None else 1),
                                 c_int(blocks), _stream()), "peak_stream")


def peak_mfma(sink: torch.Tensor, dtype: torch.dtype, iters: int, blocks: int = 1024) -> float:
    """Launches a loop of independent matrix instructions on registers; returns its flops."""
    _dev(sink)
    flops = ctypes.c_double(0.0)
    _check(_lib().tl_peak_mfma(_ptr(sink), c_int(_DT[dtype]), c_int(iters), c_int(blocks), ctypes.byref(flops), _stream()),
           "peak_mfma")
    return float(flops.value)


def peak_handover(workgroups: int = 256, rounds: int = 2000, payload: int = 16, spin_limit: int = 1 << 20) -> float:
    """Microseconds one hand-over of `payload` floats from every workgroup to every other takes inside ONE
    launch of `workgroups` resident workgroups (write-through stores, a flag per workgroup, loads past
    the caches): what a dependent phase would cost a persistent kernel, beside the time between two
    dependent launches.  Raises if a wait ran out or a value was read wrong."""
    if not (0 < workgroups <= 256 and rounds > 0 and payload > 0):
        _fail("1 to 256 workgroups, at least one round and one float")
    dev = torch.device("cuda", torch.cuda.current_device())
    flags = torch.zeros(256, dtype=torch.int32, device=dev)
    data = torch.zeros(2 * workgroups * payload, dtype=torch.float32, device=dev)
    state = torch.zeros(2, dtype=torch.int32, device=dev)

    def launch():
        _check(_lib().tl_peak_handover(_ptr(flags), _ptr(data), c_int(workgroups), c_int(rounds), c_int(payload),
                                       ctypes.c_uint(spin_limit), _ptr(state[0:1]), _ptr(state[1:2]), _stream()),
               "peak_handover")
    launch()
    torch.cuda.synchronize()
    flags.zero_()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    launch()
    e1.record()
    torch.cuda.synchronize()
    gave_up, wrong = state.cpu().tolist()
    if gave_up or wrong:
        _fail(f"hand-over probe: a wait ran out ({gave_up}) or {wrong} values were read wrong")
    return e0.elapsed_time(e1) * 1e3 / rounds


MAX_CACHE_GROUPS = 16       # cache groups the decode hand-over kernel takes (csrc/elementwise.hip)


def decode_advance(tokens: torch.Tensor, positions: torch.Tensor, seq_lens: torch.Tensor, counters: torch.Tensor,
                   sampled: torch.Tensor, history: torch.Tensor, step: torch.Tensor, slot_mappings, block_tables,
                   block_size: int) -> None:
    """Turns the metadata of a decode step into that of the next one on the device: the sampled
    token of each request becomes its input, position, cached length and sampling counter go up by
    one, the cache slot is looked up for the new position.  history [steps, R] records the tokens,
    `step` (one int32) counts the steps since the host last wrote the metadata."""
    R = tokens.numel()
    G = len(slot_mappings)
    ints = [tokens, positions, seq_lens, counters, sampled, history, step, *slot_mappings, *block_tables]
    _dev(*ints)
    for t in ints:
        if not (t.dtype == torch.int32 and t.is_contiguous()):
            _fail("decode_advance takes contiguous int32 tensors")
    if not (G == len(block_tables) and G <= MAX_CACHE_GROUPS):
        _fail(f"decode_advance takes up to {MAX_CACHE_GROUPS} cache groups")
    if not (all(t.numel() == R for t in (positions, seq_lens, counters, *slot_mappings)) and sampled.numel() >= R
            and step.numel() >= 1 and history.numel() % R == 0):
        _fail("decode_advance: one element per request in every per-request tensor")
    if not all(bt.dim() == 2 and bt.shape[0] == R and bt.shape[1] == block_tables[0].shape[1] for bt in block_tables):
        _fail("block tables must be [requests, max_blocks] of one width")
    slots_arr = (c_void_p * MAX_CACHE_GROUPS)(*[t.data_ptr() for t in slot_mappings], *[0] * (MAX_CACHE_GROUPS - G))
    tables_arr = (c_void_p * MAX_CACHE_GROUPS)(*[t.data_ptr() for t in block_tables], *[0] * (MAX_CACHE_GROUPS - G))
    _check(_lib().tl_decode_advance(_ptr(tokens), _ptr(positions), _ptr(seq_lens), _ptr(counters), _ptr(sampled),
                                    _ptr(history), _ptr(step), c_int(R), c_int(G),
                                    c_int(block_tables[0].shape[1] if G else 1), c_int(block_size),
                                    c_int(history.numel() // R), slots_arr, tables_arr, _stream()), "decode_advance")


# ------------------------------------------------- sublayers with the norm on their output
def _f32_vec(t: Optional[torch.Tensor], n: int, what: str) -> None:
    if t is not None and not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n):
        _fail(f"{what} must be contiguous float32 with {n} elements")


def _i32(*tensors) -> None:
    for t in tensors:
        if not (t.dtype == torch.int32 and t.is_contiguous()):
            _fail("index tensors must be contiguous int32")


def norm_scale_add(y: torch.Tensor, weight: torch.Tensor, eps: float, x: torch.Tensor,
                   scale: Optional[torch.Tensor] = None, copy: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += scale * weight * y / sqrt(mean(y^2) + eps), all float32; `copy` (optional, float32 or
    bfloat16, x's shape) receives the new x.  `weight` is the norm's effective weight."""
    _dev(y, weight, x, scale, copy)
    if not (y.dtype == torch.float32 and x.dtype == torch.float32 and y.dim() == 2 and y.is_contiguous()
            and x.is_contiguous() and x.shape == y.shape):
        _fail("norm_scale_add takes contiguous float32 [T, H] for the sublayer's output and the residual stream")
    T, H = y.shape
    _f32_vec(weight, H, "the norm's weight")
    _f32_vec(scale, H, "the channel scale")
    if copy is not None and not (copy.is_contiguous() and copy.shape == x.shape):
        _fail("the copy of the residual stream must be contiguous with its shape")
    _check(_lib().tl_norm_scale_add(_ptr(y), _ptr(weight), _ptr(scale), _ptr(x), _ptr(copy), c_int(T), c_int(H),
                                    c_float(eps), c_int(_dt(copy) if copy is not None else 0), _stream()),
           "norm_scale_add")
    return x


def cast_rows(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = x (float32) in out's element type."""
    _dev(x, out)
    if not (x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous() and out.shape == x.shape):
        _fail("cast_rows takes contiguous operands of one shape, the input in float32")
    _check(_lib().tl_cast_rows(_ptr(x), _ptr(out), c_int64(x.numel()), c_int(_dt(out)), _stream()), "cast_rows")
    return out


def clamped_glu(gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float, shift: float) -> torch.Tensor:
    """out[t, j] = g * sigmoid(alpha * g) * (u + shift) with g = min(gate_up[t, j], limit) and
    u = clamp(gate_up[t, I + j], -limit, limit)."""
    _dev(gate_up, out)
    _rows_2d(gate_up, "gate_up")
    T, I = out.shape
    if not (gate_up.shape[0] == T and gate_up.shape[1] >= 2 * I and out.dtype == gate_up.dtype and out.is_contiguous()):
        _fail("clamped_glu: gate_up is [T, >= 2I], the output contiguous [T, I] of the same type")
    _check(_lib().tl_clamped_glu(_ptr(gate_up), _ptr(out), c_int(T), c_int(I), c_int64(gate_up.stride(0)),
                                 c_float(limit), c_float(alpha), c_float(shift), c_int(_dt(out)), _stream()),
           "clamped_glu")
    return out


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _dev(logits)
    if not (logits.dtype == torch.float32 and logits.is_contiguous() and cap > 0):
        _fail("softcap takes contiguous float32 logits and a positive cap")
    _check(_lib().tl_softcap(_ptr(logits), c_int64(logits.numel()), c_float(cap), _stream()), "softcap")
    return logits


# ---------------------------------------------------------- attention over cached latents
LATENT_MAX_RANK = 512       # latent size the attention kernel takes (csrc/latent_attention.hip)
LATENT_MAX_QUERY = 1024     # latent size + rotated dims


def check_latent_sizes(kv_rank: int, rot: int) -> None:
    if not (0 < kv_rank <= LATENT_MAX_RANK and 0 <= rot and rot % 2 == 0 and kv_rank + rot <= LATENT_MAX_QUERY):
        _fail(f"latent attention takes latents of up to {LATENT_MAX_RANK} and an even number of rotated "
              f"dims, together at most {LATENT_MAX_QUERY}; got {kv_rank} and {rot}")


def latent_prepare(d: torch.Tensor, q_off: int, q_rank: int, w_q: Optional[torch.Tensor], eps: float,
                   cq: Optional[torch.Tensor],
                   kv_off: int = 0, kv_rank: int = 0, rot: int = 0, rdims: int = 0,
                   w_kv: Optional[torch.Tensor] = None,
                   positions: Optional[torch.Tensor] = None, cos: Optional[torch.Tensor] = None,
                   sin: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
                   latent: Optional[torch.Tensor] = None, rope: Optional[torch.Tensor] = None,
                   pairing: str = "half") -> None:
    """Row t of d holds the down projections.  cq[t] = w_q * unit_rms(d[t, q_off : q_off + q_rank]);
    with kv_rank > 0 also latent[slots[t]] = w_kv * unit_rms(d[t, kv_off : kv_off + kv_rank]) and
    rope[slots[t]] = the next `rot` columns, the first `rdims` of them rotated by the angle tables' row
    positions[t] (pairing "half": pairs (i, i + rdims/2); "interleaved": (2i, 2i + 1)).  latent / rope are the
    paged tensors [blocks, block_size, width].  q_rank == 0: the layer has no query latent (w_q and cq None)."""
    _dev(d, w_q, cq, w_kv, positions, cos, sin, slots, latent, rope)
    _rows_2d(d, "projections")
    T = d.shape[0]
    _need(pairing in ROPE_PAIRINGS, f"latent_prepare: pairing {pairing!r} is not built")
    _need(q_rank > 0 or kv_rank > 0, "latent_prepare: nothing to prepare")
    if q_rank > 0:
        _need(w_q is not None and cq is not None, "latent_prepare: a query latent needs its norm weight and its output")
        _f32_vec(w_q, q_rank, "the query latent's norm weight")
        if not (cq.dtype == d.dtype and cq.is_contiguous() and tuple(cq.shape) == (T, q_rank)
                and 0 <= q_off and q_off + q_rank <= d.shape[1]):
            _fail("latent_prepare: the query latent must be contiguous [T, q_rank] of the projections' type")
    if kv_rank > 0:
        _f32_vec(w_kv, kv_rank, "the latent's norm weight")
        _i32(positions, slots)
        if not (kv_off >= 0 and kv_off + kv_rank + rot <= d.shape[1] and positions.numel() == T and slots.numel() == T):
            _fail("latent_prepare: columns or per-token tensors do not fit")
        if not (latent.dtype == d.dtype and latent.is_contiguous() and latent.shape[-1] == kv_rank):
            _fail("latent_prepare: the latent cache must be contiguous [..., kv_rank] of the projections' type")
        if rot:
            if not (rope.dtype == d.dtype and rope.is_contiguous() and rope.shape[-1] == rot
                    and rope.numel() // rot == latent.numel() // kv_rank):
                _fail("latent_prepare: the rotated-key cache must be contiguous [..., rot] with the latent cache's slots")
            if not (cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous()
                    and sin.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rdims // 2
                    and 0 < rdims <= rot and rdims % 2 == 0):
                _fail("latent_prepare: angle tables are float32 [positions, rdims / 2]")
    _check(_lib().tl_latent_prepare(_ptr(d), c_int64(d.stride(0)), c_int(q_off), c_int(q_rank), c_int(kv_off),
                                    c_int(kv_rank), c_int(rot), c_int(rdims if kv_rank > 0 else 0), _ptr(w_q), _ptr(w_kv),
                                    c_float(eps), _ptr(positions),
                                    _ptr(cos), _ptr(sin), _ptr(slots), _ptr(cq), _ptr(latent), _ptr(rope), c_int(T),
                                    c_int(ROPE_PAIRINGS.index(pairing)), c_int(_dt(d)), _stream()), "latent_prepare")


def rotate_into(q: torch.Tensor, heads: int, head_width: int, in_off: int, rot: int, rdims: int,
                positions: torch.Tensor,
                cos: torch.Tensor, sin: torch.Tensor, out: torch.Tensor, out_off: int,
                pairing: str = "half") -> torch.Tensor:
    """out[t, h, out_off : out_off + rot] (float32) = the dims in_off : in_off + rot of head h of
    row t of q, the first `rdims` of them rotated by the angle tables' row positions[t] (pairs
    (i, i + rdims/2), or (2i, 2i + 1) with pairing "interleaved"), the others as they are."""
    _dev(q, positions, cos, sin, out)
    _need(pairing in ROPE_PAIRINGS, f"rotate_into: pairing {pairing!r} is not built")
    _rows_2d(q, "rotate_into input")
    _i32(positions)
    T = q.shape[0]
    if not (q.shape[1] >= heads * head_width and out.dtype == torch.float32 and out.is_contiguous() and out.dim() == 3
            and out.shape[0] == T and out.shape[1] == heads and positions.numel() == T
            and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous()
            and sin.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rdims // 2
            and 0 < rdims <= rot and rdims % 2 == 0):
        _fail("rotate_into: shapes do not fit")
    _check(_lib().tl_rotate_into(_ptr(q), c_int64(q.stride(0)), c_int(head_width), c_int(in_off), c_int(rot),
                                 c_int(rdims), c_int(heads), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(out), c_int(out.shape[2]),
                                 c_int(out_off), c_int(T), c_int(ROPE_PAIRINGS.index(pairing)), c_int(_dt(q)), _stream()),
           "rotate_into")
    return out


def latent_attention(qa: torch.Tensor, latent: torch.Tensor, rope: Optional[torch.Tensor], block_tables: torch.Tensor,
                     req_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, scale: float,
                     gate: Optional[torch.Tensor] = None, window: int = 0,
                     sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """qa float32 [T, heads, kv_rank + rot] = [W_uk^T q_unrotated | q_rotated]; latent / rope the paged
    tensors [blocks, block_size, kv_rank] / [blocks, block_size, rot].  out[t, h] = sigmoid(gate[t, h])
    * sum_j softmax_j((qa[t, h] . [latent_j | rope_j]) * scale) latent_j over the request's positions
    j <= positions[t].  gate [T, heads] may be a view with a row stride.  window > 0: only the positions
    j > positions[t] - window.  sinks (float32 [heads]): exp(sinks[h]) joins head h's denominator."""
    _dev(qa, latent, rope, block_tables, req_of_token, positions, out, gate, sinks)
    _i32(block_tables, req_of_token, positions)
    T, H, W = qa.shape
    _f32_vec(sinks, H, "latent_attention sinks")
    _need(window >= 0, "latent_attention: the window is 0 (none) or positive")
    kv_rank = latent.shape[-1]
    rot = W - kv_rank
    check_latent_sizes(kv_rank, rot)
    if not (qa.dtype == torch.float32 and qa.is_contiguous() and latent.dim() == 3 and latent.is_contiguous()
            and block_tables.dim() == 2 and req_of_token.numel() == T and positions.numel() == T):
        _fail("latent_attention: queries are contiguous float32 [T, heads, kv_rank + rot], the cache [blocks, block_size, kv_rank]")
    if rot and not (rope is not None and rope.dtype == latent.dtype and rope.is_contiguous()
                    and tuple(rope.shape) == (*latent.shape[:2], rot)):
        _fail("latent_attention: the rotated-key cache must be [blocks, block_size, rot] of the cache's type")
    if not (out.dtype == latent.dtype and out.is_contiguous() and tuple(out.shape) == (T, H, kv_rank)):
        _fail("latent_attention: the output is contiguous [T, heads, kv_rank] of the cache's type")
    if gate is not None and not (gate.dtype == latent.dtype and gate.dim() == 2 and gate.stride(1) == 1
                                 and tuple(gate.shape) == (T, H)):
        _fail("latent_attention: the gate is [T, heads] of the cache's type")
    _check(_lib().tl_latent_attention(_ptr(qa), _ptr(latent), _ptr(rope), _ptr(block_tables),
                                      c_int(block_tables.shape[1]), _ptr(req_of_token), _ptr(positions), _ptr(gate),
                                      c_int64(gate.stride(0) if gate is not None else 0), _ptr(out), c_int(T),
                                      c_int(H), c_int(kv_rank), c_int(rot), c_int(latent.shape[1]), c_float(scale),
                                      c_int(window), _ptr(sinks), c_int(_dt(latent)), _stream()), "latent_attention")
    return out


def latent_flash_supported(dtype: torch.dtype, kv_rank: int, rot: int) -> bool:
    """Whether the matrix-core kernel takes these sizes (bfloat16 caches; else the general kernel runs)."""
    return dtype == torch.bfloat16 and kv_rank % 16 == 0 and 0 < kv_rank <= LATENT_MAX_RANK and rot % 8 == 0 \
        and 0 <= rot and kv_rank + rot <= 576


def latent_key_splits(groups: int, max_seq_len: int) -> int:
    """Into how many workgroups the keys of one query tile are split: enough to give the chip a round
    of workgroups when the step has few tiles (decoding), never fewer than 64 keys a workgroup."""
    if groups <= 0 or groups >= 256:
        return 1
    return max(1, min(256 // groups, -(-max_seq_len // 64), 64))


def latent_flash(qa: torch.Tensor, latent: torch.Tensor, rope: Optional[torch.Tensor], block_tables: torch.Tensor,
                 tiles, positions: torch.Tensor, out: torch.Tensor, scale: float, gate: Optional[torch.Tensor] = None,
                 n_splits: int = 1, scratch_buf: Optional[torch.Tensor] = None, window: int = 0,
                 sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`latent_attention` on the matrix cores (bfloat16 caches).  tiles = (tile_req, tile_tok0, tile_ntok)
    with at most 16 // min(heads, 16) tokens of one request each, or None: tile i is token i of request i.
    n_splits > 1: scratch_buf holds n_splits * T * heads * (kv_rank + 2) floats.  window, sinks: as there."""
    _dev(qa, latent, rope, block_tables, positions, out, gate, scratch_buf, sinks)
    _i32(block_tables, positions)
    T, H, W = qa.shape
    _f32_vec(sinks, H, "latent_flash sinks")
    _need(window >= 0, "latent_flash: the window is 0 (none) or positive")
    kv_rank = latent.shape[-1]
    rot = W - kv_rank
    if not latent_flash_supported(latent.dtype, kv_rank, rot):
        _fail(f"latent_flash takes bfloat16 latents of a multiple of 16 up to 512 and rotated dims of a multiple of 8; got {kv_rank}, {rot}")
    if not (qa.dtype == torch.float32 and qa.is_contiguous() and latent.dim() == 3 and latent.is_contiguous()
            and block_tables.dim() == 2 and positions.numel() == T):
        _fail("latent_flash: queries are contiguous float32 [T, heads, kv_rank + rot], the cache [blocks, block_size, kv_rank]")
    if rot and not (rope is not None and rope.dtype == latent.dtype and rope.is_contiguous()
                    and tuple(rope.shape) == (*latent.shape[:2], rot)):
        _fail("latent_flash: the rotated-key cache must be [blocks, block_size, rot] of the cache's type")
    if not (out.dtype == latent.dtype and out.is_contiguous() and tuple(out.shape) == (T, H, kv_rank)):
        _fail("latent_flash: the output is contiguous [T, heads, kv_rank] of the cache's type")
    if gate is not None and not (gate.dtype == latent.dtype and gate.dim() == 2 and gate.stride(1) == 1
                                 and tuple(gate.shape) == (T, H)):
        _fail("latent_flash: the gate is [T, heads] of the cache's type")
    if tiles is None:
        if not (block_tables.shape[0] >= T):
            _fail("latent_flash: without tile lists every token is a request of its own")
        treq = ttok = tn = None
        n_tiles = T
    else:
        treq, ttok, tn = tiles
        _dev(treq, ttok, tn)
        _i32(treq, ttok, tn)
        n_tiles = treq.numel()
        if not (ttok.numel() == n_tiles and tn.numel() == n_tiles):
            _fail("latent_flash: the three tile lists have one length")
    if n_splits > 1 and not (scratch_buf is not None and scratch_buf.dtype == torch.float32 and scratch_buf.is_contiguous()
                             and scratch_buf.numel() >= n_splits * T * H * (kv_rank + 2)):
        _fail("latent_flash: split keys need float32 scratch of n_splits * T * heads * (kv_rank + 2)")
    _check(_lib().tl_latent_flash(_ptr(qa), _ptr(latent, 16), _ptr(rope, 16), _ptr(block_tables),
                                  c_int(block_tables.shape[1]), _ptr(treq), _ptr(ttok), _ptr(tn), _ptr(positions),
                                  _ptr(gate), c_int64(gate.stride(0) if gate is not None else 0), _ptr(out, 8),
                                  _ptr(scratch_buf, 16), c_int(n_tiles), c_int(T), c_int(H), c_int(16 // min(H, 16)),
                                  c_int(kv_rank), c_int(rot), c_int(latent.shape[1]), c_float(scale),
                                  c_int(n_splits), c_int(window), _ptr(sinks), _stream()), "latent_flash")
    return out


LATENT_PREFILL_ROWS = 64        # from this many query rows on a step's latent attention shares staged key tiles


def latent_prefill(qa: torch.Tensor, latent: torch.Tensor, rope: Optional[torch.Tensor], block_tables: torch.Tensor,
                   tiles, positions: torch.Tensor, out: torch.Tensor, scale: float,
                   gate: Optional[torch.Tensor] = None, window: int = 0,
                   sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`latent_flash` for steps with many query rows: tiles = (tile_req, tile_tok0, tile_ntok) with at most
    4 * (16 // min(heads, 16)) tokens of one request each; the four waves of a workgroup share every staged
    key tile.  Same operands and result otherwise (no split keys)."""
    _dev(qa, latent, rope, block_tables, positions, out, gate, sinks)
    _i32(block_tables, positions)
    T, H, W = qa.shape
    _f32_vec(sinks, H, "latent_prefill sinks")
    _need(window >= 0, "latent_prefill: the window is 0 (none) or positive")
    kv_rank = latent.shape[-1]
    rot = W - kv_rank
    if not latent_flash_supported(latent.dtype, kv_rank, rot):
        _fail(f"latent_prefill takes bfloat16 latents of a multiple of 16 up to 512 and rotated dims of a multiple of 8; got {kv_rank}, {rot}")
    if not (qa.dtype == torch.float32 and qa.is_contiguous() and latent.dim() == 3 and latent.is_contiguous()
            and block_tables.dim() == 2 and positions.numel() == T and W % 8 == 0):
        _fail("latent_prefill: queries are contiguous float32 [T, heads, kv_rank + rot], the cache [blocks, block_size, kv_rank]")
    if rot and not (rope is not None and rope.dtype == latent.dtype and rope.is_contiguous()
                    and tuple(rope.shape) == (*latent.shape[:2], rot)):
        _fail("latent_prefill: the rotated-key cache must be [blocks, block_size, rot] of the cache's type")
    if not (out.dtype == latent.dtype and out.is_contiguous() and tuple(out.shape) == (T, H, kv_rank)):
        _fail("latent_prefill: the output is contiguous [T, heads, kv_rank] of the cache's type")
    if gate is not None and not (gate.dtype == latent.dtype and gate.dim() == 2 and gate.stride(1) == 1
                                 and tuple(gate.shape) == (T, H)):
        _fail("latent_prefill: the gate is [T, heads] of the cache's type")
    treq, ttok, tn = tiles
    _dev(treq, ttok, tn)
    _i32(treq, ttok, tn)
    n_tiles = treq.numel()
    if not (ttok.numel() == n_tiles and tn.numel() == n_tiles):
        _fail("latent_prefill: the three tile lists have one length")
    _check(_lib().tl_latent_prefill(_ptr(qa, 16), _ptr(latent, 16), _ptr(rope, 16), _ptr(block_tables),
                                    c_int(block_tables.shape[1]), _ptr(treq), _ptr(ttok), _ptr(tn), _ptr(positions),
                                    _ptr(gate), c_int64(gate.stride(0) if gate is not None else 0), _ptr(out, 8),
                                    c_int(n_tiles), c_int(H), c_int(16 // min(H, 16)), c_int(kv_rank), c_int(rot),
                                    c_int(latent.shape[1]), c_float(scale), c_int(window), _ptr(sinks), _stream()),
           "latent_prefill")
    return out


HEAD_PRODUCT_ROWS = 32      # up to this many rows the per-head products of a step run as ONE launch
HEAD_PRODUCT_INNER = 1024


def head_product_weights(w: torch.Tensor) -> torch.Tensor:
    """w [heads, inner, cols] as `head_products` wants it: contiguous, the columns padded with zeros to
    a multiple of 8 (a lane fetches eight columns of a weight row at once)."""
    pad = -w.shape[2] % 8
    return torch.nn.functional.pad(w, (0, pad)).contiguous() if pad else w.contiguous()


def _head_gate(gate: Optional[torch.Tensor], x: torch.Tensor, T: int, H: int, cols: int, what: str):
    if gate is not None:
        _dev(gate)
        _need(gate.dim() == 2 and gate.stride(1) == 1 and tuple(gate.shape) == (T, H * cols) and gate.dtype == x.dtype,
              f"{what}: the gate is [T, heads * cols] of the input's type (rows may be wider apart)")


def head_products(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, h, :] = w[h]^T x[t, h, :] for every head in one launch (steps of few rows):
    x [T, heads, >= inner] and out [T, heads, >= cols] may be views into wider rows (any row and
    head stride, unit inner stride); w [heads, inner, cols rounded up to 8] from `head_product_weights`,
    of x's type; out float32 or x's type (its last size says how many columns are real).  gate [T, heads * cols]
    (optional, x's type): out is multiplied by sigmoid(gate) element by element."""
    _dev(x, w, out)
    T, H = x.shape[0], x.shape[1]
    inner, cols = w.shape[1], out.shape[2]
    _head_gate(gate, x, T, H, cols, "head_products")
    if not (x.dim() == 3 and out.dim() == 3 and w.dim() == 3 and w.is_contiguous() and w.shape[0] == H
            and w.dtype == x.dtype and x.stride(2) == 1 and out.stride(2) == 1 and tuple(out.shape[:2]) == (T, H)
            and x.shape[2] == inner and w.shape[2] % 8 == 0 and 0 <= w.shape[2] - cols < 8
            and inner <= HEAD_PRODUCT_INNER and (out.dtype == x.dtype or out.dtype == torch.float32)):
        _fail("head_products: x [T, heads, inner], w [heads, inner, cols rounded up to 8], out [T, heads, cols]")
    _check(_lib().tl_head_products(_ptr(x), c_int64(x.stride(0)), c_int(x.stride(1)), _ptr(w, 16), _ptr(out),
                                   c_int64(out.stride(0)), c_int(out.stride(1)), c_int(T), c_int(H), c_int(inner),
                                   c_int(cols), c_int(w.shape[2]), _ptr(gate),
                                   c_int64(gate.stride(0) if gate is not None else 0), c_int(_dt(x)), c_int(_dt(out)),
                                   _stream()), "head_products")
    return out


def head_gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, h, :] = w[h] x[t, h, :] for every head in one launch on the matrix cores (bfloat16, any
    number of rows): x [T, heads, inner] and out [T, heads, cols] may be views into wider rows; w
    [heads, cols, inner] contiguous; out bfloat16 or float32.  gate: as in `head_products`."""
    _dev(x, w, out)
    T, H = x.shape[0], x.shape[1]
    cols, inner = w.shape[1], w.shape[2]
    _head_gate(gate, x, T, H, cols, "head_gemm")
    if not (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 3 and out.dim() == 3 and w.dim() == 3
            and w.is_contiguous() and w.shape[0] == H and x.stride(2) == 1 and out.stride(2) == 1
            and tuple(out.shape[:2]) == (T, H) and x.shape[2] == inner and out.shape[2] == cols and inner % 8 == 0
            and x.stride(0) % 8 == 0 and x.stride(1) % 8 == 0 and out.dtype in (torch.bfloat16, torch.float32)):
        _fail("head_gemm: bfloat16 x [T, heads, inner] (inner and strides multiples of 8), w [heads, cols, inner], out [T, heads, cols]")
    _check(_lib().tl_head_gemm(_ptr(x, 16), c_int64(x.stride(0)), c_int(x.stride(1)), _ptr(w, 16), _ptr(out),
                               c_int64(out.stride(0)), c_int(out.stride(1)), c_int(T), c_int(H), c_int(inner),
                               c_int(cols), _ptr(gate), c_int64(gate.stride(0) if gate is not None else 0),
                               c_int(_dt(out)), _stream()), "head_gemm")
    return out


# ------------------------------------------------------------------ gated delta rule
DELTA_MAX_DIM = 256     # key channels of a head (csrc/delta_rule.hip)
DELTA_MAX_TAPS = 16


def check_delta_sizes(heads: int, kv_heads: int, dim: int, vdim: int, taps: int) -> None:
    if not (heads > 0 and kv_heads > 0 and heads % kv_heads == 0 and 0 < dim <= DELTA_MAX_DIM and vdim > 0
            and 1 <= taps <= DELTA_MAX_TAPS):
        _fail(f"delta rule: heads must be a multiple of kv heads, key channels at most {DELTA_MAX_DIM}, "
              f"taps at most {DELTA_MAX_TAPS}; got {heads}/{kv_heads} heads, {dim} x {vdim}, {taps} taps")


def delta_prepare(p: torch.Tensor, conv_off: int, b_off: int, a: torch.Tensor, conv_w: torch.Tensor,
                  a_log: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor, saved_off: int,
                  req_of_token: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor, qn: torch.Tensor,
                  kn: torch.Tensor, vc: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor, heads: int,
                  kv_heads: int, dim: int, vdim: int, taps: int, q_scale: float, decay_per_head: bool = False) -> None:
    """What enters the recurrence, per token and head, in float32: q and k after their causal
    convolution and SiLU as unit vectors (q times q_scale), v after its convolution and SiLU, beta =
    sigmoid(p[t, b_off + h]) and decay = exp(-exp(a_log[h]) * softplus(a[t, h * dim + i] + dt_bias)); with
    decay_per_head `a` and dt_bias hold one number per head (a[t, h], dt_bias[h]) and every channel of the head
    gets the same decay.  Row t of p holds [q | k | v] from column conv_off on; inputs before a request's first
    token of the step come from its state row, at saved_off."""
    _dev(p, a, conv_w, a_log, dt_bias, state, req_of_token, cu_seqlens, state_slots, qn, kn, vc, beta, decay)
    check_delta_sizes(heads, kv_heads, dim, vdim, taps)
    _rows_2d(p, "projections")
    _rows_2d(a, "decay pre-activations")
    _i32(req_of_token, cu_seqlens, state_slots)
    T = p.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    _f32_vec(conv_w, channels * taps, "convolution taps")
    _f32_vec(a_log, heads, "A_log")
    n_decay = heads if decay_per_head else heads * dim
    _f32_vec(dt_bias, n_decay, "dt_bias")
    if not (a.dtype == torch.float32 and a.shape[0] == T and a.shape[1] >= n_decay
            and conv_off >= 0 and conv_off + channels <= p.shape[1] and 0 <= b_off and b_off + heads <= p.shape[1]):
        _fail("delta_prepare: columns do not fit")
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
            and saved_off + channels * (taps - 1) <= state.shape[1] and req_of_token.numel() == T):
        _fail("delta_prepare: the state is contiguous float32 [slots, row] with room for the saved inputs")
    for t, n in ((qn, T * heads * dim), (kn, T * heads * dim), (vc, T * heads * vdim), (beta, T * heads),
                 (decay, T * heads * dim)):
        _f32_vec(t, n, "delta_prepare outputs")
    _check(_lib().tl_delta_prepare(_ptr(p), c_int64(p.stride(0)), c_int(conv_off), c_int(b_off), _ptr(a),
                                   c_int64(a.stride(0)), _ptr(conv_w), _ptr(a_log), _ptr(dt_bias), _ptr(state),
                                   c_int64(state.stride(0)), c_int64(saved_off), _ptr(req_of_token), _ptr(cu_seqlens),
                                   _ptr(state_slots), _ptr(qn), _ptr(kn), _ptr(vc), _ptr(beta), _ptr(decay), c_int(T),
                                   c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim), c_int(taps),
                                   c_float(q_scale), c_int(1 if decay_per_head else 0), c_int(_dt(p)), _stream()),
           "delta_prepare")


def conv_state_update(p: torch.Tensor, conv_off: int, channels: int, state: torch.Tensor, saved_off: int,
                      cu_seqlens: torch.Tensor, state_slots: torch.Tensor, taps: int) -> None:
    """The saved inputs of the convolutions after this step: per request and channel the last
    taps - 1 of (what was saved, the step's inputs), oldest first."""
    _dev(p, state, cu_seqlens, state_slots)
    _rows_2d(p, "projections")
    _i32(cu_seqlens, state_slots)
    R = state_slots.numel()
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous() and cu_seqlens.numel() == R + 1
            and saved_off + channels * (taps - 1) <= state.shape[1] and conv_off + channels <= p.shape[1]
            and 1 <= taps <= DELTA_MAX_TAPS):
        _fail("conv_state_update: shapes do not fit")
    _check(_lib().tl_conv_state_update(_ptr(p), c_int64(p.stride(0)), c_int(conv_off), c_int(channels), _ptr(state),
                                       c_int64(state.stride(0)), c_int64(saved_off), _ptr(cu_seqlens),
                                       _ptr(state_slots), c_int(R), c_int(taps), c_int(_dt(p)), _stream()),
           "conv_state_update")


def delta_recurrence(qn: torch.Tensor, kn: torch.Tensor, vc: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor,
                     state: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor,
                     heads: int, dim: int, vdim: int) -> torch.Tensor:
    """Walks every request's tokens of this step through S <- diag(g) S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q, with S [heads, dim, vdim] at the start of the request's state row."""
    _dev(qn, kn, vc, beta, decay, state, cu_seqlens, state_slots, out)
    _i32(cu_seqlens, state_slots)
    R = state_slots.numel()
    T = beta.numel() // heads
    for t, n in ((qn, T * heads * dim), (kn, T * heads * dim), (vc, T * heads * vdim), (beta, T * heads),
                 (decay, T * heads * dim), (out, T * heads * vdim)):
        _f32_vec(t, n, "delta_recurrence operands")
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
            and heads * dim * vdim <= state.shape[1] and cu_seqlens.numel() == R + 1 and 0 < dim <= DELTA_MAX_DIM):
        _fail("delta_recurrence: the state is contiguous float32 [slots, >= heads * dim * vdim]")
    _check(_lib().tl_delta_recurrence(_ptr(qn), _ptr(kn), _ptr(vc), _ptr(beta), _ptr(decay), _ptr(state),
                                      c_int64(state.stride(0)), _ptr(cu_seqlens), _ptr(state_slots), _ptr(out),
                                      c_int(R), c_int(heads), c_int(dim), c_int(vdim), _stream()), "delta_recurrence")
    return out


DELTA_DECODE_MAX_VDIM = 256      # a thread per value column in the one-kernel decode step
DELTA_DECODE_MAX_TAPS = 4         # and its convolutions' inputs in registers


def delta_decode(p: torch.Tensor, conv_off: int, b_off: int, a: torch.Tensor, gate: torch.Tensor, conv_w: torch.Tensor,
                 a_log: torch.Tensor, dt_bias: torch.Tensor, w_norm: torch.Tensor, state: torch.Tensor,
                 saved_off: int, cu_seqlens: torch.Tensor, state_slots: torch.Tensor, z: torch.Tensor, heads: int,
                 kv_heads: int, dim: int, vdim: int, taps: int, q_scale: float, eps: float,
                 decay_per_head: bool = False, gate_kind: str = "sigmoid") -> bool:
    """A decode step of the delta rule in one kernel (every request brings one token; row t of the
    operands is request t): what `delta_prepare`, `delta_recurrence` and `head_norm_gate` do, with the decay's
    pre-activations `a` (float32 [T, heads * dim], or [T, heads] with decay_per_head) and the gate's `gate`
    (float32 [T, heads * vdim]; both may be views into wider rows), the gate's function "sigmoid" or "silu".
    Returns whether the saved convolution inputs were brought up to date as well (every head has q/k channels
    of its own); if not, `conv_state_update` has to follow."""
    _dev(p, a, gate, conv_w, a_log, dt_bias, w_norm, state, cu_seqlens, state_slots, z)
    check_delta_sizes(heads, kv_heads, dim, vdim, taps)
    _rows_2d(p, "projections")
    _rows_2d(a, "decay pre-activations")
    _rows_2d(gate, "gate pre-activations")
    _need(gate_kind in ("sigmoid", "silu"), f"delta_decode: unknown gate {gate_kind!r}")
    n_decay = heads if decay_per_head else heads * dim
    _i32(cu_seqlens, state_slots)
    R = state_slots.numel()
    channels = 2 * kv_heads * dim + heads * vdim
    _f32_vec(conv_w, channels * taps, "convolution taps")
    _f32_vec(a_log, heads, "A_log")
    _f32_vec(dt_bias, n_decay, "dt_bias")
    _f32_vec(w_norm, vdim, "the head norm's weight")
    if not (p.shape[0] == R and a.shape[0] == R and gate.shape[0] == R and a.dtype == gate.dtype == torch.float32
            and a.shape[1] >= n_decay and gate.shape[1] >= heads * vdim and conv_off + channels <= p.shape[1] and b_off + heads <= p.shape[1]
            and cu_seqlens.numel() == R + 1 and vdim <= DELTA_DECODE_MAX_VDIM and taps <= DELTA_DECODE_MAX_TAPS
            and vdim % 4 == 0 and state.stride(0) % 4 == 0
            and state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
            and saved_off + channels * (taps - 1) <= state.shape[1] and heads * dim * vdim <= saved_off
            and (z.dtype == p.dtype or p.dtype == torch.float32) and z.is_contiguous() and tuple(z.shape) == (R, heads * vdim)):
        _fail("delta_decode: shapes do not fit (one row per request)")
    _check(_lib().tl_delta_decode(_ptr(p), c_int64(p.stride(0)), c_int(conv_off), c_int(b_off), _ptr(a),
                                  c_int64(a.stride(0)), c_int(1 if decay_per_head else 0), _ptr(gate),
                                  c_int64(gate.stride(0)), c_int(1 if gate_kind == "silu" else 0), _ptr(conv_w), _ptr(a_log), _ptr(dt_bias), _ptr(w_norm),
                                  _ptr(state), c_int64(state.stride(0)), c_int64(saved_off), _ptr(cu_seqlens),
                                  _ptr(state_slots), _ptr(z), c_int(R), c_int(heads), c_int(kv_heads), c_int(dim),
                                  c_int(vdim), c_int(taps), c_float(q_scale), c_float(eps), c_int(heads == kv_heads),
                                  c_int(_dt(p)), c_int(_dt(z)), _stream()),
           "delta_decode")
    return heads == kv_heads


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, out: torch.Tensor, heads: int,
                   vdim: int, eps: float, gate_kind: str = "sigmoid", scale: float = 1.0) -> torch.Tensor:
    """out[t, h, :] = scale * weight * o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * act(gate[t, h, :]);
    o float32 [T, heads * vdim], gate float32 [T, heads * vdim] (a view with a row stride is fine);
    weight [vdim] (shared by the heads) or [heads * vdim]; act "sigmoid" or "silu" (g * sigmoid(g))."""
    _dev(o, weight, gate, out)
    T = out.shape[0]
    _f32_vec(o, T * heads * vdim, "head_norm_gate input")
    per_head = weight.numel() == heads * vdim and heads > 1
    _f32_vec(weight, heads * vdim if per_head else vdim, "the head norm's weight")
    if gate_kind not in ("sigmoid", "silu"):
        _fail(f"head_norm_gate: unknown gate {gate_kind!r}")
    if not (gate.dtype == torch.float32 and gate.dim() == 2 and gate.stride(1) == 1
            and tuple(gate.shape) == (T, heads * vdim) and out.is_contiguous() and tuple(out.shape) == (T, heads * vdim)):
        _fail("head_norm_gate: gate and output are [T, heads * vdim]")
    _check(_lib().tl_head_norm_gate(_ptr(o), _ptr(weight), c_int(vdim if per_head else 0), _ptr(gate),
                                    c_int64(gate.stride(0)), _ptr(out), c_int(T), c_int(heads), c_int(vdim), c_float(eps),
                                    c_int(1 if gate_kind == "silu" else 0), c_float(scale), c_int(_dt(out)), _stream()),
           "head_norm_gate")
    return out


# ------------------------------------------------- norm after the sum, with weight and bias
def layer_norm_sum(y: Optional[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor, x: torch.Tensor, alpha: float,
                   eps: float, copy: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[t] <- (v - mean(v)) / sqrt(var(v) + eps) * weight + bias with v = alpha * x[t] + y[t] (y None: alpha * x[t]),
    in place, float32; `copy` ([T, H], any element type of the engine) receives the new rows too."""
    _dev(y, weight, bias, x, copy)
    if not (x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()):
        _fail("layer_norm_sum: the stream is contiguous float32 [T, H]")
    T, H = x.shape
    if y is not None and not (y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (T, H)):
        _fail("layer_norm_sum: the sublayer's result is contiguous float32 [T, H]")
    _f32_vec(weight, H, "the layer norm's weight")
    _f32_vec(bias, H, "the layer norm's bias")
    if copy is not None and not (copy.is_contiguous() and tuple(copy.shape) == (T, H)):
        _fail("layer_norm_sum: the copy is contiguous [T, H]")
    _check(_lib().tl_layer_norm_sum(_ptr(y), _ptr(weight), _ptr(bias), _ptr(x), _ptr(copy), c_int(T), c_int(H),
                                    c_float(alpha), c_float(eps), c_int(_dt(copy) if copy is not None else 0), _stream()),
           "layer_norm_sum")
    return x


LAYER_NORM_ADD_MAX = 8192       # widest row `layer_norm_add` keeps in registers (csrc/layer_norm.hip)


def layer_norm_add(y: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, x: torch.Tensor, mult: float, eps: float,
                   then=None) -> torch.Tensor:
    """x[t] <- x[t] + mult * (LN(y[t]) * weight + bias), in place, float32 (y the sublayer's result, float32 [T, H]).
    then = (weight2, bias2, eps2, out): out[t] ([T, H] of either element type) also receives LN(x[t]) * weight2 +
    bias2 of the new rows, in the same kernel."""
    _dev(y, weight, bias, x)
    if not (x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()):
        _fail("layer_norm_add: the stream is contiguous float32 [T, H]")
    T, H = x.shape
    _need(H <= LAYER_NORM_ADD_MAX, f"layer_norm_add: rows of at most {LAYER_NORM_ADD_MAX} elements")
    if not (y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (T, H)):
        _fail("layer_norm_add: the sublayer's result is contiguous float32 [T, H]")
    _f32_vec(weight, H, "the layer norm's weight")
    _f32_vec(bias, H, "the layer norm's bias")
    w2 = b2 = out = None
    eps2 = 0.0
    if then is not None:
        w2, b2, eps2, out = then
        _dev(w2, b2, out)
        _f32_vec(w2, H, "the next norm's weight")
        _f32_vec(b2, H, "the next norm's bias")
        if not (out.is_contiguous() and tuple(out.shape) == (T, H)):
            _fail("layer_norm_add: the next norm's output is contiguous [T, H]")
    _check(_lib().tl_layer_norm_add(_ptr(y), _ptr(weight), _ptr(bias), _ptr(x), _ptr(w2), _ptr(b2), _ptr(out), c_int(T),
                                    c_int(H), c_float(mult), c_float(eps), c_float(eps2),
                                    c_int(_dt(out) if out is not None else 0), _stream()), "layer_norm_add")
    return x


def layer_norm_rows(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out: torch.Tensor,
                    rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i] = layer norm of x[rows[i] or i] (float32 [T, H]) times weight plus bias."""
    _dev(x, weight, bias, out, rows)
    if not (x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()):
        _fail("layer_norm_rows: the stream is contiguous float32 [T, H]")
    H, n = x.shape[1], out.shape[0]
    _f32_vec(weight, H, "the layer norm's weight")
    _f32_vec(bias, H, "the layer norm's bias")
    if not (out.dim() == 2 and out.is_contiguous() and out.shape[1] == H):
        _fail("layer_norm_rows: the output is contiguous [n, H]")
    if rows is None:
        _need(n == x.shape[0], "layer_norm_rows: output rows must match input rows")
    else:
        _i32(rows)
        _need(rows.numel() == n, "layer_norm_rows: one row index per output row")
    _check(_lib().tl_layer_norm_rows(_ptr(x), _ptr(rows), _ptr(weight), _ptr(bias), _ptr(out), c_int(n), c_int(H),
                                     c_float(eps), c_int(_dt(out)), _stream()), "layer_norm_rows")
    return out


# ------------------------------------------- queries and keys between their product and the attention
def qk_prepare(p: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor, cos: Optional[torch.Tensor],
               sin: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], q_out: torch.Tensor,
               k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], num_heads: int, num_kv_heads: int,
               head_dim: int, rot: int, pairing: str, unit_norm: bool, eps: float, values_are_keys: bool,
               v_off: int = -1) -> torch.Tensor:
    """From the float32 product p [T, >= (heads + kv_heads) * head_dim] (query heads, then key heads): bias added,
    the first `rot` dims of every head rotated by the token's position, every head divided by its root mean square
    (unit_norm); queries go to q_out [T, heads * head_dim], keys into k_cache at the tokens' slots.  values_are_keys:
    the keys as projected (bias added, before rotation and norm) go into v_cache; else the value heads at column
    v_off of p do (v_off < 0: no values are written).  A negative slot stores nothing."""
    _dev(p, bias, positions, cos, sin, slot_mapping, q_out, k_cache, v_cache)
    _rows_2d(p, "qk_prepare input")
    _rows_2d(q_out, "qk_prepare queries")
    T = p.shape[0]
    width = (num_heads + num_kv_heads) * head_dim
    _need(p.dtype == torch.float32 and p.shape[1] >= width, f"qk_prepare: the product is float32 [T, >= {width}]")
    _need(tuple(q_out.shape) == (T, num_heads * head_dim), "qk_prepare: queries are [T, heads * head_dim]")
    _need(head_dim % 2 == 0 and 0 < head_dim <= MAX_HEAD_DIM and 0 <= rot <= head_dim and rot % 2 == 0,
          f"qk_prepare: head_dim {head_dim} must be even and at most {MAX_HEAD_DIM}, rot even and within it")
    if pairing not in ROPE_PAIRINGS:
        _fail(f"rotary pairing {pairing!r} is not built; known: {', '.join(ROPE_PAIRINGS)}")
    if bias is not None:
        _f32_vec(bias, width, "qk_prepare bias")
    _i32(positions)
    _need(positions.numel() == T, "qk_prepare: one position per token")
    if rot:
        for t in (cos, sin):
            _need(t is not None and t.dtype == torch.float32 and t.is_contiguous() and t.dim() == 2
                  and t.shape[1] == rot // 2, "qk_prepare: angle tables are float32 [positions, rot / 2]")
    block = 1
    if slot_mapping is not None:
        _i32(slot_mapping)
        _need(slot_mapping.numel() == T, "qk_prepare: one slot per token")
        for c in (k_cache, v_cache):
            _need(c is not None and c.is_contiguous() and c.dim() == 4 and c.shape[1] == num_kv_heads
                  and c.shape[3] == head_dim and c.dtype == q_out.dtype,
                  "qk_prepare: caches are contiguous [blocks, kv_heads, block, head_dim] of the queries' type")
        _need(k_cache.shape == v_cache.shape, "qk_prepare: key and value caches have one shape")
        block = k_cache.shape[2]
    if not values_are_keys and v_off >= 0:
        _need(p.shape[1] >= v_off + num_kv_heads * head_dim, "qk_prepare: the value heads lie within the product's rows")
    _check(_lib().tl_qk_prepare(_ptr(p), c_int64(p.stride(0)), _ptr(bias), _ptr(positions), _ptr(cos), _ptr(sin),
                                _ptr(slot_mapping), _ptr(q_out), c_int64(q_out.stride(0)), _ptr(k_cache), _ptr(v_cache),
                                c_int(T), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_int(rot),
                                c_int(ROPE_PAIRINGS.index(pairing)), c_int(1 if unit_norm else 0), c_float(eps),
                                c_int(1 if values_are_keys else 0), c_int(v_off), c_int(block), c_int(_dt(q_out)),
                                _stream()), "qk_prepare")
    return q_out


def head_gate(a: torch.Tensor, g: torch.Tensor, out: torch.Tensor, heads: int, head_dim: int, scale: float = 1.0):
    """out[t, h, :] = a[t, h, :] * sigmoid(g[t, h]) * scale; a and out [T, heads * head_dim] of one type (out may be a),
    g float32 [T, heads] (a view with a row stride is fine)."""
    _dev(a, g, out)
    _rows_2d(a, "head_gate input")
    _rows_2d(out, "head_gate output")
    _rows_2d(g, "head_gate gates")
    T = a.shape[0]
    _need(tuple(a.shape) == (T, heads * head_dim) and a.shape == out.shape and a.dtype == out.dtype,
          "head_gate: input and output are [T, heads * head_dim] of one type")
    _need(g.dtype == torch.float32 and tuple(g.shape) == (T, heads), "head_gate: gates are float32 [T, heads]")
    _check(_lib().tl_head_gate(_ptr(a), c_int64(a.stride(0)), _ptr(g), c_int64(g.stride(0)), _ptr(out),
                               c_int64(out.stride(0)), c_int(T), c_int(heads), c_int(head_dim), c_float(scale),
                               c_int(_dt(a)), _stream()), "head_gate")
    return out


def gelu_glu(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, j] = gelu_tanh(gate_up[t, j]) * gate_up[t, F + j]; gate_up [T, 2F], out [T, F] contiguous, one type."""
    _dev(gate_up, out)
    _rows_2d(gate_up, "gelu_glu input")
    T, F = out.shape
    _need(gate_up.shape[0] == T and gate_up.shape[1] == 2 * F and out.is_contiguous() and out.dtype == gate_up.dtype,
          "gelu_glu: input [T, 2F], output contiguous [T, F] of the same type")
    _check(_lib().tl_gelu_glu(_ptr(gate_up), _ptr(out), c_int(T), c_int(F), c_int64(gate_up.stride(0)),
                              c_int(_dt(out)), _stream()), "gelu_glu")
    return out


# -------------------------------------------------------- time mixing with a decaying state
TIME_MIX_MAX_DIM = 256      # key channels of a head (csrc/time_mix.hip)
TIME_MIX_SLICE = 4


def time_mix_slices(dim: int) -> int:
    """Slices of 4 key channels a head's state is cut into (a power of two)."""
    p = 1
    while p * TIME_MIX_SLICE < dim:
        p *= 2
    return p


def time_mix_state_floats(heads: int, dim: int, vdim: int) -> int:
    """Floats of a request's state row that hold S, in the recurrence kernel's own layout."""
    return heads * TIME_MIX_SLICE * time_mix_slices(dim) * vdim


def shift_mix(h: torch.Tensor, state: torch.Tensor, prev_off: int, req_of_token: torch.Tensor, cu_seqlens: torch.Tensor,
              state_slots: torch.Tensor, mu: torch.Tensor, out: torch.Tensor, save_single: bool = False) -> torch.Tensor:
    """out[m, t] = h[t] + (h[t - 1] - h[t]) * mu[m]; for the first token a request brings in this step h[t - 1] is what
    its state row keeps at prev_off.  h [T, W] and out [M, T, W] of one type, mu float32 [M, W], state float32 rows.
    save_single: a request that brings exactly one token gets it saved as `shift_save` would (a step in which no
    request brings more needs no `shift_save` then)."""
    _dev(h, state, req_of_token, cu_seqlens, state_slots, mu, out)
    _rows_2d(h, "shift_mix input")
    T, W = h.shape
    M = mu.shape[0]
    _need(mu.dtype == torch.float32 and mu.is_contiguous() and tuple(mu.shape) == (M, W), "shift_mix: mu is float32 [M, W]")
    _need(out.is_contiguous() and tuple(out.shape) == (M, T, W) and out.dtype == h.dtype,
          "shift_mix: the output is contiguous [M, T, W] of the input's type")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= prev_off + W,
          "shift_mix: state rows are float32 and hold W values from prev_off")
    _i32(req_of_token, cu_seqlens, state_slots)
    _need(req_of_token.numel() == T and cu_seqlens.numel() == state_slots.numel() + 1,
          "shift_mix: one request index per token, cu_seqlens one entry more than there are requests")
    _check(_lib().tl_shift_mix(_ptr(h), c_int64(h.stride(0)), _ptr(state), c_int64(state.stride(0)), c_int64(prev_off),
                               _ptr(req_of_token), _ptr(cu_seqlens), _ptr(state_slots), _ptr(mu), _ptr(out), c_int(T),
                               c_int(M), c_int(W), c_int(1 if save_single else 0), c_int(_dt(h)), _stream()), "shift_mix")
    return out


def shift_save(h: torch.Tensor, state: torch.Tensor, prev_off: int, cu_seqlens: torch.Tensor,
               state_slots: torch.Tensor) -> None:
    """The last token every request brings in this step becomes its state row's saved h (float32)."""
    _dev(h, state, cu_seqlens, state_slots)
    _rows_2d(h, "shift_save input")
    W = h.shape[1]
    R = state_slots.numel()
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= prev_off + W,
          "shift_save: state rows are float32 and hold W values from prev_off")
    _i32(cu_seqlens, state_slots)
    _need(cu_seqlens.numel() == R + 1, "shift_save: cu_seqlens has one entry more than there are requests")
    _check(_lib().tl_shift_save(_ptr(h), c_int64(h.stride(0)), _ptr(state), c_int64(state.stride(0)), c_int64(prev_off),
                                _ptr(cu_seqlens), _ptr(state_slots), c_int(R), c_int(W), c_int(_dt(h)), _stream()),
           "shift_save")


def time_mix_recurrence(x: torch.Tensor, r_off: int, k_off: int, v_off: int, w_off: int, w0: torch.Tensor,
                        u: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor,
                        o: torch.Tensor, heads: int, dim: int, vdim: int) -> torch.Tensor:
    """Per request and head, over the request's tokens of this step in order, S from its state row:
    o_t = (S + diag(u) k_t v_t^T)^T r_t, then S <- diag(exp(-exp(x_w + w0))) S + k_t v_t^T.
    x float32 rows with r, k, the decay's pre-activation (heads * dim columns each) and v (heads * vdim) at the
    given column offsets; o float32 [T, heads * vdim].  A request that brings no token keeps its state."""
    _dev(x, w0, u, state, cu_seqlens, state_slots, o)
    _rows_2d(x, "time_mix_recurrence input")
    T = x.shape[0]
    R = state_slots.numel()
    _need(x.dtype == torch.float32, "time_mix_recurrence: the input is float32")
    _need(0 < dim <= TIME_MIX_MAX_DIM and vdim > 0 and 0 < heads <= 65535 and R <= 65535,
          f"time_mix_recurrence: heads of 1 to {TIME_MIX_MAX_DIM} key channels")
    for off, n in ((r_off, heads * dim), (k_off, heads * dim), (w_off, heads * dim), (v_off, heads * vdim)):
        _need(0 <= off and off + n <= x.shape[1], "time_mix_recurrence: a column range lies outside the input's rows")
    _f32_vec(w0, heads * dim, "the decay's bias")
    _f32_vec(u, heads * dim, "the bonus")
    _f32_vec(o, T * heads * vdim, "time_mix_recurrence output")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= time_mix_state_floats(heads, dim, vdim), "time_mix_recurrence: state rows are too short")
    _i32(cu_seqlens, state_slots)
    _need(cu_seqlens.numel() == R + 1, "time_mix_recurrence: cu_seqlens has one entry more than there are requests")
    _check(_lib().tl_time_mix_recurrence(_ptr(x), c_int64(x.stride(0)), c_int(r_off), c_int(k_off), c_int(v_off),
                                         c_int(w_off), _ptr(w0), _ptr(u), _ptr(state), c_int64(state.stride(0)),
                                         _ptr(cu_seqlens), _ptr(state_slots), _ptr(o), c_int(R), c_int(heads), c_int(dim),
                                         c_int(vdim), _stream()), "time_mix_recurrence")
    return o


def tanh_rows(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = tanh(x); x float32 [T, n] (a row stride is fine), out contiguous [T, n] of the engine's type."""
    _dev(x, out)
    _rows_2d(x, "tanh input")
    _need(x.dtype == torch.float32 and out.is_contiguous() and out.shape == x.shape, "tanh: float32 in, contiguous out")
    _check(_lib().tl_tanh_rows(_ptr(x), c_int64(x.stride(0)), _ptr(out), c_int(x.shape[0]), c_int(x.shape[1]),
                               c_int(_dt(out)), _stream()), "tanh_rows")
    return out


# ------------------------------------------------------------ experts looked up in a table
MOE_ACTIVATIONS = {None: 0, "relu2": 1}      # what may follow an expert's first product (csrc/moe.hip)
MOE_GATED = "swiglu"                         # `table_moe_up` only: an expert's rows are (gate_j, up_j) pairs, out = silu(gate) * up


def table_moe_up(a: torch.Tensor, w: torch.Tensor, tokens: Optional[torch.Tensor], table: torch.Tensor, out: torch.Tensor,
                 act: Optional[str] = None) -> torch.Tensor:
    """out[t * top + j] = act(w[table[tokens[t], j]] @ a[t]); a [T, K], w [E, N, K] of one type, table int32 [vocab, top],
    out contiguous [T * top, N].  tokens None: the table has a row per row of a (the experts a router chose).
    act None, "relu2" (the square of max(., 0)) or "swiglu": an expert's N rows are (gate_0, up_0, gate_1, up_1, ...) and
    out [T * top, N / 2] = silu(gate) * up, formed from the float32 sums."""
    _dev(a, w, tokens, table, out)
    _need(act in MOE_ACTIVATIONS or act == MOE_GATED, f"table_moe_up: activation {act!r} is not built")
    _rows_2d(a, "table_moe_up input")
    T, K = a.shape
    E, N, _ = w.shape
    V, top = table.shape
    _need(w.is_contiguous() and w.shape[2] == K and w.dtype == a.dtype == out.dtype, "table_moe_up: w is contiguous [E, N, K]")
    n_out = N // 2 if act == MOE_GATED else N
    _need(N % 2 == 0 or act != MOE_GATED, "table_moe_up: gated experts have an even number of rows")
    _need(out.is_contiguous() and tuple(out.shape) == (T * top, n_out), f"table_moe_up: the output is contiguous [T * top, {n_out}]")
    _i32(table)
    if tokens is not None:
        _i32(tokens)
        _need(tokens.numel() == T, "table_moe_up: one token id per row")
    else:
        _need(V >= T and table.is_contiguous(), "table_moe_up: without token ids the table has a row per row of the input")
    _check(_lib().tl_table_moe_up(_ptr(a), c_int64(a.stride(0)), _ptr(w), _ptr(tokens), _ptr(table), _ptr(out), c_int(T),
                                  c_int(top), c_int(E), c_int(V), c_int(N), c_int(K),
                                  c_int(2 if act == MOE_GATED else MOE_ACTIVATIONS[act]), c_int(_dt(a)), _stream()),
           "table_moe_up")
    return out


def table_moe_down(z: torch.Tensor, w: torch.Tensor, tokens: Optional[torch.Tensor], table: torch.Tensor,
                   out: torch.Tensor, coef: float, base: Optional[torch.Tensor] = None,
                   base_scale: Optional[torch.Tensor] = None, row_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = base[t] * base_scale[t] + coef * sum_j row_weights[t, j] * w[table[tokens[t], j]] @ z[t * top + j];
    z [T * top, K], w [E, N, K], out float32 [T, N] (may be base); base float32 [T, N], base_scale float32 [T],
    row_weights float32 [T, top], all three optional.  tokens None: the table has a row per token of the step."""
    _dev(z, w, tokens, table, out, base, base_scale, row_weights)
    E, N, K = w.shape
    V, top = table.shape
    T = tokens.numel() if tokens is not None else out.shape[0]
    if tokens is None:
        _need(V >= T and table.is_contiguous(), "table_moe_down: without token ids the table has a row per token")
    if row_weights is not None:
        _f32_vec(row_weights, T * top, "table_moe_down row_weights")
    _need(w.is_contiguous() and z.is_contiguous() and tuple(z.shape) == (T * top, K) and z.dtype == w.dtype,
          "table_moe_down: z is contiguous [T * top, K], w contiguous [E, N, K]")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, N),
          "table_moe_down: the output is contiguous float32 [T, N]")
    if base is not None:
        _need(base.dtype == torch.float32 and base.is_contiguous() and base.shape == out.shape,
              "table_moe_down: base is contiguous float32 [T, N]")
    if base_scale is not None:
        _f32_vec(base_scale, T, "table_moe_down base_scale")
    _i32(table)
    if tokens is not None:
        _i32(tokens)
    _check(_lib().tl_table_moe_down(_ptr(z), _ptr(w), _ptr(tokens), _ptr(table), _ptr(base), _ptr(base_scale),
                                    _ptr(row_weights), _ptr(out),
                                    c_int(T), c_int(top), c_int(E), c_int(V), c_int(N), c_int(K), c_float(coef),
                                    c_int(_dt(z)), _stream()), "table_moe_down")
    return out


MOE_TILE_ROWS = 32          # rows of one expert a tile of the grouped product holds (csrc/moe.hip)


MOE_RUN_ROWS = 256          # rows of one expert a run of the tiled product's rows holds (a multiple of its tile heights)


def moe_max_tiles(rows: int, experts: int, tile_rows: int = MOE_TILE_ROWS) -> int:
    return -(-rows // tile_rows) + experts


def moe_plan_ints(rows: int, experts: int, tile_rows: int = MOE_TILE_ROWS) -> int:
    """int32 elements of the plan `moe_plan` fills for `rows` (= tokens * top) rows."""
    return 3 * experts + 2 + 3 * moe_max_tiles(rows, experts, tile_rows) + rows


def moe_plan(tokens: Optional[torch.Tensor], table: torch.Tensor, plan: torch.Tensor, experts: int,
             tile_rows: int = MOE_TILE_ROWS, num_tokens: Optional[int] = None) -> torch.Tensor:
    """Sorts the step's rows (token t, its j-th expert: row t * top + j) by expert on the device and lists
    tiles of at most `tile_rows` rows of one expert each; `plan` is int32 scratch of `moe_plan_ints` elements:
    counts[E], cursors[E], offsets[E + 1], the number of tiles, then per tile (capacity `moe_max_tiles`) its
    expert (-1 behind the last tile), its first place in the sorted rows and its number of rows, then the rows
    sorted by expert.  tokens None: the table has a row per token of the step, `num_tokens` of them."""
    _dev(tokens, table, plan)
    _i32(table, plan)
    V, top = table.shape
    if tokens is not None:
        _i32(tokens)
        T = tokens.numel()
    else:
        T = int(num_tokens)
        _need(0 < T <= V and table.is_contiguous(), "moe_plan: without token ids the table has a row per token")
    _need(plan.numel() >= moe_plan_ints(T * top, experts, tile_rows), "moe_plan: the plan is too short")
    _need(0 < experts <= 1024, "moe_plan: 1 to 1024 experts")
    plan[:2 * experts].zero_()          # counts and cursors (a fill kernel: fine inside a captured step)
    _check(_lib().tl_moe_plan(_ptr(tokens), _ptr(table), _ptr(plan), c_int(T), c_int(top), c_int(experts), c_int(V),
                              c_int(moe_max_tiles(T * top, experts, tile_rows)), c_int(tile_rows), _stream()), "moe_plan")
    return plan


def moe_tile_experts(plan: torch.Tensor, rows: int, experts: int, tile_rows: int) -> torch.Tensor:
    """The plan's list of experts by tile (-1: the tile holds no row)."""
    at = 3 * experts + 2
    return plan[at:at + moe_max_tiles(rows, experts, tile_rows)]


def moe_gather(a: Optional[torch.Tensor], a_div: int, plan: torch.Tensor, rows: int, experts: int, tile_rows: int,
               dst: Optional[torch.Tensor], row_pos: Optional[torch.Tensor]) -> None:
    """The plan's rows side by side, a tile after the other: dst[tile * tile_rows + i] = a[row // a_div] (bfloat16;
    a None: nothing is copied) and row_pos[row] = tile * tile_rows + i (int32 [rows]; None: not wanted)."""
    _dev(a, plan, dst, row_pos)
    _i32(plan)
    mt = moe_max_tiles(rows, experts, tile_rows)
    _need(plan.numel() >= moe_plan_ints(rows, experts, tile_rows), "moe_gather: the plan is too short")
    K = 8
    if a is not None:
        _rows_2d(a, "moe_gather input")
        K = a.shape[1]
        _need(a.dtype == torch.bfloat16 and dst is not None and dst.dtype == torch.bfloat16 and dst.is_contiguous()
              and tuple(dst.shape) == (mt * tile_rows, K) and K % 8 == 0 and a.stride(0) % 8 == 0
              and a.shape[0] * a_div >= rows, "moe_gather: a [*, K] and contiguous dst [tiles * tile_rows, K] are bfloat16")
    if row_pos is not None:
        _i32(row_pos)
        _need(row_pos.numel() >= rows, "moe_gather: one place per row")
    _check(_lib().tl_moe_gather(_ptr(a, 16), c_int64(a.stride(0) if a is not None else 0), c_int(a_div), _ptr(dst, 16),
                                _ptr(row_pos), _ptr(plan), c_int(experts), c_int(mt), c_int(tile_rows), c_int(K),
                                _stream()), "moe_gather")


def linear_grouped(a: torch.Tensor, w: torch.Tensor, tile_group: torch.Tensor, out: torch.Tensor,
                   epilogue: Optional[str] = None) -> torch.Tensor:
    """out = a @ w[g]^T by runs of 256 rows: run r of a (bfloat16 [runs * 256, K]) multiplies w[tile_group[r]]
    (bfloat16 [G, N, K]); a run whose entry is negative is skipped (its rows of out are not written).  out
    [runs * 256, N] bfloat16 or float32.  The tiled product of `linear` with a weight matrix per run of rows.
    epilogue="swiglu" as there: the N columns are (gate_j, up_j) pairs and out [runs * 256, N / 2] (bfloat16) =
    silu(gate) * up, from the float32 accumulators."""
    _dev(a, w, tile_group, out)
    _rows_2d(a, "linear_grouped input")
    _rows_2d(out, "linear_grouped output")
    M, K = a.shape
    G, N, _ = w.shape
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.is_contiguous() and w.shape[2] == K,
          "linear_grouped: a [M, K] and contiguous w [G, N, K] are bfloat16")
    _need(M % MOE_RUN_ROWS == 0 and K % 8 == 0 and a.stride(0) % 8 == 0, "linear_grouped: runs of 256 rows, K a multiple of 8")
    swiglu = _epilogue(epilogue)
    if swiglu:
        _need(N % 2 == 0 and tuple(out.shape) == (M, N // 2) and out.dtype == torch.bfloat16,
              "linear_grouped: the SiLU-gate epilogue writes bfloat16 [M, N / 2]")
    else:
        _need(tuple(out.shape) == (M, N), "linear_grouped: out is [M, N]")
    _i32(tile_group)
    _need(tile_group.numel() >= M // MOE_RUN_ROWS, "linear_grouped: one group per run of rows")
    _check(_lib().tl_linear_grouped(_ptr(a, 16), _ptr(w, 16), _ptr(out, 16), _ptr(tile_group), c_int(MOE_RUN_ROWS),
                                    c_int(M), c_int(N), c_int(K), c_int64(a.stride(0)), c_int64(out.stride(0)),
                                    c_int(_dt(out)), c_int(swiglu), _stream()), "linear_grouped")
    return out


def moe_combine_at(y: torch.Tensor, row_pos: torch.Tensor, out: torch.Tensor, top: int, coef: float,
                   base: Optional[torch.Tensor] = None, base_scale: Optional[torch.Tensor] = None,
                   row_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = base[t] * base_scale[t] + coef * sum_j row_weights[t, j] * y[row_pos[t * top + j]]; y float32 [*, N],
    out float32 [T, N]; row_weights float32 [T, top], optional."""
    _dev(y, row_pos, out, base, base_scale, row_weights)
    T, N = out.shape
    if row_weights is not None:
        _f32_vec(row_weights, T * top, "moe_combine_at row_weights")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "moe_combine_at: out is contiguous float32 [T, N]")
    _need(y.dtype == torch.float32 and y.is_contiguous() and y.dim() == 2 and y.shape[1] == N,
          "moe_combine_at: y is contiguous float32 [*, N]")
    _i32(row_pos)
    _need(row_pos.numel() >= T * top, "moe_combine_at: one place per row")
    if base is not None:
        _need(base.dtype == torch.float32 and base.is_contiguous() and base.shape == out.shape,
              "moe_combine_at: base is contiguous float32 [T, N]")
    if base_scale is not None:
        _f32_vec(base_scale, T, "moe_combine_at base_scale")
    _check(_lib().tl_moe_combine_at(_ptr(y), _ptr(row_pos), _ptr(base), _ptr(base_scale), _ptr(row_weights), _ptr(out),
                                    c_int(T), c_int(N),
                                    c_int(top), c_float(coef), _stream()), "moe_combine_at")
    return out


def grouped_rows_gemm(a: torch.Tensor, a_div: int, w: torch.Tensor, plan: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[r] = w[expert of row r] @ a[r // a_div] for every row r of the plan, on the matrix cores (bfloat16
    operands, float32 sums); a [*, K], w [E, N, K] bfloat16, out contiguous [rows, N] bfloat16 or float32."""
    _dev(a, w, plan, out)
    _rows_2d(a, "grouped_rows_gemm input")
    E, N, K = w.shape
    rows = out.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.is_contiguous() and a.shape[1] == K,
          "grouped_rows_gemm: a [*, K] and contiguous w [E, N, K] are bfloat16")
    _need(K % 8 == 0 and a.stride(0) % 8 == 0, "grouped_rows_gemm: inner size and row stride are multiples of 8")
    _need(out.is_contiguous() and out.shape[1] == N and a.shape[0] * a_div >= rows,
          "grouped_rows_gemm: out is contiguous [rows, N], a holds rows / a_div rows")
    _i32(plan)
    _need(plan.numel() >= moe_plan_ints(rows, E), "grouped_rows_gemm: the plan is too short (tiles of 32 rows)")
    _check(_lib().tl_grouped_rows_gemm(_ptr(a, 16), c_int64(a.stride(0)), c_int(a_div), _ptr(w, 16), _ptr(out),
                                       _ptr(plan), c_int(rows), c_int(E), c_int(moe_max_tiles(rows, E)), c_int(N),
                                       c_int(K), c_int(_dt(out)), _stream()), "grouped_rows_gemm")
    return out


def moe_combine(y: torch.Tensor, out: torch.Tensor, top: int, coef: float, base: Optional[torch.Tensor] = None,
                base_scale: Optional[torch.Tensor] = None, row_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = base[t] * base_scale[t] + coef * sum_j row_weights[t, j] * y[t * top + j]; all float32, out may be
    base; row_weights [T, top], optional."""
    _dev(y, out, base, base_scale, row_weights)
    T, N = out.shape
    if row_weights is not None:
        _f32_vec(row_weights, T * top, "moe_combine row_weights")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "moe_combine: out is contiguous float32 [T, N]")
    _f32_vec(y, T * top * N, "moe_combine input")
    if base is not None:
        _need(base.dtype == torch.float32 and base.is_contiguous() and base.shape == out.shape,
              "moe_combine: base is contiguous float32 [T, N]")
    if base_scale is not None:
        _f32_vec(base_scale, T, "moe_combine base_scale")
    _check(_lib().tl_moe_combine(_ptr(y), _ptr(base), _ptr(base_scale), _ptr(row_weights), _ptr(out), c_int(T), c_int(N),
                                 c_int(top),
                                 c_float(coef), _stream()), "moe_combine")
    return out


def row_dot_sigmoid(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = sigmoid(a[t] . w); a [T, K] and w [K] of one type, out float32 [T]."""
    _dev(a, w, out)
    _rows_2d(a, "row_dot_sigmoid input")
    T, K = a.shape
    _need(w.is_contiguous() and w.numel() == K and w.dtype == a.dtype, "row_dot_sigmoid: w is [K] of the input's type")
    _f32_vec(out, T, "row_dot_sigmoid output")
    _check(_lib().tl_row_dot_sigmoid(_ptr(a), c_int64(a.stride(0)), _ptr(w), _ptr(out), c_int(T), c_int(K),
                                     c_int(_dt(a)), _stream()), "row_dot_sigmoid")
    return out


MOE_MAX_ROUTED = 1024       # experts the router kernel takes (csrc/moe.hip)


def moe_route(z: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, groups: int = 1, keep: int = 1,
              scale: float = 1.0, bias: Optional[torch.Tensor] = None) -> None:
    """A router over the logits z (float32 [T, E], rows may be wider apart; `bias`, float32 [E], is added to every
    row if given): scores s = softmax(z) over all experts;
    the experts lie in `groups` equal runs of neighbours, a run's score is its largest, and only experts of the
    `keep` best runs may be chosen (groups <= 1: all may); ids[t] (int32 [T, top]) names the `top` largest scores
    among those, largest first (equal scores: the lower index first), and weights[t] (float32 [T, top]) =
    their scores / (their sum + 1e-20) * scale."""
    _dev(z, ids, weights)
    _rows_2d(z, "moe_route logits")
    T, E = z.shape
    top = ids.shape[1] if ids.dim() == 2 else 0
    _need(z.dtype == torch.float32, "moe_route: logits are float32")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and tuple(ids.shape) == (T, top) and top > 0,
          "moe_route: ids are contiguous int32 [T, top]")
    _f32_vec(weights, T * top, "moe_route weights")
    if bias is not None:
        _dev(bias)
        _f32_vec(bias, E, "moe_route bias")
    _need(0 < top <= E <= MOE_MAX_ROUTED, f"moe_route: 1 to {MOE_MAX_ROUTED} experts, top within them")
    if groups > 1:
        _need(E % groups == 0 and 0 < keep <= groups and top <= keep * (E // groups),
              "moe_route: equal groups, 1 to `groups` of them kept, holding at least `top` experts")
    _check(_lib().tl_moe_route(_ptr(z), c_int64(z.stride(0)), _ptr(bias), _ptr(ids), _ptr(weights), c_int(T), c_int(E), c_int(top),
                               c_int(groups), c_int(keep), c_float(scale), _stream()), "moe_route")


def activate_rows(x: torch.Tensor, out: torch.Tensor, act: Optional[str]) -> torch.Tensor:
    """out = act(x) element by element (act as in `table_moe_up`); x [T, N] float32 or of out's type, its rows may be
    wider apart; out contiguous [T, N]."""
    _dev(x, out)
    _rows_2d(x, "activate_rows input")
    _need(act in MOE_ACTIVATIONS, f"activate_rows: activation {act!r} is not built")
    _need(out.is_contiguous() and out.shape == x.shape and (x.dtype == out.dtype or x.dtype == torch.float32),
          "activate_rows: out is contiguous, of the input's shape, and of its type unless the input is float32")
    _check(_lib().tl_activate_rows(_ptr(x), c_int64(x.stride(0)), _ptr(out), c_int(x.shape[0]), c_int(x.shape[1]),
                                   c_int(MOE_ACTIVATIONS[act]), c_int(_dt(x)), c_int(_dt(out)), _stream()), "activate_rows")
    return out


def gate_rows(a: torch.Tensor, g: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = a * sigmoid(g) element by element; a, g, out [T, N] of one type, each may be a view into wider rows
    (out may be a)."""
    _dev(a, g, out)
    for t, name in ((a, "gate_rows input"), (g, "gate_rows gate"), (out, "gate_rows output")):
        _rows_2d(t, name)
    _need(a.shape == g.shape == out.shape and a.dtype == g.dtype == out.dtype, "gate_rows: one shape and one type")
    _check(_lib().tl_gate_rows(_ptr(a), c_int64(a.stride(0)), _ptr(g), c_int64(g.stride(0)), _ptr(out),
                               c_int64(out.stride(0)), c_int(a.shape[0]), c_int(a.shape[1]), c_int(_dt(a)), _stream()),
           "gate_rows")
    return out


def embedding_pairs(tokens: torch.Tensor, positions: torch.Tensor, req_of_token: torch.Tensor, cu_seqlens: torch.Tensor,
                    state_slots: torch.Tensor, prev_state: torch.Tensor, table: torch.Tensor, pairs: torch.Tensor,
                    out: torch.Tensor, mul_prev: int, mul_cur: int, scale: float) -> torch.Tensor:
    """out[t] = table[tokens[t]] * scale + pairs[(prev * mul_prev + tokens[t] * mul_cur) mod buckets] as float32,
    `prev` the token before it in its request; a request's first token (position 0) takes the last row of pairs
    ([buckets + 1, H]).  prev_state (int32, one element per state slot) keeps every request's last token between
    steps: read for the first token a request brings, then overwritten with the last one it brings."""
    _dev(tokens, positions, req_of_token, cu_seqlens, state_slots, prev_state, table, pairs, out)
    _i32(tokens, positions, req_of_token, cu_seqlens, state_slots, prev_state)
    T = tokens.numel()
    V, H = table.shape
    _need(table.is_contiguous() and pairs.is_contiguous() and pairs.dtype == table.dtype and pairs.dim() == 2
          and pairs.shape[1] == H and pairs.shape[0] >= 2, "embedding_pairs: tables are contiguous [rows, H] of one type")
    _need(positions.numel() == T and req_of_token.numel() == T, "embedding_pairs: one position and request per token")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, H),
          f"embedding_pairs: the output is float32 [{T}, {H}]")
    _need(abs(int(mul_prev)) < (1 << 31) and abs(int(mul_cur)) < (1 << 31), "embedding_pairs: multipliers fit 32 bits")
    _check(_lib().tl_embedding_pairs(_ptr(tokens), _ptr(positions), _ptr(req_of_token), _ptr(cu_seqlens),
                                     _ptr(state_slots), _ptr(prev_state), _ptr(table), _ptr(pairs), _ptr(out), c_int(T),
                                     c_int(H), c_int(V), c_int(pairs.shape[0] - 1), c_int(int(mul_prev)),
                                     c_int(int(mul_cur)), c_float(scale), c_int(_dt(table)), _stream()), "embedding_pairs")
    return out


# ------------------------------------------- the general step between the q/k/v product and the attention kernel
ATTN_PREPARE_MAX_DIM = 256      # numbers a unit (one map of one head) may have, and the padded head size D


def attn_prepare(p: torch.Tensor, bias: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], positions: torch.Tensor,
                 cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor],
                 q_out: torch.Tensor, k_caches, v_cache: Optional[torch.Tensor], heads: int, kv_heads: int, maps: int,
                 dim: int, vdim: int, v_off: int, rot: int = 0, pairing: str = "half", whole_norm: bool = False,
                 unit_norm: bool = False, eps: float = 1e-6, q_temp=None) -> None:
    """From the float32 product p [T, >= v_off + kv_heads * vdim] = [q: heads * maps units of dim | k: kv_heads * maps
    units | v: kv_heads heads of vdim, from column v_off]: bias added (float32 over [q | k | v]), an RMS norm over ALL of
    a token's q numbers (and all of its k numbers) with weights norm_w (float32 over [q | k], `whole_norm`), the first
    `rot` dims of every unit rotated by the token's position, every unit divided by its own root mean square
    (`unit_norm`), queries times 1 + coef * ln(floor((pos + 1) / every) + 1) (`q_temp` = (coef, every)).  Queries leave
    as q_out [maps, T, heads * D] rounded to the engine's type, keys of map m go to k_caches[m] and values to v_cache
    (pages [blocks, kv_heads, block, D]) at the tokens' slots; D is q_out's head size, what lies beyond dim or vdim is
    written as zeros.  slot_mapping None (or a negative slot) stores nothing."""
    k_caches = tuple(k_caches) if k_caches is not None else ()
    _dev(p, bias, norm_w, positions, cos, sin, slot_mapping, q_out, v_cache, *k_caches)
    _rows_2d(p, "attn_prepare input")
    T = p.shape[0]
    _need(p.dtype == torch.float32, "attn_prepare: the product is float32")
    _need(maps in (1, 2) and heads > 0 and kv_heads > 0 and heads % kv_heads == 0, "attn_prepare: one or two maps, heads a "
          "multiple of kv heads")
    _need(q_out.dim() == 3 and q_out.is_contiguous() and q_out.shape[0] == maps and q_out.shape[1] == T
          and q_out.shape[2] % heads == 0, "attn_prepare: queries leave as contiguous [maps, T, heads * D]")
    D = q_out.shape[2] // heads
    _need(0 < dim <= D and 0 < vdim <= D and D <= ATTN_PREPARE_MAX_DIM, f"attn_prepare: dim and vdim within D = {D} <= "
          f"{ATTN_PREPARE_MAX_DIM}")
    q_size, k_size, v_size = heads * maps * dim, kv_heads * maps * dim, kv_heads * vdim
    _need(v_off >= q_size + k_size and v_off + v_size <= p.shape[1], "attn_prepare: columns do not fit")
    if bias is not None:
        _f32_vec(bias, q_size + k_size + v_size, "attn_prepare bias")
    if whole_norm:
        _need(norm_w is not None, "attn_prepare: the norm over the whole projection needs its weights")
        _f32_vec(norm_w, q_size + k_size, "attn_prepare norm weights")
    _need(pairing in ROPE_PAIRINGS, f"attn_prepare: rotary pairing {pairing!r} is not built")
    _need(rot % 2 == 0 and 0 <= rot <= dim, "attn_prepare: the rotated dims are even and within dim")
    _i32(positions)
    _need(positions.numel() == T, "attn_prepare: one position per row")
    if rot:
        _need(cos is not None and sin is not None and cos.dtype == sin.dtype == torch.float32 and cos.is_contiguous()
              and sin.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rot // 2,
              "attn_prepare: angle tables are float32 [positions, rot / 2]")
    block_size = 1
    if slot_mapping is not None:
        _i32(slot_mapping)
        _need(slot_mapping.numel() == T and len(k_caches) == maps and v_cache is not None,
              "attn_prepare: one slot per row, a key cache per map and a value cache")
        for c in k_caches + (v_cache,):
            _need(c.dtype == q_out.dtype and c.dim() == 4 and c.is_contiguous() and c.shape[1] == kv_heads
                  and c.shape[3] == D and c.shape == v_cache.shape, "attn_prepare: caches are contiguous "
                  "[blocks, kv_heads, block, D] of the queries' type")
        block_size = v_cache.shape[2]
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 0)
    _need(every >= 0, "attn_prepare: the temperature's step is positive")
    store = slot_mapping is not None
    _check(_lib().tl_attn_prepare(_ptr(p), c_int64(p.stride(0)), _ptr(bias), _ptr(norm_w), _ptr(positions), _ptr(cos),
                                  _ptr(sin), _ptr(slot_mapping), _ptr(q_out), c_int64(q_out.stride(1)),
                                  c_int64(q_out.stride(0)), _ptr(k_caches[0] if store else None),
                                  _ptr(k_caches[1] if store and maps == 2 else None), _ptr(v_cache if store else None),
                                  c_int(T), c_int(heads), c_int(kv_heads), c_int(maps), c_int(dim), c_int(vdim), c_int(D),
                                  c_int(v_off), c_int(rot), c_int(ROPE_PAIRINGS.index(pairing)),
                                  c_int(1 if whole_norm else 0), c_int(1 if unit_norm else 0), c_float(eps), c_float(coef),
                                  c_int(every), c_int(block_size), c_int(_dt(q_out)), _stream()), "attn_prepare")


ATTN_GATES = {None: 0, "head": 1, "element": 2}


def attn_finish(a0: torch.Tensor, a1: Optional[torch.Tensor], gate: Optional[torch.Tensor], z: torch.Tensor, heads: int,
                vdim: int, lam: float = 0.0, sub_norm: bool = False, eps: float = 1e-6, scale: float = 1.0,
                gate_kind: Optional[str] = None, tail: int = 0) -> torch.Tensor:
    """Behind the attention kernel: of every head's D numbers the first vdim, o = a0 - lam * a1 (a1 None: o = a0),
    divided by the head's root mean square (`sub_norm`), times `scale`, times sigmoid(gate) (float32, one number per
    token and head for "head", per element [T, heads * vdim] for "element"); a0 and a1 are float32 or of z's type;
    z[t] = the heads side by side, then
    `tail` columns 1, 0, 0, ... (the one meets a bias kept as one more column of the next product's weight)."""
    _dev(a0, a1, gate, z)
    _rows_2d(a0, "attn_finish input")
    _rows_2d(z, "attn_finish output")
    T = a0.shape[0]
    _need(a0.shape[1] % heads == 0, "attn_finish: the input is [T, heads * D]")
    D = a0.shape[1] // heads
    _need(0 < vdim <= D and vdim <= ATTN_PREPARE_MAX_DIM and a0.dtype in (z.dtype, torch.float32) and z.shape[0] == T
          and z.shape[1] == heads * vdim + tail and 0 <= tail <= 64, "attn_finish: z is [T, heads * vdim + tail]; the "
          "input has its type or is float32")
    if a1 is not None:
        _need(a1.dtype == a0.dtype and a1.shape == a0.shape and a1.stride() == a0.stride(),
              "attn_finish: the second map has the first one's layout")
    _need(gate_kind in ATTN_GATES, f"attn_finish: unknown gate {gate_kind!r}")
    if gate_kind is not None:
        _rows_2d(gate, "attn_finish gate")
        _need(gate.dtype == torch.float32 and gate.shape[0] == T
              and gate.shape[1] == (heads if gate_kind == "head" else heads * vdim), "attn_finish: the gate is float32, "
              "one number per head or per element")
    _check(_lib().tl_attn_finish(_ptr(a0), _ptr(a1), c_int64(a0.stride(0)), _ptr(gate if gate_kind else None),
                                 c_int64(gate.stride(0) if gate_kind else 0), _ptr(z), c_int64(z.stride(0)), c_int(T),
                                 c_int(heads), c_int(vdim), c_int(D), c_float(lam), c_int(1 if sub_norm else 0),
                                 c_float(eps), c_float(scale), c_int(ATTN_GATES[gate_kind]), c_int(tail), c_int(_dt(a0)),
                                 c_int(_dt(z)), _stream()), "attn_finish")
    return z


def stream_join(a: torch.Tensor, b: torch.Tensor, vec: Optional[torch.Tensor], operand: torch.Tensor,
                init: torch.Tensor) -> None:
    """operand[t] = [a[t] | b[t]] in operand's element type (a, b float32 [T, W]); init[t] = vec (float32 [W]; zeros
    without one): the row a product over `operand` then adds its result to."""
    _dev(a, b, vec, operand, init)
    T, W = a.shape
    for t in (a, b, init):
        _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (T, W),
              "stream_join: streams and the initial rows are contiguous float32 [T, W]")
    _need(operand.is_contiguous() and tuple(operand.shape) == (T, 2 * W), "stream_join: the operand is contiguous [T, 2W]")
    if vec is not None:
        _f32_vec(vec, W, "stream_join vector")
    _check(_lib().tl_stream_join(_ptr(a), _ptr(b), _ptr(vec), _ptr(operand), _ptr(init), c_int(T), c_int(W),
                                 c_int(_dt(operand)), _stream()), "stream_join")
