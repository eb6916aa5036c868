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
def embedding(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[tokens[t], :] as float32."""
    _dev(tokens, table, out)
    T = tokens.numel()
    V, H = table.shape
    if not (tokens.dtype == torch.int32 and tokens.is_contiguous()):
        _fail("tokens must be contiguous int32")
    if not (table.is_contiguous()):
        _fail("embedding table must be contiguous")
    if not (out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, H)):
        _fail(f"embedding output must be float32 [{T}, {H}]")
    _check(_lib().tl_embedding(_ptr(tokens), _ptr(table), _ptr(out), c_int(T), c_int(H), c_int(V),
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


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, j] = silu(gate_up[t, j]) * gate_up[t, I + j]."""
    _dev(gate_up, out)
    T, I2 = gate_up.shape
    if not (I2 % 2 == 0 and gate_up.is_contiguous()):
        _fail("gate_up must be contiguous [T, 2I]")
    if not (out.dtype == gate_up.dtype and out.is_contiguous() and tuple(out.shape) == (T, I2 // 2)):
        _fail("silu_mul output must be contiguous [T, I] of the input's type")
    _check(_lib().tl_silu_mul(_ptr(gate_up), _ptr(out), c_int(T), c_int(I2 // 2), c_int(_dt(gate_up)),
                              _stream()), "silu_mul")
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


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_tables: torch.Tensor, req_of_token: torch.Tensor, positions: torch.Tensor,
                    out: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                    window: int = 0) -> torch.Tensor:
    """Causal attention of every row of q (at its absolute position) over its
    request's cached keys 0..position (the last `window` of them if window > 0)."""
    _dev(q, k_cache, v_cache, block_tables, req_of_token, positions, out)
    _rows_2d(q, "q")
    _rows_2d(out, "attention output")
    T = q.shape[0]
    if not (q.shape[1] == num_heads * head_dim and tuple(out.shape) == (T, num_heads * head_dim)):
        _fail("q and the attention output must be [T, heads * head_dim]")
    if not (q.dtype == k_cache.dtype == v_cache.dtype == out.dtype):
        _fail("q, caches and output must share an element type")
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
        c_float(scale), c_int(window), c_int(_dt(q)), _stream()), "paged_attention")
    return out


F32_CHUNK_KEYS = 256     # keys per chunk of the float32 attention kernel's fixed merge tree


def attention_f32_supported(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Sizes the float32 matrix-core attention kernel takes; everything else goes to `paged_attention`."""
    return (dtype == torch.float32 and head_dim % 16 == 0 and head_dim <= 128 and num_kv_heads > 0
            and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16)


def attention_f32(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                  tiles, positions: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                  head_dim: int, scale: float, window: int = 0, n_chunks: int = 1,
                  scratch: Optional[torch.Tensor] = None) -> torch.Tensor:
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
        c_int(num_kv_heads), c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale), c_int(window),
        c_int(n_chunks), _stream()), "attention_f32")
    return out


def flash_attention_supported(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Sizes the MFMA attention kernel takes; everything else goes to `paged_attention`."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 128 and num_kv_heads > 0
            and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16)


def flash_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    tiles, positions: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                    head_dim: int, scale: float, window: int = 0, n_splits: int = 1,
                    scratch: Optional[torch.Tensor] = None, fused_rope=None, static_scratch: bool = False) -> torch.Tensor:
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
    if not (q.dtype == k_cache.dtype == v_cache.dtype == out.dtype):
        _fail("q, caches and output must share an element type")
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
            c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale), c_int(window), c_int(n_splits), _ptr(cos),
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
        c_int(window), c_int(n_splits), _ptr(cos), _ptr(sin), c_int(1 if fused_rope is not None else 0),
        _stream()), "flash_attention")
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
                  scratch: Optional[torch.Tensor] = None) -> torch.Tensor:
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
    if not (q.dtype == k_cache.dtype == v_cache.dtype == out.dtype):
        _fail("q, caches and output must share an element type")
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
        _ptr(out, 8), c_int64(out.stride(0)), _ptr(part_o, 16), _ptr(part_ml), c_int(n_tiles), c_int(T),
        c_int(num_heads), c_int(num_kv_heads),
        c_int(head_dim), c_int(k_cache.shape[2]), c_float(scale), c_int(window), c_int(tile_waves), c_int(n_splits),
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
