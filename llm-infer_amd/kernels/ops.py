"""Python face of the HIP kernels: argument checks on the host, then one launch
on torch's current stream.  Every shape that a kernel and its grid assume is
checked here before the launch; nothing falls back to another implementation.
"""
from __future__ import annotations

import ctypes
import functools
from ctypes import c_float, c_int, c_int64, c_uint64, c_void_p

import torch

from . import build
from ..tensor import Tensor

PAGE = 64
DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
EPI_STORE, EPI_ADD, EPI_SWIGLU, EPI_ROPE, EPI_GEGLU = 0, 1, 2, 3, 4
GATED = (EPI_SWIGLU, EPI_GEGLU)             # gate and up rows interleaved in W, act(gate) * up written
_STATUS = {1: "bad argument", 2: "unsupported size or alignment", 3: "HIP launch error"}


class KernelError(RuntimeError):
    pass


def _ptr(t):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current HIP stream of the current device (looked up for every launch: a graph is
    recorded on a stream of its own)."""
    if _raw_stream is not None:
        return c_void_p(_raw_stream(torch.cuda.current_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int, what: str):
    if rc != 0:
        raise KernelError(f"{what}: {_STATUS.get(rc, rc)}")


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*tensors):
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operands must lie on the GPU")
            _need(t.is_contiguous(), "kernel operands must be contiguous")


_core = None


def core():
    global _core
    if _core is None:
        lib = build.core_library()
        lib.li_uniform01.restype = c_float
        lib.li_uniform01.argtypes = [c_uint64, c_uint64]
        _core = lib
    return _core


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """x[t] = float32(table[tokens[t]])"""
    _dev(table, tokens)
    _need(tokens.dtype == torch.int32 and tokens.dim() == 1, "tokens: int32 [T]")
    _need(table.dim() == 2 and table.dtype in DT, "table: [V, d] float")
    n, (vocab, d) = tokens.numel(), table.shape
    if out is None:
        out = torch.empty((n, d), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (n, d), "out: float32 [T, d]")
    _drop_row_stats(out)
    _check(core().li_embed(_ptr(table), DT[table.dtype], _ptr(tokens), _ptr(out), n, d, vocab, _stream()), "embed")
    return out


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype, rows: torch.Tensor | None = None,
            n_rows: int | None = None) -> torch.Tensor:
    """out[r] = x[rows[r]] / sqrt(mean(x^2) + eps) * w, float32 inside."""
    _dev(x, w, rows)
    _need(x.dtype == torch.float32 and x.dim() == 2, "x: float32 [T, d]")
    _need(w.dtype == torch.float32 and w.shape == (x.shape[1],), "norm weight: float32 [d]")
    if rows is not None:
        _need(rows.dtype == torch.int32, "rows: int32")
        n = rows.numel() if n_rows is None else n_rows
    else:
        n = x.shape[0]
    out = torch.empty((n, x.shape[1]), dtype=out_dtype, device=x.device)
    # for the few rows of a decode step in float16: a power of two near 1 / (8 rms) of each row, for the product
    # that adds into these rows next and hands them on in 16 bits (see LazyNorm)
    row_scale = None
    if rows is None and n <= 16 and out_dtype == torch.float16:
        row_scale = torch.empty((16,), dtype=torch.float32, device=x.device)
    _check(core().li_rmsnorm(_ptr(x), _ptr(w), _ptr(rows), _ptr(out), DT[out_dtype], n, x.shape[1],
                             c_float(eps), _ptr(row_scale), _stream()), "rmsnorm")
    if row_scale is not None:
        x._li_row_scale = row_scale
    return out


class _RowsOut(ctypes.Structure):
    _fields_ = [("ss", c_void_p), ("xw", c_void_p), ("w", c_void_p), ("scale", c_float), ("row_scale", c_void_p)]


class _RowScale(ctypes.Structure):
    _fields_ = [("ss", c_void_p), ("P", c_int), ("eps", c_float), ("inv_scale", c_float), ("row_scale", c_void_p),
                ("next_scale", c_void_p)]


class LazyNorm:
    """A norm whose last step has not been taken yet, for the few rows of a decode step.  The product that
    last added into the float32 rows ``x`` also left ``xw`` = x * weight * scale in the 16-bit type and
    the rows' sums of squares as partial sums ``ss`` [P, 16]; the product that reads the norm takes
    ``xw`` as its X and multiplies its sums by 1 / (scale * rms).  ``linear`` does that where its kernel
    can (up to 16 rows against a tiled weight); everywhere else ``tensor()`` runs the norm kernel.

    ``scale`` keeps x * weight inside float16's range (bfloat16 has float32's and takes 1).  A fixed factor
    cannot: a residual stream of the order of 0.01 under norm weights of 0.02 would fall below float16's
    normal numbers, one of the order of 1000 above its largest.  So in float16 each row has a power of two of its
    own, ``row_scales`` [16]: near 1 / (8 rms) of the row when a norm was last taken of it (by the norm kernel, or
    by the product that finished the norm before this one, which leaves the next one's scales on the residual
    tensor as ``_li_row_scale``); rows about which nothing is known take the fixed ``scale``."""

    def __init__(self, x, weight, eps, dtype, xw, ss, scale, row_scales=None):
        self.x, self.weight, self.eps, self.dtype = x, weight, float(eps), dtype
        self.xw, self.ss, self.scale, self.row_scales = xw, ss, float(scale), row_scales
        self.shape, self.device = x.shape, x.device

    def dim(self):
        return 2

    def tensor(self) -> torch.Tensor:
        return rmsnorm(self.x, self.weight, self.eps, self.dtype)


def expect_norm(x: torch.Tensor, weight, eps: float | None = None) -> None:
    """Says which RMS norm (weight float32 [width], or None; its eps) will read the rows of ``x`` next.
    A product that adds into ``x`` may then prepare that norm (``LazyNorm``) or take it whole
    (``prepared_rmsnorm``).  Only a hint: a norm with another weight or eps, or rows that something else
    has written to since, get the norm kernel."""
    x._li_next_norm = weight
    x._li_next_eps = eps


def _drop_row_stats(x) -> None:
    """Whatever a kernel of this library is about to write into ``x``, what was prepared for a norm of its rows
    is void: on ``x`` itself and, if ``x`` is a view (``out=rows[:n]``), on the tensor it is a view of, whose
    ``_version`` a write through ctypes does not move."""
    while x is not None:
        if getattr(x, "_li_rows", None) is not None:
            x._li_rows = None
        if getattr(x, "_li_normed", None) is not None:
            x._li_normed = None
        x = getattr(x, "_base", None)


def prepared_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype):
    """The norm of all rows of ``x`` if the product that last added into ``x`` has taken it already (with K
    split, the kernel that adds the partial sums has the finished rows in its hands): same weight tensor,
    same eps and type, and nothing has written to ``x`` since; else None."""
    rec = getattr(x, "_li_normed", None)
    if rec is None:
        return None
    normed, weight, rec_eps, version = rec
    if weight is not w or rec_eps != eps or version != x._version or normed.dtype != out_dtype or normed.shape != x.shape:
        return None
    return normed


def lazy_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype):
    """A ``LazyNorm`` of ``x`` if the product that last added into ``x`` prepared this very norm (same
    weight tensor, same 16-bit type) and nothing has written to ``x`` since (torch counts its own
    in-place writes in ``_version``; every kernel of this library that writes into a tensor drops the
    record first); else None."""
    rec = getattr(x, "_li_rows", None)
    if rec is None:
        return None
    xw, ss, scale, weight, version, row_scales = rec
    if weight is not w or version != x._version or xw.dtype != out_dtype or xw.shape != x.shape:
        return None
    return LazyNorm(x, w, eps, out_dtype, xw, ss, scale, row_scales)


class _NormAfter(ctypes.Structure):
    _fields_ = [("w", c_void_p), ("out", c_void_p), ("out_dt", c_int), ("eps", c_float)]


class _RopeStore(ctypes.Structure):
    _fields_ = [("inv_freq", c_void_p), ("cos_sin", c_void_p), ("pos", c_void_p), ("tok_slot", c_void_p), ("page_table", c_void_p),
                ("q_out", c_void_p), ("k_pages", c_void_p), ("v_pages", c_void_p), ("page_stride", c_int64),
                ("rotary_dim", c_int), ("H", c_int), ("K", c_int), ("hd", c_int), ("max_pages", c_int),
                ("dt", c_int)]


def is_tiled(w) -> bool:
    """True for a ``Tensor`` in tiled layout: a 16-bit matrix [n, k] kept in the order in which the matrix
    cores take it (csrc/gemm.hip, "Tiled weights"; rows padded to a multiple of 16)."""
    return getattr(w, "layout", "rows") == "tiled"


def matrix_shape(w) -> tuple:
    """(n, k) of a matrix operand, whatever its layout."""
    return tuple(w.logical) if is_tiled(w) else tuple(w.shape)


def can_tile(w: torch.Tensor) -> bool:
    return not is_tiled(w) and w.dim() == 2 and w.dtype in (torch.float16, torch.bfloat16) and w.shape[1] % 32 == 0 and w.is_cuda


def prepare_weight(w: torch.Tensor):
    """The form in which a linear layer keeps its matrix: tiled where the kernels can use that
    (16-bit, K a multiple of 32), else as it is."""
    if can_tile(w):
        return tile_weight(w)
    return w if isinstance(w, Tensor) else Tensor.wrap(w)


_ws_cache: dict = {}
_ws_retired: list = []


def _workspace(n_floats: int, device) -> torch.Tensor:
    """Scratch for split-K partial sums, one per device and stream.  A workspace that has become
    too small is kept alive beside its larger successor: a captured graph may still write to it."""
    key = (device, _stream().value)
    ws = _ws_cache.get(key)
    if ws is None or ws.numel() < n_floats:
        if ws is not None:
            _ws_retired.append(ws)
        ws = torch.empty(max(n_floats, 1 << 22, 2 * (ws.numel() if ws is not None else 0)),
                         dtype=torch.float32, device=device)
        _ws_cache[key] = ws
    return ws


def linear(x: torch.Tensor, w, mode: int = EPI_STORE, out: torch.Tensor | None = None,
           out_dtype=None, force: str | None = None, _rope=None) -> torch.Tensor:
    """C = X W^T with the epilogue ``mode``: store, add into ``out`` (float32), or act(gate) * up over
    interleaved gate/up rows of W (C has N/2 columns; EPI_SWIGLU: silu, EPI_GEGLU: gelu).  ``force`` picks a kernel for tests."""
    tiled = is_tiled(w)
    wd = w
    w_shape = matrix_shape(w)
    _drop_row_stats(out)                   # whatever this call writes into `out`, an older record is void
    lazy = None
    if isinstance(x, LazyNorm):
        # the kernel that finishes the norm: gemv_tiled, for up to 16 rows
        if tiled and force is None and x.dtype == w.dtype and x.shape[0] <= 16 and wd.data_ptr() % 16 == 0:
            lazy = x
            x = lazy.xw
        else:
            x = x.tensor()
    _dev(x, wd, out)
    _need(x.dim() == 2 and len(w_shape) == 2 and x.shape[1] == w_shape[1], f"linear: x {tuple(x.shape)} w {w_shape}")
    m, k = x.shape
    n = w_shape[0]
    n_out = n // 2 if mode in GATED else n
    if mode == EPI_ADD:
        _need(out is not None and out.dtype == torch.float32, "add epilogue needs a float32 output")
    rs = ctypes.byref(_rope) if _rope is not None else None
    if mode == EPI_ROPE:
        _need(_rope is not None, "the rotation epilogue needs its arguments (use linear_rope_store)")
    elif out is None:
        out = torch.empty((m, n_out), dtype=out_dtype or x.dtype, device=x.device)
    if mode != EPI_ROPE:
        _need(out.shape == (m, n_out), f"linear: out {tuple(out.shape)}, expected {(m, n_out)}")
    out_dt = DT[out.dtype] if out is not None else 0
    if mode in GATED:
        _need(n % 2 == 0, "a gated epilogue needs an even number of rows of W")
    if m == 0:
        return out
    lib = core()
    same16 = x.dtype == w.dtype and x.dtype in (torch.float16, torch.bfloat16)
    fast_ok = same16 and k % 8 == 0 and x.data_ptr() % 16 == 0 and wd.data_ptr() % 16 == 0
    kind = force or ("fma" if not fast_ok else ("gemv_mfma" if m <= 16 else ("big" if m > 32 else "mfma")))
    if tiled:
        _need(fast_ok and kind != "fma", "a tiled weight needs 16-bit activations of its dtype")
        # up to 16 rows (32 for a small matrix) every wave fetches the rows of X itself; beyond that
        # the tiled GEMM is faster
        # 9 to 16 rows against a wide matrix with an activation (gate and up): the tiled GEMM's tile of 64 rows of X
        # fetches the rows of X once per 112 rows of W, gemv_tiled once per 16 or 32 (measured at 16 rows and
        # 28,672 x 4,096: 44.6 against 51.7 us, at 12 rows 44.2 against 48.7, at 8 rows 44.0 against 43.5)
        wide = (force is None and 8 < m <= 16 and mode in GATED and n * k >= (1 << 26) and m * k * 2 < (1 << 32)
                and _wreg_plan(m, n, k) == (2, 1))
        if not wide and (kind == "gemv_mfma" or (force is None and (m <= 16 or (m <= 32 and n * k <= (1 << 25))))):
            ro = rsc = None
            # 9 to 16 rows with the residual sum against a matrix with a long K (down): gemm_rows, one tile of W a
            # workgroup (measured at 16 rows and 4,096 x 14,336: 25.5 against 30.3 us, at 12 rows 24.4 against 27.1, at 8
            # rows the same; 4,096 x 11,008 at 16 rows 20.9 against 25.9, 2,048 x 8,192 10.2 against 11.9; against
            # 4,096 x 4,096 gemv_tiled is as fast)
            tall = (force is None and 8 < m <= 16 and mode == EPI_ADD and lazy is None and k >= 8192 and n >= 2048 and n % 16 == 0
                    and x.stride(0) % 8 == 0 and x.stride(1) == 1)
            nxt = getattr(out, "_li_next_norm", None) if mode == EPI_ADD else None
            if (nxt is not None and m <= 16 and n % 32 == 0 and out.data_ptr() % 16 == 0 and nxt.dtype == torch.float32
                    and nxt.shape == (n,) and nxt.is_cuda and nxt.data_ptr() % 16 == 0):
                # the rows of `out` are about to be complete rows of a residual stream that this norm reads
                # next: leave x * weight in 16 bits and the sums of squares for the product behind the norm
                blocks = n // 16 if tall else lib.li_gemv_tiled_blocks(m, n, k, 0, 0)
                ss = torch.empty((blocks, 16), dtype=torch.float32, device=x.device)
                xw = torch.empty((m, n), dtype=x.dtype, device=x.device)
                scale = 0.125 if x.dtype == torch.float16 else 1.0        # x * w stays inside float16's range
                row_scales = getattr(out, "_li_row_scale", None) if x.dtype == torch.float16 else None
                ro = _RowsOut(ss.data_ptr(), xw.data_ptr(), nxt.data_ptr(), scale,
                              row_scales.data_ptr() if row_scales is not None else None)
            if lazy is not None:
                rsc = _finish_norm(lazy, x)
            if tall:
                _check(lib.li_gemm_rows(_ptr(x), _ptr(wd), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k, x.stride(0), 1, 4,
                                        rs, ctypes.byref(ro) if ro is not None else None, _stream()), "gemm_rows")
            else:
                _check(lib.li_gemv_tiled(_ptr(x), _ptr(wd), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k, 0, 0, rs,
                                         ctypes.byref(ro) if ro is not None else None,
                                         ctypes.byref(rsc) if rsc is not None else None, _stream()), "gemv_tiled")
            if ro is not None:
                out._li_rows = (xw, ss, scale, nxt, out._version, row_scales)
            return out
        _need(lazy is None or wide, "a norm is finished by gemv_tiled, or by gemm_wreg for gate and up")
        if force is None and m <= 128 and not wide:
            # 17 to 128 rows: all of K in one workgroup and every epilogue the product's own (gemm_rows), where
            # that is estimated faster than the tiled GEMM with K split and its second kernel
            norm_rides = mode == EPI_ADD and getattr(out, "_li_next_norm", None) is not None
            nt = _rows_plan(m, n, k, norm_rides)
            if nt:
                kind = f"rows:{nt}"
        if force is None and kind != "fma" and not kind.startswith("rows") and m * k * 2 < (1 << 32):
            kind = "wreg"
    if kind.startswith("rows"):                                # "rows[:<tiles of W a workgroup>]" (a test's choice)
        _need(tiled and fast_ok and m <= 128, "gemm_rows: a tiled weight, at most 128 rows of X")
        parts = kind.split(":")
        _check(lib.li_gemm_rows(_ptr(x), _ptr(wd), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k, x.stride(0),
                                int(parts[1]) if len(parts) > 1 else 0, int(parts[2]) if len(parts) > 2 else 0,
                                rs, None, _stream()), "gemm_rows")
        return out
    if kind.startswith("wreg"):                                # "wreg[:<tile>[:<splits>[:<few rows>]]]" (a test's choice)
        _need(tiled and fast_ok and m * k * 2 < (1 << 32), "gemm_wreg: a tiled weight, X below 4 GiB")
        parts = kind.split(":")
        tile, splits = _wreg_plan(m, n, k)
        # up to 64 rows against the narrowest tile: a tile of 64 rows of X (none fetched or multiplied that is not
        # there) with W four steps ahead (measured at 64 rows: gate/up 53.9 -> 46.0 us, down 35.9 -> 35.0 and 29.5
        # with K in 8; the same depth with 128 rows of X leaves room for one workgroup a CU and gained nothing in a
        # decode step at batch 128: 11.41 and 11.47 ms).  65 to 128 rows: W three steps ahead, which still lets two
        # workgroups share a CU (by itself gate/up at 96 rows 58.9 -> 52.1 us, at 128 rows 60.6 -> 54.1; in a decode
        # step at batch 96 9.68 -> 9.55 ms, at batch 128 11.52 -> 11.46; from 192 rows on it gains nothing)
        few_rows = (1 if m <= 64 else (3 if m <= 128 else 0)) if tile == 2 else 0
        wg_blocks = _wreg_blocks(tile, splits, m, n)
        if len(parts) > 1:                                     # "wreg:<tile>:<splits>:<few rows>:<blocks of W>"
            tile, splits = int(parts[1]), int(parts[2]) if len(parts) > 2 else 1
            few_rows = int(parts[3]) if len(parts) > 3 else 0
            wg_blocks = int(parts[4]) if len(parts) > 4 else 0
        ws = _workspace(splits * m * n, x.device) if splits > 1 else None
        # with K split, the kernel that adds the partial sums to the residual also takes the norm that reads
        # the finished rows next, if the block has said which one that is
        na = normed = None
        nxt, eps = getattr(out, "_li_next_norm", None), getattr(out, "_li_next_eps", None)
        k_split = -(-(-(-k // splits)) // 32) * 32
        if (mode == EPI_ADD and -(-k // k_split) > 1 and nxt is not None and eps is not None and n % 4 == 0 and n <= 8192
                and nxt.dtype == torch.float32 and nxt.shape == (n,) and nxt.is_cuda
                and (ws.data_ptr() | out.data_ptr() | nxt.data_ptr()) % 16 == 0):
            normed = torch.empty((m, n), dtype=x.dtype, device=x.device)
            na = _NormAfter(nxt.data_ptr(), normed.data_ptr(), DT[x.dtype], eps)
        rsc = _finish_norm(lazy, x) if lazy is not None else None
        _check(lib.li_gemm_wreg(_ptr(x), _ptr(wd), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k, tile, splits,
                                _ptr(ws), rs, ctypes.byref(na) if na is not None else None, few_rows, wg_blocks,
                                ctypes.byref(rsc) if rsc is not None else None, _stream()),
               "gemm_wreg")
        if na is not None:
            out._li_normed = (normed, nxt, eps, out._version)
        return out
    if kind == "fma":
        _check(lib.li_gemm_fma(_ptr(x), DT[x.dtype], _ptr(w), DT[w.dtype], _ptr(out), out_dt, mode,
                               m, n, k, rs, _stream()), "gemm_fma")
    elif kind == "gemv_mfma":
        _need(fast_ok and m <= 16, "gemv_mfma: 16-bit operands, K a multiple of 8, at most 16 rows")
        _check(lib.li_gemv_mfma(_ptr(x), _ptr(w), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k, rs, _stream()),
               "gemv_mfma")
    elif kind.startswith("big"):
        _need(fast_ok, "gemm_big: 16-bit operands and K a multiple of 8")
        parts = kind.split(":")
        tile = int(parts[1]) if len(parts) > 1 else _big_tile(m, n)
        groups = -(-m // 128) * -(-n // (256 if tile else 128))
        splits = int(parts[2]) if len(parts) > 2 else (1 if groups >= 192 else max(1, min(384 // groups, k // 512, 16)))
        ws = _workspace(splits * m * n, x.device) if splits > 1 else None
        _check(lib.li_gemm_big(_ptr(x), _ptr(wd), int(tiled), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k, tile,
                               splits, _ptr(ws), rs, _stream()), "gemm_big")
    else:
        _need(fast_ok, "gemm_mfma: 16-bit operands and K a multiple of 8")
        tile = 0 if m > 64 else (1 if m > 32 else 2)
        bm = (128, 64, 32)[tile]
        blocks = ((n + 127) // 128) * ((m + bm - 1) // bm)
        splits = 1
        if blocks < 256:
            splits = max(1, min(512 // blocks, k // 256, 16))
        if kind.startswith("mfma:"):                       # "mfma:<tile>:<splits>" for tests
            _, t_, s_ = kind.split(":")
            tile, splits = int(t_), int(s_)
        ws = _workspace(splits * m * n, x.device) if splits > 1 else None
        _check(lib.li_gemm_mfma(_ptr(x), _ptr(wd), int(tiled), DT[x.dtype], _ptr(out), out_dt, mode, m, n, k,
                                tile, splits, _ptr(ws), rs, _stream()), "gemm_mfma")
    return out


def _finish_norm(lazy: "LazyNorm", x: torch.Tensor) -> _RowScale:
    """What the product that reads an unfinished norm needs of it.  In float16 its kernel also leaves the scales
    for the product that adds into these rows next."""
    nxt_scale = torch.empty((16,), dtype=torch.float32, device=x.device) if x.dtype == torch.float16 else None
    rsc = _RowScale(lazy.ss.data_ptr(), lazy.ss.shape[0], lazy.eps, 1.0 / lazy.scale,
                    lazy.row_scales.data_ptr() if lazy.row_scales is not None else None,
                    nxt_scale.data_ptr() if nxt_scale is not None else None)
    if nxt_scale is not None:
        lazy.x._li_row_scale = nxt_scale
    return rsc


# rows of W x rows of X of a workgroup of gemm_wreg
_WREG_TILES = {0: (256, 128), 1: (192, 128), 2: (128, 128)}
# Microseconds that one round of workgroups takes, measured on MI355X, as (a, c): a K / 4096 + c.  Entry i
# is a round with i + 1 workgroups on every CU: two share a CU (three of the narrowest tile), and those of a
# last round that is less full run at the shorter time.
_WREG_ROUND_US = {0: ((53.0, 9.0), (103.0, 5.0)), 1: ((35.0, 13.0), (73.0, 12.0)),
                  2: ((31.4, 3.4), (57.1, 3.8), (89.0, 0.0))}


def _wreg_blocks(tile: int, splits: int, m: int, n: int) -> int:
    """Blocks of 16 rows of W that a workgroup of gemm_wreg takes: all of its tile's, or, for a product of up to
    64 rows against the narrowest tile (one workgroup a CU at a time, one tile of X), as few as make the rounds of
    256 workgroups times the blocks of each the least (28,672 rows of W: 224 workgroups of 8 blocks leave 32 CUs
    idle, 256 workgroups of 7 none; measured at 64 rows: 49.3 -> 46.8 us, and 22,016 rows of W with 6 blocks
    44.8 -> 37.5).  With the 128-row tile of X the same measured no gain, and where K is split the splits are what
    fills the CUs."""
    full = _WREG_TILES[tile][0] // 16
    if tile != 2 or m > 64 or splits > 1:
        return full
    blocks16 = -(-n // 16)
    return min(range(full, full // 2, -1), key=lambda b: -(-(-(-blocks16 // b) * splits) // 256) * b)


def _wreg_cost(tile: int, splits: int, m: int, n: int, k: int) -> float:
    """Estimated microseconds of one gemm_wreg launch (and its split-K reduction): rounds of workgroups
    at the measured time of a round, not below the time to stream W once; a fixed cost for the launch,
    the first tiles and the epilogue; the partial sums written and read back."""
    bn, bm = _WREG_TILES[tile]
    times = _WREG_ROUND_US[tile]
    wg_blocks = _wreg_blocks(tile, splits, m, n)
    groups = -(-m // bm) * -(-(-(-n // 16)) // wg_blocks) * splits
    full, rest = divmod(groups, 256 * len(times))
    k_split = -(-(-(-k // splits)) // 32) * 32
    us = 0.0
    for count, (a, c) in ((full, times[-1]), (1 if rest else 0, times[-(-rest // 256) - 1])):
        us += count * (a * wg_blocks * 16 / bn * k_split / 4096 + c)
    # W streams at 5.5 TB/s when every CU has a workgroup, at less with fewer workgroups
    main = max(us, n * k * 2 / (5.5e6 * min(1.0, groups / 256)))
    if tile == 2 and m <= 64:
        main *= 0.87                                  # the 64-row tile of X with W four steps ahead
    reduce = 2.5 + 2 * splits * m * n * 4 / 3.0e6 if splits > 1 else 0.0
    return main + 5.5 + reduce


@functools.lru_cache(maxsize=4096)
def _wreg_plan(m: int, n: int, k: int) -> tuple[int, int]:
    """Tile and splits of K for a product: the pair with the least estimated time (`_wreg_cost`).  Few rows
    of X want K split so that most CUs get a workgroup, but every split adds partial sums to write and
    read; the narrower tiles are for products whose tiles would leave much of the last round empty."""
    options = [(t, s) for t in (0, 1, 2) for s in (1, 2, 3, 4, 6, 8, 12, 16) if s == 1 or k // s >= 1024]
    return min(options, key=lambda o: (_wreg_cost(o[0], o[1], m, n, k), o[1], o[0]))


def _rows_cost(nt: int, m: int, n: int, k: int) -> float:
    """Estimated microseconds of one gemm_rows launch, fitted to measurements on MI355X (24 to 128 rows against
    the matrices of the 8B shape): W streamed once (at the rate of 256 workgroups, slower with fewer), plus the
    rows of X, which every workgroup fetches from L2 in blocks of 16, plus a launch."""
    blocks16 = 2 if m <= 32 else (4 if m <= 64 else (6 if m <= 96 else 8))
    groups = -(-(-(-n // 16)) // nt)
    w_mb, x_mb = n * k * 2 / 1e6, groups * blocks16 * 16 * k * 2 / 1e6
    # one workgroup a CU at a time (its stages fill the LDS): a last round that is not full runs as long as a full one
    uneven = -(-groups // 256) * 256 / groups
    return 2.5 + (w_mb / 6.2 + x_mb / 22.0) * uneven


@functools.lru_cache(maxsize=4096)
def _rows_plan(m: int, n: int, k: int, norm_rides: bool = False) -> int:
    """Tiles of 16 rows of W a workgroup (1 or 2) if gemm_rows is the faster kernel for this product of 17 to
    128 rows, else 0 (the tiled GEMM).  ``norm_rides``: the product adds into the residual stream and the
    norm that follows is known; with K split, the tiled GEMM's second kernel takes that norm along, gemm_rows
    leaves it to the norm kernel."""
    rows, nt = min((_rows_cost(t, m, n, k), t) for t in (1, 2))
    tile, splits = _wreg_plan(m, n, k)
    other = _wreg_cost(tile, splits, m, n, k)
    if norm_rides:
        rows += 4.5 if splits > 1 else 0.0
    return nt if rows < other else 0


def _big_tile(m: int, n: int) -> int:
    """The tile of gemm_big for a product of this size (measured on MI355X): the wider tile pays
    once there are several rounds of workgroups for the chip's 256 CUs."""
    return 1 if (-(-m // 128)) * (-(-n // 256)) >= 1024 else 0


def swiglu(gu: torch.Tensor, out_dtype, gelu: bool = False) -> torch.Tensor:
    """h[:, j] = act(gu[:, 2j]) * gu[:, 2j+1] for float32 gu; act is silu, or the reference's gelu."""
    _dev(gu)
    _need(gu.dtype == torch.float32 and gu.dim() == 2 and gu.shape[1] % 2 == 0, "gu: float32 [T, 2F]")
    h = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=out_dtype, device=gu.device)
    _check(core().li_swiglu(_ptr(gu), _ptr(h), DT[out_dtype], c_int64(h.numel()), int(gelu), _stream()), "swiglu")
    return h


def rope_store(qkv, inv_freq, rotary_dim, half_pairing, pos, tok_slot, page_table, page_stride, k_pages, v_pages,
               n_heads, n_kv_heads, head_dim, out_dtype, kv_round=None) -> torch.Tensor:
    """Rotate q and k by position, write k and v into the pages; returns q [T, H, hd].
    With n_kv_heads == 0 only q is rotated (a layer that reads another layer's cache).
    ``kv_round`` (a 16-bit dtype): k and v take that type's values before they are stored."""
    _dev(qkv, inv_freq, pos, tok_slot, page_table, k_pages, v_pages)
    t = qkv.shape[0]
    _need(qkv.dtype == torch.float32 and qkv.dim() == 2, "qkv: float32 [T, (H+2K) hd]")
    _need(qkv.shape[1] >= (n_heads + 2 * n_kv_heads) * head_dim, "qkv row too short")
    _need(pos.dtype == torch.int32 and pos.numel() >= t, "pos: int32 [T]")
    if rotary_dim > 0:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() >= rotary_dim // 2,
              "inv_freq: float32 [rotary_dim / 2]")
    if n_kv_heads > 0:
        _need(tok_slot.dtype == torch.int32 and tok_slot.numel() >= t, "tok_slot: int32 [T]")
        _need(page_table.dtype == torch.int32 and page_table.dim() == 2, "page_table: int32 [slots, pages]")
        _need(k_pages.dtype == out_dtype and v_pages.dtype == out_dtype, "cache dtype differs from q dtype")
    q = torch.empty((t, n_heads, head_dim), dtype=out_dtype, device=qkv.device)
    _check(core().li_rope_store(
        _ptr(qkv), qkv.shape[1], _ptr(inv_freq), rotary_dim, int(half_pairing), _ptr(pos), _ptr(tok_slot),
        _ptr(page_table), page_table.shape[1] if page_table is not None else 0, c_int64(page_stride or 0),
        _ptr(q), _ptr(k_pages),
        _ptr(v_pages), DT[out_dtype], t, n_heads, n_kv_heads, head_dim, DT[kv_round or torch.float32], _stream()),
        "rope_store")
    return q


def rope_table(inv_freq: torch.Tensor, pos: torch.Tensor, n_tokens: int) -> torch.Tensor:
    """cos and sin of pos * inv_freq for the tokens of a step: float32 [T, n_freq, 2]."""
    _dev(inv_freq, pos)
    _need(inv_freq.dtype == torch.float32 and pos.dtype == torch.int32 and pos.numel() >= n_tokens,
          "rope_table: float32 frequencies, int32 positions")
    out = torch.empty((n_tokens, inv_freq.numel(), 2), dtype=torch.float32, device=inv_freq.device)
    _check(core().li_rope_table(_ptr(inv_freq), _ptr(pos), _ptr(out), n_tokens, inv_freq.numel(), _stream()),
           "rope_table")
    return out


def linear_rope_store(x, w, inv_freq, rotary_dim, pos, tok_slot, page_table, page_stride, k_pages, v_pages,
                      n_heads, n_kv_heads, head_dim, out_dtype, force=None, cos_sin=None) -> torch.Tensor:
    # (x may be a LazyNorm: linear sorts that out)
    """q, k, v = x W^T with the rotation (adjacent pairs) and the cache write done in the product's
    epilogue, on the float32 accumulators: the same result as linear (float32) followed by
    rope_store, without the round trip.  Returns q [T, H, hd]."""
    _dev(inv_freq, pos, tok_slot, page_table, k_pages, v_pages)
    t = x.shape[0]
    _need(matrix_shape(w)[0] == (n_heads + 2 * n_kv_heads) * head_dim, "linear_rope_store: rows of W are not (H + 2K) hd")
    _need(head_dim % 16 == 0, "head size must be a multiple of 16")
    _need(pos.dtype == torch.int32 and pos.numel() >= t, "pos: int32 [T]")
    if rotary_dim > 0:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() >= rotary_dim // 2,
              "inv_freq: float32 [rotary_dim / 2]")
    if n_kv_heads > 0:
        _need(tok_slot.dtype == torch.int32 and tok_slot.numel() >= t, "tok_slot: int32 [T]")
        _need(page_table.dtype == torch.int32 and page_table.dim() == 2, "page_table: int32 [slots, pages]")
        _need(k_pages.dtype == out_dtype and v_pages.dtype == out_dtype, "cache dtype differs from q dtype")
    q = torch.empty((t, n_heads, head_dim), dtype=out_dtype, device=x.device)
    if cos_sin is not None:
        _dev(cos_sin)
        _need(cos_sin.dtype == torch.float32 and cos_sin.numel() >= t * (rotary_dim // 2) * 2 and
              cos_sin.shape[1] == rotary_dim // 2, "cos_sin: float32 [T, rotary_dim / 2, 2]")
    rs = _RopeStore(inv_freq.data_ptr() if inv_freq is not None else None,
                    cos_sin.data_ptr() if cos_sin is not None else None, pos.data_ptr(),
                    tok_slot.data_ptr() if tok_slot is not None else None,
                    page_table.data_ptr() if page_table is not None else None, q.data_ptr(),
                    k_pages.data_ptr() if k_pages is not None else None,
                    v_pages.data_ptr() if v_pages is not None else None, int(page_stride or 0), rotary_dim,
                    n_heads, n_kv_heads, head_dim, page_table.shape[1] if page_table is not None else 0,
                    DT[out_dtype])
    linear(x, w, EPI_ROPE, force=force, _rope=rs)
    return q


def decode_prepare(seq_slot, lens, pos, ctx, n, scratch_slot: int = -1, inv_freq=None):
    """The bookkeeping of a decode step on the device: row i's token gets position lens[seq_slot[i]], its
    context is one more, the length grows by one; a row on ``scratch_slot`` (an idle row) gets position 0 and
    changes no length.  With ``inv_freq`` the kernel also fills and returns the step's table of angles
    (what ``rope_table`` computes from these positions)."""
    _dev(seq_slot, lens, pos, ctx, inv_freq)
    for a in (seq_slot, lens, pos, ctx):
        _need(a.dtype == torch.int32, "decode_prepare: int32 arrays")
    _need(seq_slot.numel() >= n and pos.numel() >= n and ctx.numel() >= n, "decode_prepare: arrays too short")
    table = None
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() > 0, "decode_prepare: float32 frequencies")
        table = torch.empty((n, inv_freq.numel(), 2), dtype=torch.float32, device=inv_freq.device)
    _check(core().li_decode_prepare(_ptr(seq_slot), _ptr(lens), _ptr(pos), _ptr(ctx), n, int(scratch_slot),
                                    _ptr(inv_freq), _ptr(table), inv_freq.numel() if inv_freq is not None else 0,
                                    _stream()), "decode_prepare")
    return table


# ---------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------
_attn: dict = {}


def _attn_lib(head_dim: int):
    lib = _attn.get(head_dim)
    if lib is None:
        lib = build.attention_library(head_dim)
        _need(lib.li_attn_head_dim() == head_dim, "attention library built for another head size")
        _attn[head_dim] = lib
    return lib


def _check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, dtype):
    _need(k_pages.dtype == dtype and v_pages.dtype == dtype, "cache dtype differs from q dtype")
    _need(page_table.dtype == torch.int32 and page_table.dim() == 2, "page_table: int32 [slots, pages]")


Q_TILE = 128            # tokens of one workgroup of the prefill attention kernel


PREFILL_TILES_KEY = ("attention_prefill_tiles", Q_TILE)      # under this key a step shares the list of tiles


def prefill_tiles(qlens) -> tuple:
    """The tiles of attention_prefill for sequences that bring ``qlens`` tokens: one for every Q_TILE tokens
    of every sequence, as (sequence of the tile, first token of the tile within its sequence's tokens)."""
    tile_seq, tile_q0 = [], []
    for i, n in enumerate(qlens):
        for q0 in range(0, n, Q_TILE):
            tile_seq.append(i)
            tile_q0.append(q0)
    return tile_seq, tile_q0


def prefill_meta(ctx) -> dict:
    """The index arrays of attention_prefill for a step: the per-sequence arrays of the step and the
    kernel's own list of tiles, which is made and uploaded once per step, by the first attention layer that
    runs (a recorded step brings it along under the same key, padded with tiles that begin beyond their
    sequence's tokens)."""
    def tiles():
        tile_seq, tile_q0 = prefill_tiles(ctx.host_qlens)
        both = torch.tensor([tile_seq, tile_q0], dtype=torch.int32).to(ctx.device)
        return {"tile_seq": both[0], "tile_q0": both[1], "n_tiles": len(tile_seq)}
    return dict(ctx.shared(PREFILL_TILES_KEY, tiles), seq_slot=ctx.seq_slot,
                seq_qstart=ctx.seq_qstart, seq_qlen=ctx.seq_qlen, seq_ctx=ctx.seq_ctx)


def attention_prefill(q, kv, meta, n_heads, n_kv_heads, head_dim, scale, window) -> torch.Tensor:
    """16-bit attention for a step with whole prompts.  ``kv``: (k_pages, v_pages, page_stride,
    page_table); ``meta``: dict of int32 device arrays tile_seq, tile_q0, seq_slot, seq_qstart,
    seq_qlen, seq_ctx and the int n_tiles."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table)
    _need(q.dtype in (torch.float16, torch.bfloat16) and q.shape[1:] == (n_heads, head_dim), "q: 16-bit [T, H, hd]")
    _check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, q.dtype)
    out = torch.empty_like(q)
    _check(_attn_lib(head_dim).li_attn_prefill(
        _ptr(q), _ptr(out), DT[q.dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(meta["tile_seq"]), _ptr(meta["tile_q0"]), meta["n_tiles"], _ptr(meta["seq_slot"]),
        _ptr(meta["seq_qstart"]), _ptr(meta["seq_qlen"]), _ptr(meta["seq_ctx"]), n_heads, n_kv_heads,
        c_float(scale), int(window or 0), _stream()), "attn_prefill")
    return out


def attention_decode(q, kv, seq_slot, seq_ctx, n_seqs, n_heads, n_kv_heads, head_dim, scale, window,
                     splits: int = 1) -> torch.Tensor:
    """16-bit attention for one new token per sequence; q [B, H, hd]."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table, seq_slot, seq_ctx)
    _need(q.dtype in (torch.float16, torch.bfloat16) and q.shape == (n_seqs, n_heads, head_dim), "q: 16-bit [B, H, hd]")
    _check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, q.dtype)
    _need(seq_slot.numel() >= n_seqs and seq_ctx.numel() >= n_seqs, "per-sequence arrays too short")
    out = torch.empty_like(q)
    part_o = part_ml = None
    lib = _attn_lib(head_dim)
    # two or four splits are merged inside a workgroup; more are merged by a second kernel
    parts = lib.li_attn_decode_parts(splits)
    _need(1 <= parts <= 64, f"attention_decode: {splits} splits")
    if parts > 1:
        part_o = torch.empty((n_seqs, n_heads, parts, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_seqs, n_heads, parts, 2), dtype=torch.float32, device=q.device)
    _check(lib.li_attn_decode(
        _ptr(q), _ptr(out), DT[q.dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(seq_slot), _ptr(seq_ctx), n_seqs, n_heads, n_kv_heads, c_float(scale),
        int(window or 0), splits, _ptr(part_o), _ptr(part_ml), _stream()), "attn_decode")
    return out


def attention_f32(q, kv, pos, tok_slot, n_heads, n_kv_heads, head_dim, scale, window) -> torch.Tensor:
    """float32 attention for any step: every token reads its sequence's cache up to its position."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table, pos, tok_slot)
    _need(q.dtype == torch.float32 and q.shape[1:] == (n_heads, head_dim), "q: float32 [T, H, hd]")
    _check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, torch.float32)
    _need(pos.numel() >= q.shape[0] and tok_slot.numel() >= q.shape[0], "per-token arrays too short")
    out = torch.empty_like(q)
    _check(_attn_lib(head_dim).li_attn_f32(
        _ptr(q), _ptr(out), _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(pos), _ptr(tok_slot), q.shape[0], n_heads, n_kv_heads, c_float(scale),
        int(window or 0), _stream()), "attn_f32")
    return out


# ---------------------------------------------------------------------------
# sampling
# ---------------------------------------------------------------------------
def argmax(logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    _dev(logits, out)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits: float32 [B, V]")
    if out is None:
        out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    _need(out.dtype == torch.int32 and out.numel() >= logits.shape[0], "out: int32 [B]")
    n = logits.shape[0] * core().li_argmax_chunks(logits.shape[1])
    part_v = torch.empty((n,), dtype=torch.float32, device=logits.device)
    part_i = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _check(core().li_argmax(_ptr(logits), logits.shape[0], logits.shape[1], _ptr(part_v), _ptr(part_i), _ptr(out),
                            _stream()), "argmax")
    return out


def sample(logits, temperature: float, seq_slot=None, state=None, forced_r=None, out=None,
           temperature_dev=None) -> torch.Tensor:
    """Temperature sampling; ``state`` is the [slots, 2] int64 (key, counter) table, ``forced_r``
    (float32 [B]) replaces the generator for tests.  ``temperature_dev`` (float32 [1] on the device, holding
    the same positive value) is what the kernels read if given, so that a recorded step serves any temperature."""
    _dev(logits, seq_slot, state, forced_r, out, temperature_dev)
    if temperature_dev is not None:
        _need(temperature_dev.dtype == torch.float32 and temperature_dev.numel() >= 1, "temperature_dev: float32 [1]")
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits: float32 [B, V]")
    b = logits.shape[0]
    if temperature <= 0:
        return argmax(logits, out)
    if out is None:
        out = torch.empty((b,), dtype=torch.int32, device=logits.device)
    if temperature > 0 and forced_r is None:
        _need(seq_slot is not None and seq_slot.dtype == torch.int32 and seq_slot.numel() >= b, "seq_slot: int32 [B]")
        _need(state is not None and state.dtype == torch.int64 and state.dim() == 2 and state.shape[1] == 2,
              "state: int64 [slots, 2]")
    if forced_r is not None:
        _need(forced_r.dtype == torch.float32 and forced_r.numel() >= b, "forced_r: float32 [B]")
    ws = torch.empty((b * core().li_sample_ws_floats(logits.shape[1]),), dtype=torch.float32, device=logits.device)
    _check(core().li_sample(_ptr(logits), b, logits.shape[1], c_float(temperature), _ptr(temperature_dev),
                            _ptr(seq_slot), _ptr(state), _ptr(forced_r), _ptr(ws), _ptr(out), _stream()), "sample")
    return out


def token_prob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """softmax(logits[r])[tokens[r]] at temperature 1, float32 [B]; 0 for a token outside the vocabulary
    (tools/infer.cpp:77-81)."""
    _dev(logits, tokens)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits: float32 [B, V]")
    b = logits.shape[0]
    _need(tokens.dtype == torch.int32 and tokens.numel() == b, "tokens: int32 [B]")
    out = torch.empty((b,), dtype=torch.float32, device=logits.device)
    ws = torch.empty((b * core().li_sample_ws_floats(logits.shape[1]),), dtype=torch.float32, device=logits.device)
    _check(core().li_token_prob(_ptr(logits), b, logits.shape[1], _ptr(tokens), _ptr(ws), _ptr(out), _stream()),
           "token_prob")
    return out


def uniform01(key: int, counter: int) -> float:
    """The generator's value for (key, counter), computed on the host by the same function."""
    return float(core().li_uniform01(c_uint64(key & (2 ** 64 - 1)), c_uint64(counter & (2 ** 64 - 1))))


def tile_weight(w: torch.Tensor) -> Tensor:
    """A 16-bit matrix [N, K] (K a multiple of 32) as a device-owned ``Tensor`` in tiled layout."""
    _dev(w)
    _need(can_tile(w), "tile_weight: 16-bit [N, K] on the GPU with K a multiple of 32")
    n, k = w.shape
    out = torch.empty(((n + 15) // 16 * 16 * k,), dtype=w.dtype, device=w.device)
    _check(core().li_tile_weight(_ptr(w), _ptr(out), DT[w.dtype], n, k, _stream()), "tile_weight")
    return Tensor.wrap(out, "tiled", (n, k))


def untile(w: Tensor) -> torch.Tensor:
    """The matrix [N, K] that a tiled ``Tensor`` holds, in rows (for inspection and tests; on the device)."""
    _need(is_tiled(w), "untile: a tiled Tensor")
    n, k = w.logical
    flat = w.as_subclass(torch.Tensor)
    # [n/16][k/32][lane = 16 * ((k % 32) / 8) + n % 16][k % 8]  ->  [n][k]
    t = flat.view((n + 15) // 16, k // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(-1, k)
    return t[:n].contiguous()


def gemv_tiled(x, w: Tensor, mode=EPI_STORE, out_dtype=None, nt=0, kw=0):
    """gemv_tiled with a chosen shape of workgroup (for tuning and tests)."""
    m, k = x.shape
    n = w.logical[0]
    n_out = n // 2 if mode in GATED else n
    out = torch.empty((m, n_out), dtype=out_dtype or x.dtype, device=x.device)
    _check(core().li_gemv_tiled(_ptr(x), _ptr(w), DT[x.dtype], _ptr(out), DT[out.dtype], mode, m, n, k,
                                nt, kw, None, None, None, _stream()), "gemv_tiled")
    return out
