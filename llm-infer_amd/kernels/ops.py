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
EPI_STORE, EPI_ADD, EPI_SWIGLU, EPI_ROPE, EPI_GEGLU, EPI_BIAS, EPI_CLAMPGLU = 0, 1, 2, 3, 4, 5, 6
GATED = (EPI_SWIGLU, EPI_GEGLU, EPI_CLAMPGLU)   # gate and up rows interleaved in W, act(gate) * up written
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


class _GluParams(ctypes.Structure):
    _fields_ = [("bias", c_void_p), ("limit", c_float), ("tail_limit", c_float), ("alpha", c_float), ("shift", c_float),
                ("tail_col", c_int)]


def glu_params(bias=None, limit: float = 1.0, tail_limit: float | None = None, alpha: float = 1.702, shift: float = 1.0,
               tail_col: int | None = None):
    """What ``linear`` needs for EPI_BIAS (``bias`` float32 [N]) and EPI_CLAMPGLU (gate and up columns interleaved; a bias
    for every column or None; g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(alpha g) (u + shift); the
    outputs from ``tail_col`` on take ``tail_limit``).  Keeps the bias alive as long as it lives itself."""
    _need(bias is None or (bias.dtype == torch.float32 and bias.dim() == 1 and bias.is_contiguous() and bias.is_cuda),
          "a float32 bias on the device")
    p = _GluParams(bias.data_ptr() if bias is not None else None, limit, limit if tail_limit is None else tail_limit, alpha, shift,
                   (1 << 30) if tail_col is None else tail_col)
    p._bias = bias
    return p


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
           out_dtype=None, force: str | None = None, _rope=None, params=None) -> torch.Tensor:
    """C = X W^T with the epilogue ``mode``: store, add into ``out`` (float32), or act(gate) * up over
    interleaved gate/up rows of W (C has N/2 columns; EPI_SWIGLU: silu, EPI_GEGLU: gelu).  EPI_BIAS stores the sums plus
    a bias, EPI_CLAMPGLU the clamped gated activation of biased sums; both take ``params`` (``glu_params``).
    ``force`` picks a kernel for tests."""
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
    if mode in (EPI_BIAS, EPI_CLAMPGLU):
        _need(isinstance(params, _GluParams) and (mode != EPI_BIAS or (params._bias is not None and params._bias.numel() == n)) and
              (params._bias is None or params._bias.numel() == n), "this epilogue needs its parameters (glu_params), a bias for every column")
        rs = ctypes.byref(params)
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


def attention_prefill(q, kv, meta, n_heads, n_kv_heads, head_dim, scale, window, block=None, sink=None, slopes=None,
                      gate=None, gate_col: int = 0) -> torch.Tensor:
    """16-bit attention for a step with whole prompts.  ``kv``: (k_pages, v_pages, page_stride,
    page_table); ``meta``: dict of int32 device arrays tile_seq, tile_q0, seq_slot, seq_qstart,
    seq_qlen, seq_ctx and the int n_tiles.  ``block`` b: a token at position p reads no key before p - p % b;
    ``sink`` (float32 [H]): every head's sum of weights also counts exp(sink[h]); ``slopes`` (float32 [H]): the
    score of the key at position j loses slopes[h] * (p - j); ``gate`` (float32 rows [T, >= gate_col + H]): head
    h's output is multiplied by sigmoid(gate[t][gate_col + h])."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table, sink, slopes, gate)
    for name, vec in (("sink", sink), ("slopes", slopes)):
        _need(vec is None or (vec.dtype == torch.float32 and vec.numel() == n_heads and vec.is_contiguous()), f"{name}: float32 [H]")
    _need(gate is None or (gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == q.shape[0] and gate.stride(1) == 1
                           and 0 <= gate_col and gate_col + n_heads <= gate.shape[1]), "gate: float32 rows with a column for every head")
    _need(q.dtype in (torch.float16, torch.bfloat16) and q.shape[1:] == (n_heads, head_dim), "q: 16-bit [T, H, hd]")
    _check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, q.dtype)
    out = torch.empty_like(q)
    _check(_attn_lib(head_dim).li_attn_prefill(
        _ptr(q), _ptr(out), DT[q.dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(meta["tile_seq"]), _ptr(meta["tile_q0"]), meta["n_tiles"], _ptr(meta["seq_slot"]),
        _ptr(meta["seq_qstart"]), _ptr(meta["seq_qlen"]), _ptr(meta["seq_ctx"]), n_heads, n_kv_heads,
        c_float(scale), int(window or 0), int(block or 0), _ptr(sink), _ptr(slopes), _ptr(gate),
        gate.stride(0) if gate is not None else 0, int(gate_col), _stream()), "attn_prefill")
    return out


def attention_decode(q, kv, seq_slot, seq_ctx, n_seqs, n_heads, n_kv_heads, head_dim, scale, window,
                     splits: int = 1, block=None, sink=None, slopes=None, gate=None, gate_col: int = 0) -> torch.Tensor:
    """16-bit attention for one new token per sequence; q [B, H, hd].  ``block``, ``sink``, ``slopes``, ``gate``: as
    for ``attention_prefill``."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table, seq_slot, seq_ctx, sink, slopes, gate)
    for name, vec in (("sink", sink), ("slopes", slopes)):
        _need(vec is None or (vec.dtype == torch.float32 and vec.numel() == n_heads and vec.is_contiguous()), f"{name}: float32 [H]")
    _need(gate is None or (gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] >= n_seqs and gate.stride(1) == 1
                           and 0 <= gate_col and gate_col + n_heads <= gate.shape[1]), "gate: float32 rows with a column for every head")
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
        int(window or 0), splits, _ptr(part_o), _ptr(part_ml), int(block or 0), _ptr(sink), _ptr(slopes), _ptr(gate),
        gate.stride(0) if gate is not None else 0, int(gate_col), _stream()), "attn_decode")
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


# ---------------------------------------------------------------------------
# the other mixers, norms and activations (csrc/mixers.hip)
# ---------------------------------------------------------------------------
_mixers = None


def mixers():
    global _mixers
    if _mixers is None:
        _mixers = build.mixers_library()
    return _mixers


def _f32_rows(x, what):
    _need(x.dtype == torch.float32 and x.dim() == 2, f"{what}: float32 [T, n]")


def layernorm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype, rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = (x[rows[r]] - mean) / sqrt(var + eps) * w, float32 inside; no bias."""
    _dev(x, w, rows)
    _f32_rows(x, "layernorm x")
    _need(w.dtype == torch.float32 and w.shape == (x.shape[1],), "norm weight: float32 [d]")
    if rows is not None:
        _need(rows.dtype == torch.int32, "rows: int32")
    n = x.shape[0] if rows is None else rows.numel()
    out = torch.empty((n, x.shape[1]), dtype=out_dtype, device=x.device)
    _check(mixers().li_layernorm(_ptr(x), _ptr(w), _ptr(rows), _ptr(out), DT[out_dtype], n, x.shape[1], c_float(eps),
                                 _stream()), "layernorm")
    return out


def add_layernorm(x, alpha: float, addends, w, eps: float, copy_dtype=None):
    """x <- LN(alpha * x + sum of scale_i * y_i) * w in place on the float32 rows of ``x``; ``addends``: one or
    two (y, scale) with y float32 of x's shape.  ``copy_dtype`` (a 16-bit type): the new rows are returned in
    that type as well (else None)."""
    _need(1 <= len(addends) <= 2, "add_layernorm: one or two addends")
    (y1, s1), (y2, s2) = addends[0], (addends[1] if len(addends) > 1 else (None, 0.0))
    _dev(x, y1, y2, w)
    _f32_rows(x, "add_layernorm x")
    for y in (y1, y2):
        _need(y is None or (y.dtype == torch.float32 and y.shape == x.shape), "add_layernorm: addends float32 like x")
    _need(w.dtype == torch.float32 and w.shape == (x.shape[1],), "norm weight: float32 [d]")
    _drop_row_stats(x)
    copy = None
    if copy_dtype is not None and copy_dtype != torch.float32:
        copy = torch.empty(x.shape, dtype=copy_dtype, device=x.device)
    _check(mixers().li_add_layernorm(_ptr(x), c_float(alpha), _ptr(y1), c_float(s1), _ptr(y2), c_float(s2), _ptr(w),
                                     c_float(eps), _ptr(copy), DT[copy.dtype] if copy is not None else 0, x.shape[0],
                                     x.shape[1], _stream()), "add_layernorm")
    return copy


def add_scaled(x, addends) -> None:
    """x += sum of scale_i * y_i (one or two addends, float32 of x's shape)."""
    _need(1 <= len(addends) <= 2, "add_scaled: one or two addends")
    (y1, s1), (y2, s2) = addends[0], (addends[1] if len(addends) > 1 else (None, 0.0))
    _dev(x, y1, y2)
    for y in (x, y1, y2):
        _need(y is None or (y.dtype == torch.float32 and y.shape == x.shape), "add_scaled: float32 tensors of one shape")
    _drop_row_stats(x)
    _check(mixers().li_add_scaled(_ptr(x), _ptr(y1), c_float(s1), _ptr(y2), c_float(s2), c_int64(x.numel()), _stream()),
           "add_scaled")


def cast(x: torch.Tensor, dtype) -> torch.Tensor:
    """float32 -> a 16-bit type (a float32 ``dtype`` gives ``x`` itself back)."""
    if dtype == torch.float32:
        return x
    _dev(x)
    _need(x.dtype == torch.float32 and dtype in (torch.float16, torch.bfloat16), "cast: float32 to a 16-bit type")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _check(mixers().li_cast(_ptr(x), _ptr(out), DT[dtype], c_int64(x.numel()), _stream()), "cast")
    return out


def token_shift(x, mu, state, pos, tok_slot, out_dtype, single: bool = False) -> torch.Tensor:
    """out_t = x_t + (x_{t-1} - x_t) * mu with the row before from this step or from ``state[slot]`` (zeros at
    position 0); afterwards ``state[slot]`` holds each sequence's last row of this step.  ``single``: every
    sequence brings exactly one row (a decode step), which one kernel then serves."""
    _dev(x, mu, state, pos, tok_slot)
    _f32_rows(x, "token_shift x")
    t, d = x.shape
    _need(mu.dtype == torch.float32 and mu.shape == (d,), "token_shift: float32 [d] mixing weights")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == d, "token_shift: state float32 [slots, d]")
    _need(pos.dtype == torch.int32 and tok_slot.dtype == torch.int32 and pos.numel() >= t and tok_slot.numel() >= t,
          "token_shift: int32 positions and slots for every token")
    out = torch.empty((t, d), dtype=out_dtype, device=x.device)
    _check(mixers().li_token_shift(_ptr(x), _ptr(mu), _ptr(state), _ptr(pos), _ptr(tok_slot), _ptr(out), DT[out_dtype],
                                   t, d, int(bool(single)), _stream()), "token_shift")
    return out


def rope_norm_store(qkv, inv_freq, rotary_dim, half_pairing, unit_eps, pos, tok_slot, kv, n_heads, n_kv_heads,
                    head_dim, v_head_dim, q_dim, k_dim, v_dim, out_dtype, col0: int = 0, cos_sin=None) -> torch.Tensor:
    """q and k of a step rotated by position (half or adjacent pairing), then, with ``unit_eps`` not None,
    divided by their root mean square per head; k and v written into the pages (``kv`` = (k_pages, v_pages,
    page_stride, page_table); head sizes ``k_dim`` and ``v_dim`` in the pages, zeros beyond the true ones).
    ``col0``: the column of ``qkv`` at which q begins (a product shared with other mixers).  ``cos_sin``: the
    step's table of angles (``rope_table`` of the same frequencies and positions), read instead of computed.
    Returns q [T, H, q_dim]."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(qkv, inv_freq, pos, tok_slot, k_pages, v_pages, page_table)
    _f32_rows(qkv, "rope_norm_store qkv")
    t = qkv.shape[0]
    _need(col0 >= 0 and qkv.shape[1] >= col0 + (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_head_dim, "qkv row too short")
    _need(pos.dtype == torch.int32 and tok_slot.dtype == torch.int32 and pos.numel() >= t and tok_slot.numel() >= t,
          "int32 positions and slots for every token")
    _need(max(head_dim, q_dim, k_dim, v_dim) <= 256 and q_dim >= head_dim and k_dim >= head_dim and v_dim >= v_head_dim
          and k_dim % 16 == 0 and v_dim % 16 == 0, "head sizes up to 256, padded sizes multiples of 16")
    if rotary_dim > 0:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() >= rotary_dim // 2,
              "inv_freq: float32 [rotary_dim / 2]")
    _need(k_pages.dtype == out_dtype and v_pages.dtype == out_dtype, "cache dtype differs from q dtype")
    _need(page_table.dtype == torch.int32 and page_table.dim() == 2, "page_table: int32 [slots, pages]")
    if cos_sin is not None and rotary_dim > 0:
        _dev(cos_sin)
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[0] >= t and
              cos_sin.shape[1:] == (rotary_dim // 2, 2), "cos_sin: float32 [T, rotary_dim / 2, 2]")
    else:
        cos_sin = None
    q = torch.empty((t, n_heads, q_dim), dtype=out_dtype, device=qkv.device)
    _check(mixers().li_rope_norm_store(
        c_void_p(qkv.data_ptr() + 4 * col0), qkv.shape[1], _ptr(inv_freq), _ptr(cos_sin), rotary_dim, int(half_pairing),
        c_float(-1.0 if unit_eps is None else unit_eps), _ptr(pos), _ptr(tok_slot), _ptr(k_pages), _ptr(v_pages),
        c_int64(page_stride), _ptr(page_table), page_table.shape[1], _ptr(q), DT[out_dtype], t, n_heads, n_kv_heads,
        head_dim, v_head_dim, q_dim, k_dim, v_dim, _stream()), "rope_norm_store")
    return q


def sigmoid_attention(q, kv, pos, tok_slot, bias, n_heads, n_kv_heads, k_dim, v_head_dim, v_dim, scale, window=None):
    """out[t, h] = sum over visible keys j of sigmoid(q_t . k_j * scale + bias[h]) v_j (no normalisation over
    the keys); q [T, H, k_dim] and the pages in one type, scores and weights float32.  Returns [T, H, v_head_dim]."""
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table, pos, tok_slot, bias)
    _need(q.dtype in DT and q.dim() == 3 and q.shape[1:] == (n_heads, k_dim), "q: [T, H, k_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv_heads, k_dim, q.dtype)
    _need(n_heads % n_kv_heads == 0, "query heads: a multiple of the key/value heads")
    _need(pos.numel() >= q.shape[0] and tok_slot.numel() >= q.shape[0], "per-token arrays too short")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_heads), "bias: float32 [H]")
    out = torch.empty((q.shape[0], n_heads, v_head_dim), dtype=q.dtype, device=q.device)
    _check(mixers().li_sigmoid_attn(_ptr(q), _ptr(out), DT[q.dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride),
                                    _ptr(page_table), page_table.shape[1], _ptr(pos), _ptr(tok_slot), _ptr(bias),
                                    q.shape[0], n_heads, n_kv_heads, k_dim, v_head_dim, v_dim, c_float(scale),
                                    int(window or 0), _stream()), "sigmoid_attn")
    return out


_sigattn: dict = {}


def _sigattn_lib(key_dim: int, value_dim: int):
    lib = _sigattn.get((key_dim, value_dim))
    if lib is None:
        lib = build.sigmoid_attention_library(key_dim, value_dim)
        _need(lib.li_sigattn_key_dim() == key_dim and lib.li_sigattn_value_dim() == value_dim,
              "sigmoid attention library built for other head sizes")
        _sigattn[key_dim, value_dim] = lib
    return lib


def _sigattn_check(q, kv, bias, n_heads, n_kv_heads, k_dim, v_head_dim, v_dim):
    k_pages, v_pages, page_stride, page_table = kv
    _dev(q, k_pages, v_pages, page_table, bias)
    _need(q.dtype in (torch.float16, torch.bfloat16) and q.dim() == 3 and q.shape[1:] == (n_heads, k_dim),
          "q: 16-bit [T, H, k_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv_heads, k_dim, q.dtype)
    _need(n_heads % n_kv_heads == 0 and 0 < v_head_dim <= v_dim, "heads and head sizes do not fit")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_heads), "bias: float32 [H]")
    return k_pages, v_pages, page_stride, page_table


def sigmoid_attention_prefill(q, kv, meta, bias, n_heads, n_kv_heads, k_dim, v_head_dim, v_dim, scale, window=None):
    """16-bit sigmoid attention for a step with prompts (or portions of prompts) on the matrix cores; ``meta`` as
    for ``attention_prefill``.  Returns [T, H, v_head_dim]."""
    k_pages, v_pages, page_stride, page_table = _sigattn_check(q, kv, bias, n_heads, n_kv_heads, k_dim, v_head_dim, v_dim)
    out = torch.empty((q.shape[0], n_heads, v_head_dim), dtype=q.dtype, device=q.device)
    _check(_sigattn_lib(k_dim, v_dim).li_sigattn_prefill(
        _ptr(q), _ptr(out), DT[q.dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(meta["tile_seq"]), _ptr(meta["tile_q0"]), meta["n_tiles"], _ptr(meta["seq_slot"]),
        _ptr(meta["seq_qstart"]), _ptr(meta["seq_qlen"]), _ptr(meta["seq_ctx"]), _ptr(bias), n_heads, n_kv_heads,
        v_head_dim, c_float(scale), int(window or 0), _stream()), "sigattn_prefill")
    return out


def sigmoid_attention_decode(q, kv, seq_slot, seq_ctx, n_seqs, bias, n_heads, n_kv_heads, k_dim, v_head_dim, v_dim,
                             scale, window=None, splits: int = 1):
    """16-bit sigmoid attention for one new token per sequence; q [B, H, k_dim].  The context is cut into
    ``splits`` parts whose sums are added in ascending order."""
    k_pages, v_pages, page_stride, page_table = _sigattn_check(q, kv, bias, n_heads, n_kv_heads, k_dim, v_head_dim, v_dim)
    _dev(seq_slot, seq_ctx)
    _need(q.shape[0] == n_seqs and seq_slot.numel() >= n_seqs and seq_ctx.numel() >= n_seqs, "per-sequence arrays too short")
    _need(1 <= splits <= 64, f"sigmoid_attention_decode: {splits} splits")
    out = torch.empty((n_seqs, n_heads, v_head_dim), dtype=q.dtype, device=q.device)
    part = None
    if splits > 1:
        part = torch.empty((n_seqs, n_heads, splits, v_head_dim), dtype=torch.float32, device=q.device)
    _check(_sigattn_lib(k_dim, v_dim).li_sigattn_decode(
        _ptr(q), _ptr(out), DT[q.dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(seq_slot), _ptr(seq_ctx), _ptr(bias), n_seqs, n_heads, n_kv_heads, v_head_dim,
        c_float(scale), int(window or 0), splits, _ptr(part), _stream()), "sigattn_decode")
    return out


DECAY_CHUNK = 32        # tokens of one chunk of the chunked decay attention


def decay_padded_dim(d: int) -> int:
    """The width in which the chunked kernels hold a head of ``d`` dimensions: 32 times the number of 32-row
    blocks they are compiled for (1, 2, 4 or 8), as csrc/mixers.hip li_decay_attn_chunked picks it."""
    return 32 if d <= 32 else (64 if d <= 64 else (128 if d <= 128 else 256))


def decay_chunk_lists(qlens) -> tuple:
    """The chunks of the chunked decay attention for sequences that bring ``qlens`` tokens: for every chunk its
    sequence and its first token within the sequence's tokens, and for every sequence its first chunk."""
    chunk_seq, chunk_t0, seq_chunk0 = [], [], []
    for i, n in enumerate(qlens):
        seq_chunk0.append(len(chunk_seq))
        for t0 in range(0, n, DECAY_CHUNK):
            chunk_seq.append(i)
            chunk_t0.append(t0)
    return chunk_seq, chunk_t0, seq_chunk0


def decay_chunks(ctx) -> dict:
    """The chunk lists of a step on the device, made and uploaded once per step by the first layer that asks."""
    def make():
        chunk_seq, chunk_t0, seq_chunk0 = decay_chunk_lists(ctx.host_qlens)
        flat = torch.tensor(chunk_seq + chunk_t0 + seq_chunk0, dtype=torch.int32).to(ctx.device)
        n = len(chunk_seq)
        return {"chunk_seq": flat[:n], "chunk_t0": flat[n:2 * n], "seq_chunk0": flat[2 * n:], "n_chunks": n}
    return ctx.shared(("decay_attention_chunks", DECAY_CHUNK), make)


def decay_attention(proj, q_off, k_off, v_off, state, decay, seq_slot, seq_qstart, seq_qlen, n_seqs, n_heads,
                    head_dim, v_head_dim, round_to=None, chunked: bool = False, chunks=None) -> torch.Tensor:
    """Linear attention with a constant decay per head over the tokens of a step, from and into the float32
    ``state`` [slots, H, d, dv]: S <- decay S + k v^T, o = S^T q, with q, k, v = silu of the columns of ``proj``
    (float32 [T, n]) at the given offsets.  ``seq_qstart`` / ``seq_qlen`` None: one token per sequence.
    ``round_to`` (a 16-bit type): q, k and v take that type's values after the silu.  ``chunked`` (needs
    ``round_to``, the per-sequence arrays and ``chunks`` = ``decay_chunks(ctx)``): 32 tokens at a time on the
    matrix cores, for prompts; else token by token.  Returns float32 [T, H * dv]."""
    _dev(proj, state, decay, seq_slot, seq_qstart, seq_qlen)
    _f32_rows(proj, "decay_attention proj")
    H, d, dv = n_heads, head_dim, v_head_dim
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == (H, d, dv), "state: float32 [slots, H, d, dv]")
    _need(decay.dtype == torch.float32 and decay.numel() == H, "decay: float32 [H]")
    _need(max(q_off + H * d, k_off + H * d, v_off + H * dv) <= proj.shape[1], "decay_attention: columns outside proj")
    _need(seq_slot.dtype == torch.int32 and seq_slot.numel() >= n_seqs, "seq_slot: int32 [sequences]")
    if seq_qstart is None:
        _need(seq_qlen is None and proj.shape[0] >= n_seqs, "one token per sequence needs a row for each")
    else:
        _need(seq_qlen is not None and seq_qstart.dtype == torch.int32 and seq_qlen.dtype == torch.int32 and
              seq_qstart.numel() >= n_seqs and seq_qlen.numel() >= n_seqs, "seq_qstart, seq_qlen: int32 [sequences]")
    _need(round_to in (None, torch.float32, torch.float16, torch.bfloat16), "round_to: a 16-bit type or None")
    out = torch.empty((proj.shape[0], H * dv), dtype=torch.float32, device=proj.device)
    if chunked:
        _need(round_to in (torch.float16, torch.bfloat16) and seq_qstart is not None and chunks is not None,
              "the chunked kernels multiply 16-bit numbers and need the sequences' rows and the list of chunks")
        n_chunks = chunks["n_chunks"]
        ds = torch.empty((max(1, n_chunks), H, d, dv), dtype=torch.float32, device=proj.device)
        # q in 16 bits for the carry kernel, rows as wide as the kernels' template holds them: 32, 64, 128 or 256
        # (the kernels index with that width; a narrower buffer would be written past its end)
        qa = torch.empty((proj.shape[0], H, decay_padded_dim(d)), dtype=round_to, device=proj.device)
        _check(mixers().li_decay_attn_chunked(_ptr(proj), proj.shape[1], q_off, k_off, v_off, _ptr(state), _ptr(decay),
                                              _ptr(seq_slot), _ptr(seq_qstart), _ptr(seq_qlen), _ptr(chunks["seq_chunk0"]),
                                              _ptr(chunks["chunk_seq"]), _ptr(chunks["chunk_t0"]), n_chunks, _ptr(out),
                                              _ptr(ds), _ptr(qa), qa.shape[2], n_seqs, H, d, dv, DT[round_to], _stream()),
               "decay_attn_chunked")
        return out
    _check(mixers().li_decay_attn(_ptr(proj), proj.shape[1], q_off, k_off, v_off, _ptr(state), _ptr(decay),
                                  _ptr(seq_slot), _ptr(seq_qstart), _ptr(seq_qlen), _ptr(out), n_seqs, H, d, dv,
                                  DT[round_to or torch.float32], _stream()), "decay_attn")
    return out


def gated_rmsnorm(o, w, gate_rows, gate_off, eps, out_dtype) -> torch.Tensor:
    """o / sqrt(mean(o^2) + eps) * w * sigmoid(gate): o float32 [T, n]; the gate is columns gate_off .. gate_off + n
    of the float32 rows ``gate_rows``."""
    _dev(o, w, gate_rows)
    _f32_rows(o, "gated_rmsnorm o")
    _f32_rows(gate_rows, "gated_rmsnorm gate")
    t, n = o.shape
    _need(w.dtype == torch.float32 and w.shape == (n,), "norm weight: float32 [n]")
    _need(gate_rows.shape[0] == t and gate_off + n <= gate_rows.shape[1], "gate columns outside their rows")
    out = torch.empty((t, n), dtype=out_dtype, device=o.device)
    gate = gate_rows.view(-1)[gate_off:]
    _check(mixers().li_gated_rmsnorm(_ptr(o), _ptr(w), _ptr(gate), gate_rows.shape[1], _ptr(out), DT[out_dtype], t, n,
                                     c_float(eps), _stream()), "gated_rmsnorm")
    return out


def polynorm(z, coef, eps, out_dtype) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e over float32 rows; coef float32 [4] = (a, b, c, e)."""
    _dev(z, coef)
    _f32_rows(z, "polynorm z")
    _need(coef.dtype == torch.float32 and coef.numel() == 4, "polynorm: float32 [4] coefficients")
    out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
    _check(mixers().li_polynorm(_ptr(z), _ptr(coef), _ptr(out), DT[out_dtype], z.shape[0], z.shape[1], c_float(eps),
                                _stream()), "polynorm")
    return out


# ---------------------------------------------------------------------------
# hybrid decoders (csrc/hybrid.hip): differential attention over blocks of positions, the state-space mixer,
# routed experts, a scaled embedding with sinusoidal positions
# ---------------------------------------------------------------------------
_hybrid = None
ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu2": 3}


def hybrid():
    global _hybrid
    if _hybrid is None:
        _hybrid = build.hybrid_library()
    return _hybrid


def _i32(t, n, what):
    _need(t is not None and t.dtype == torch.int32 and t.numel() >= n, f"{what}: int32, one for each of {n}")


def embed_positions(table, tokens, pos, freq, scale: float) -> torch.Tensor:
    """x[t] = float32(table[tokens[t]]) * scale + P(pos[t]); P(p)[2i] = sin(p freq[i]), P(p)[2i+1] = cos(p freq[i])
    (``freq`` None: no positions)."""
    _dev(table, tokens, pos, freq)
    n, (vocab, d) = tokens.numel(), table.shape
    _need(tokens.dtype == torch.int32 and table.dim() == 2 and table.dtype in DT, "embed: int32 tokens, a float table")
    if freq is not None:
        _i32(pos, n, "embed positions")
        _need(freq.dtype == torch.float32 and freq.numel() >= (d + 1) // 2, "embed: a float32 frequency for every pair")
    out = torch.empty((n, d), dtype=torch.float32, device=table.device)
    _check(hybrid().li_embed_pos(_ptr(table), DT[table.dtype], _ptr(tokens), _ptr(pos), _ptr(freq), _ptr(out), n, d,
                                 c_float(scale), _stream()), "embed_pos")
    return out


def concat_cast(a, b, dtype) -> torch.Tensor:
    """[a | b] row by row in ``dtype`` (a, b float32 of one shape)."""
    _dev(a, b)
    _f32_rows(a, "concat a")
    _need(b.dtype == torch.float32 and b.shape == a.shape and dtype in DT, "concat: two float32 tensors of one shape")
    out = torch.empty((a.shape[0], 2 * a.shape[1]), dtype=dtype, device=a.device)
    _check(hybrid().li_concat_cast(_ptr(a), _ptr(b), _ptr(out), DT[dtype], a.shape[0], a.shape[1], _stream()), "concat_cast")
    return out


def activation(z, kind: str, out_dtype) -> torch.Tensor:
    """act(z) for float32 z in ``out_dtype``; kind: gelu (erf), gelu_tanh, silu, relu2 (the square of relu)."""
    _dev(z)
    _need(z.dtype == torch.float32 and kind in ACTIVATIONS and out_dtype in DT, f"activation {kind!r}: float32 in, one of {', '.join(ACTIVATIONS)}")
    out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
    _check(hybrid().li_activation(_ptr(z), _ptr(out), DT[out_dtype], c_int64(z.numel()), ACTIVATIONS[kind], _stream()),
           "activation")
    return out


def padded_map_dim(d: int) -> int:
    """The width of one map's keys in the pages and in q: the next multiple of 16 (zeros behind the d dimensions)."""
    return (d + 15) // 16 * 16


def _map_pages_check(kv, n_kv_heads, key_width, v_dim):
    k_pages, v_pages, page_stride, page_table = kv
    _dev(k_pages, v_pages, page_table)
    _need(k_pages.dtype == v_pages.dtype and k_pages.dtype in DT, "cache: one float type for keys and values")
    _need(page_table.dtype == torch.int32 and page_table.dim() == 2, "page_table: int32 [slots, pages]")
    _need(page_stride >= n_kv_heads * PAGE * (key_width + (v_dim + 31) // 32 * 32), "a page is too small for these keys and values")
    return k_pages, v_pages, page_stride, page_table


def qk_norm_store(qkv, col0, q_weight, k_weight, eps, pos, tok_slot, kv, n_heads, n_kv_heads, maps, d, dv) -> torch.Tensor:
    """From the float32 rows of a q/k/v product (columns from ``col0``: q [H, maps, d] | k [G, maps, d] | v [G, dv]):
    each map of each q and k head divided by its root mean square over d and multiplied by a weight [d] (``eps``
    None: no norm).  Returns q [T, H, maps * DP] in the cache's type, DP = ``padded_map_dim(d)`` with zeros behind
    a map's d dimensions; k (padded likewise) and v go into the pages in matrix-operand order (csrc/common.h, keys
    of head size maps * DP) at each token's position."""
    _dev(qkv, q_weight, k_weight, pos, tok_slot)
    _f32_rows(qkv, "qk_norm_store rows")
    t = qkv.shape[0]
    kw = maps * padded_map_dim(d)
    _need(col0 >= 0 and col0 + (n_heads + n_kv_heads) * maps * d + n_kv_heads * dv <= qkv.shape[1], "qk_norm_store: columns beyond the rows")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.shape == (d,)), "q/k norm weight: float32 [d]")
    _i32(pos, t, "positions")
    _i32(tok_slot, t, "slots")
    k_pages, v_pages, page_stride, page_table = _map_pages_check(kv, n_kv_heads, kw, dv)
    q = torch.empty((t, n_heads, kw), dtype=k_pages.dtype, device=qkv.device)
    _check(hybrid().li_qk_norm_store(_ptr(qkv), qkv.shape[1], col0, _ptr(q_weight), _ptr(k_weight),
                                     c_float(-1.0 if eps is None else eps), _ptr(pos), _ptr(tok_slot), _ptr(q), _ptr(k_pages),
                                     _ptr(v_pages), c_int64(page_stride), _ptr(page_table), page_table.shape[1],
                                     DT[k_pages.dtype], t, n_heads, n_kv_heads, maps, d, dv, _stream()), "qk_norm_store")
    return q


DIFF_TILE = 32            # tokens of one wave of the matrix-core differential attention
_diffattn: dict = {}


def _diffattn_lib(map_dim: int, value_dim: int):
    lib = _diffattn.get((map_dim, value_dim))
    if lib is None:
        lib = build.diff_attention_library(map_dim, value_dim)
        _need(lib.li_diffattn_map_dim() == map_dim and lib.li_diffattn_value_dim() == value_dim,
              "differential attention library built for other head sizes")
        _diffattn[map_dim, value_dim] = lib
    return lib


def diff_tile_pairs(qlens, lens_before, block, window) -> tuple:
    """The work items of the matrix-core differential attention for sequences that bring ``qlens`` tokens behind
    ``lens_before``: tiles of up to DIFF_TILE consecutive tokens of one sequence, paired so that a tile that sees many
    keys shares a wave with one that sees few.  Returns (first rows, row counts), two entries an item (a missing
    second tile has no rows)."""
    tiles, at = [], 0
    for q, before in zip(qlens, lens_before):
        for lo in range(0, q, DIFF_TILE):
            n = min(DIFF_TILE, q - lo)
            first, last = before + lo, before + lo + n - 1
            start = first - first % block if block else 0
            if window:
                start = max(start, first - window + 1)
            tiles.append((last // 32 - start // 32 + 1, at + lo, n))         # (steps of 32 keys, first row, rows)
        at += q
    tiles.sort(key=lambda t: (-t[0], t[1]))
    t0, n = [], []
    for k in range((len(tiles) + 1) // 2):
        heavy, light = tiles[k], tiles[len(tiles) - 1 - k]
        t0 += [heavy[1], light[1] if light is not heavy else 0]
        n += [heavy[2], light[2] if light is not heavy else 0]
    return t0, n


def diff_tiles(ctx, block=None, window=None):
    """The work items of the matrix-core differential attention for a step (``diff_tile_pairs``) as int32 device
    arrays and their number; made once per step for each (block, window) and shared.  None for a step in which every
    sequence brings one token (every token is then an item of its own)."""
    if ctx.n_tokens == ctx.n_seqs or getattr(ctx, "host_qlens", None) is None:
        return None

    def make():
        t0, n = diff_tile_pairs(ctx.host_qlens, ctx.host_lens_before, int(block or 0), int(window or 0))
        both = torch.tensor([t0, n], dtype=torch.int32).to(ctx.device)
        return both[0], both[1], len(t0) // 2
    return ctx.shared(("diff_attention_tiles", DIFF_TILE, int(block or 0), int(window or 0)), make)


def diff_attention(q, kv, pos, tok_slot, n_heads, n_kv_heads, maps, d, dv, scale, block, window, lam, out_eps, out_scale,
                   out_dtype, tiles=None, sink=None, key_shares: int = 1, slopes=None, gate=None, gate_col: int = 0) -> torch.Tensor:
    """Attention of ``maps`` softmax maps (1 or 2) over the same values: o = a_1 - lam a_2, then (``out_eps`` not
    None) o divided by its root mean square over dv, times ``out_scale``.  A token at position p sees the keys
    from p - p % block on (``block`` 0: from 0; ``window`` w: at most the last w).  q [T, H, maps * DP] as
    ``qk_norm_store`` leaves it; returns [T, H * dv] in ``out_dtype``, the cache's type.  A float32 cache runs one
    workgroup per (token, head); a 16-bit cache runs on the matrix cores, one wave per (pair of tiles, head) with
    ``tiles`` from ``diff_tiles`` for the same block and window (None: every token an item of its own).
    ``sink`` (float32 [H]): every map's sum of weights also counts exp(sink[head]), which has no key and no value.
    ``key_shares`` (a decode step on the matrix cores with four or more query heads on a key/value head): that many
    workgroups share a token's keys, and a second kernel adds up their states in order.
    ``slopes`` (float32 [H]): the score of the key at position j loses slopes[head] * (p - j); the sink loses nothing.
    ``gate`` (float32 rows [T, >= gate_col + H]): head h's output is multiplied by sigmoid(gate[t][gate_col + h])."""
    _dev(q, pos, tok_slot, sink, slopes, gate)
    _need(sink is None or (sink.dtype == torch.float32 and sink.numel() == n_heads), "sink: float32 [H]")
    _need(slopes is None or (slopes.dtype == torch.float32 and slopes.numel() == n_heads and slopes.is_contiguous()), "slopes: float32 [H]")
    _need(gate is None or (gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == q.shape[0] and gate.stride(1) == 1
                           and 0 <= gate_col and gate_col + n_heads <= gate.shape[1]), "gate: float32 rows with a column for every head")
    extra = (_ptr(slopes), _ptr(gate), gate.stride(0) if gate is not None else 0, int(gate_col))
    t = q.shape[0]
    dp = padded_map_dim(d)
    _need(maps in (1, 2) and dv <= 512 and n_heads % n_kv_heads == 0, "diff_attention: one or two maps, values up to 512 wide")
    _i32(pos, t, "positions")
    _i32(tok_slot, t, "slots")
    k_pages, v_pages, page_stride, page_table = _map_pages_check(kv, n_kv_heads, maps * dp, dv)
    _need(q.dtype == k_pages.dtype and q.shape == (t, n_heads, maps * dp), "q: [T, H, maps * DP] in the cache's type")
    _need(out_dtype == k_pages.dtype, "diff_attention: the output has the cache's type")
    out = torch.empty((t, n_heads * dv), dtype=out_dtype, device=q.device)
    tail = (c_float(scale), int(block or 0), int(window or 0), c_float(lam), c_float(-1.0 if out_eps is None else out_eps),
            c_float(out_scale), _ptr(sink), _stream())
    if out_dtype == torch.float32 or not diff_attention_fits(d, dv):
        # (also a 16-bit cache whose sizes the matrix-core kernel does not take)
        _check(hybrid().li_diff_attn(_ptr(q), _ptr(out), DT[out_dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride),
                                     _ptr(page_table), page_table.shape[1], _ptr(pos), _ptr(tok_slot), t, n_heads, n_kv_heads,
                                     maps, d, dv, *tail[:-1], *extra, tail[-1]), "diff_attn")
        return out
    tile_t0, tile_n, n_tiles = tiles if tiles is not None else (None, None, t)
    if tiles is not None:
        _i32(tile_t0, 2 * n_tiles, "tile starts")
        _i32(tile_n, 2 * n_tiles, "tile sizes")
    vd = (dv + 31) // 32 * 32
    part = None
    key_shares = max(1, min(int(key_shares), 64))
    if tiles is None and key_shares > 1 and n_heads // n_kv_heads >= 4:
        part = torch.empty((t, n_heads, key_shares, maps, 2 + vd), dtype=torch.float32, device=q.device)
    _check(_diffattn_lib(dp, vd).li_diffattn(
        _ptr(q), _ptr(out), DT[out_dtype], _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table),
        page_table.shape[1], _ptr(pos), _ptr(tok_slot), _ptr(tile_t0), _ptr(tile_n), n_tiles, n_heads, n_kv_heads, maps, dv,
        *tail[:-1], key_shares if part is not None else 1, _ptr(part), *extra, tail[-1]), "diffattn")
    return out


def diff_attention_fits(d: int, dv: int) -> bool:
    """True if the matrix-core kernel takes a map's keys of size ``d`` and values of size ``dv``."""
    return padded_map_dim(d) <= 256 and (dv + 31) // 32 * 32 <= 256


def small_logits(h, w) -> torch.Tensor:
    """h W^T in float32 for a float32 matrix of a few rows (a router's): every sum in one fixed order."""
    _dev(h, w)
    _need(h.dim() == 2 and h.dtype in DT and w.dtype == torch.float32 and w.dim() == 2 and w.shape[1] == h.shape[1],
          "small_logits: h [T, width], a float32 matrix [n, width]")
    out = torch.empty((h.shape[0], w.shape[0]), dtype=torch.float32, device=h.device)
    _check(hybrid().li_small_logits(_ptr(h), DT[h.dtype], _ptr(w), _ptr(out), h.shape[0], h.shape[1], w.shape[0], _stream()),
           "small_logits")
    return out


def conv_silu(rows, col0, channels, weight, bias, history, ctx) -> torch.Tensor:
    """silu of a causal convolution per channel over ``channels`` columns of the float32 ``rows`` from ``col0`` on;
    weight float32 [channels, taps] (last column: the current token), bias [channels] or None; ``history``
    float32 [slots, taps - 1, channels] holds every sequence's last inputs and is brought up to date."""
    _dev(rows, weight, bias, history)
    _f32_rows(rows, "conv rows")
    t, taps = rows.shape[0], weight.shape[1]
    _need(weight.dtype == torch.float32 and weight.shape == (channels, taps) and 1 <= taps <= 16, "conv weight: float32 [channels, taps <= 16]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (channels,)), "conv bias: float32 [channels]")
    _need(0 <= col0 and col0 + channels <= rows.shape[1], "conv: columns beyond the rows")
    _need(history.dtype == torch.float32 and history.dim() == 3 and tuple(history.shape[1:]) == (max(taps - 1, 1), channels),
          "conv history: float32 [slots, taps - 1, channels]")
    _i32(ctx.pos, t, "positions")
    _i32(ctx.tok_slot, t, "slots")
    _i32(ctx.seq_slot, ctx.n_seqs, "sequence slots")
    qstart, qlen = getattr(ctx, "seq_qstart", None), getattr(ctx, "seq_qlen", None)
    _need((qstart is None) == (qlen is None) and (qstart is not None or t == ctx.n_seqs), "conv: per-sequence starts and lengths")
    out = torch.empty((t, channels), dtype=torch.float32, device=rows.device)
    _check(hybrid().li_conv_silu(_ptr(rows), rows.shape[1], col0, _ptr(weight), _ptr(bias), _ptr(history), _ptr(ctx.pos),
                                 _ptr(ctx.tok_slot), _ptr(ctx.seq_slot), _ptr(qstart), _ptr(qlen), _ptr(out), t, ctx.n_seqs,
                                 channels, taps, _stream()), "conv_silu")
    return out


SSM_SEGMENT = 128          # most tokens of a segment when a prompt's recurrence runs in segments side by side
SSM_WAVES = 3072           # segments are made short enough for about this many waves (three a SIMD)


def ssm_segments(ctx, length: int | None = None) -> dict:
    """The segments of a step's sequences for ``ssm_scan`` (made once per step and shared): every sequence's tokens
    cut every ``length`` tokens; int32 device arrays seg_seq, seg_t0, seg_n, seq_seg0, seq_nseg and the count."""
    length = length or SSM_SEGMENT

    def make():
        seg_seq, seg_t0, seg_n, seq_seg0, seq_nseg = [], [], [], [], []
        for i, n in enumerate(ctx.host_qlens):
            seq_seg0.append(len(seg_seq))
            for t0 in range(0, n, length):
                seg_seq.append(i)
                seg_t0.append(t0)
                seg_n.append(min(length, n - t0))
            seq_nseg.append(len(seg_seq) - seq_seg0[-1])
        k, b = len(seg_seq), len(seq_seg0)
        flat = torch.tensor(seg_seq + seg_t0 + seg_n + seq_seg0 + seq_nseg, dtype=torch.int32).to(ctx.device)
        return {"seg_seq": flat[:k], "seg_t0": flat[k:2 * k], "seg_n": flat[2 * k:3 * k], "seq_seg0": flat[3 * k:3 * k + b],
                "seq_nseg": flat[3 * k + b:], "n": k}
    return ctx.shared(("ssm_segments", length), make)


def ssm_scan(xbc, proj, dt_col, dt_bias, a_log, d_skip, state, ctx, heads, groups, n_state, dv, segments=None) -> torch.Tensor:
    """The selective state-space recurrence in float32.  ``xbc`` float32 [T, heads * dv + 2 groups n_state] (x | B |
    C), the raw step sizes in ``proj`` columns dt_col .. dt_col + heads; ``state`` float32 [slots, heads, n_state,
    dv], read and left up to date; returns y float32 [T, heads * dv].  ``segments`` (``ssm_segments``): the tokens
    run in segments side by side, each twice (first for what it adds to the state, then, from the state before it,
    for y); None: every sequence token by token in order."""
    _dev(xbc, proj, dt_bias, a_log, d_skip, state)
    _f32_rows(xbc, "ssm x/B/C")
    _f32_rows(proj, "ssm projections")
    t = xbc.shape[0]
    _need(heads % groups == 0 and n_state <= 256, "ssm: heads a multiple of groups, a state of up to 256")
    _need(xbc.shape[1] == heads * dv + 2 * groups * n_state and proj.shape[0] == t and dt_col + heads <= proj.shape[1], "ssm: row widths")
    for v in (dt_bias, a_log, d_skip):
        _need(v is None or (v.dtype == torch.float32 and v.shape == (heads,)), "ssm: float32 [heads] vectors")
    _need(dt_bias is not None and a_log is not None, "ssm: dt_bias and A_log")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == (heads, n_state, dv), "ssm state: float32 [slots, heads, N, dv]")
    _i32(ctx.seq_slot, ctx.n_seqs, "sequence slots")
    qstart, qlen = getattr(ctx, "seq_qstart", None), getattr(ctx, "seq_qlen", None)
    _need((qstart is None) == (qlen is None) and (qstart is not None or t == ctx.n_seqs), "ssm: per-sequence starts and lengths")
    y = torch.empty((t, heads * dv), dtype=torch.float32, device=xbc.device)
    if segments is not None:
        _need(qstart is not None, "ssm in segments: per-sequence starts and lengths")
        k = segments["n"]
        for name, n in (("seg_seq", k), ("seg_t0", k), ("seg_n", k), ("seq_seg0", ctx.n_seqs), ("seq_nseg", ctx.n_seqs)):
            _i32(segments[name], n, "ssm " + name)
        seg_state = torch.empty((k, heads, n_state, dv), dtype=torch.float32, device=xbc.device)
        seg_decay = torch.empty((k, heads), dtype=torch.float32, device=xbc.device)
        _check(hybrid().li_ssm_scan_segments(
            _ptr(xbc), xbc.shape[1], _ptr(proj), proj.shape[1], dt_col, _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(state),
            _ptr(ctx.seq_slot), _ptr(qstart), _ptr(qlen), _ptr(y), ctx.n_seqs, heads, groups, n_state, dv,
            _ptr(segments["seg_seq"]), _ptr(segments["seg_t0"]), _ptr(segments["seg_n"]), _ptr(segments["seq_seg0"]),
            _ptr(segments["seq_nseg"]), k, _ptr(seg_state), _ptr(seg_decay), _stream()), "ssm_scan_segments")
        return y
    _check(hybrid().li_ssm_scan(_ptr(xbc), xbc.shape[1], _ptr(proj), proj.shape[1], dt_col, _ptr(dt_bias), _ptr(a_log),
                                _ptr(d_skip), _ptr(state), _ptr(ctx.seq_slot), _ptr(qstart), _ptr(qlen), _ptr(y), ctx.n_seqs,
                                heads, groups, n_state, dv, _stream()), "ssm_scan")
    return y


def gated_group_norm(y, zrows, z_col, weight, groups, eps, out_dtype) -> torch.Tensor:
    """(y * silu(z)) divided, in ``groups`` equal parts of a row, by each part's root mean square, times weight."""
    _dev(y, zrows, weight)
    _f32_rows(y, "gated norm y")
    _f32_rows(zrows, "gated norm z")
    t, n = y.shape
    _need(n % groups == 0 and zrows.shape[0] == t and 0 <= z_col and z_col + n <= zrows.shape[1], "gated norm: sizes")
    _need(weight.dtype == torch.float32 and weight.shape == (n,), "gated norm weight: float32 [n]")
    out = torch.empty((t, n), dtype=out_dtype, device=y.device)
    _check(hybrid().li_gated_group_norm(_ptr(y), _ptr(zrows), zrows.shape[1], z_col, _ptr(weight), _ptr(out), DT[out_dtype],
                                        t, n, groups, c_float(eps), _stream()), "gated_group_norm")
    return out


def moe_route(logits, correction, h, residual, n_route, n_real, top, has_gate, scale, sigmoid_scores: bool = False,
              renorm: bool = True) -> torch.Tensor:
    """Routing weights of every token: softmax over the first ``n_route`` columns of ``logits`` (float32), the ``top``
    largest of score + correction chosen, their scores divided by their sum (+ 1e-20) times ``scale``.  Returns
    float32 [T, n_real (+ 1)]: the weights of the first ``n_real`` outputs (0 where not chosen) and, with
    ``has_gate`` 1, sigmoid of the column behind the router's (2: the constant 1; 0: no such column).  The outputs from ``n_real`` on pass the token on:
    residual[t] += (their weights' sum) * h[t].  ``sigmoid_scores``: the scores are the sigmoid of every output's logit
    instead of the softmax; ``renorm`` False: a chosen output's weight is its own score times ``scale``."""
    _dev(logits, correction, h, residual)
    _f32_rows(logits, "router logits")
    t, width = h.shape
    has_gate = int(has_gate)
    _need(logits.shape[0] == t and logits.shape[1] >= n_route + int(has_gate == 1), "router logits: a row for every token")
    _need(1 <= top <= n_route and 0 <= n_real <= n_route, "router: top within the outputs")
    _need(correction is None or (correction.dtype == torch.float32 and correction.shape == (n_route,)), "router correction: float32 [outputs]")
    _need(h.dtype in DT and residual.dtype == torch.float32 and residual.shape == h.shape, "router: h and the float32 residual rows")
    _drop_row_stats(residual)
    w = torch.empty((t, n_real + int(bool(has_gate))), dtype=torch.float32, device=h.device)
    _check(hybrid().li_moe_route(_ptr(logits), logits.shape[1], _ptr(correction), _ptr(h), DT[h.dtype], _ptr(residual), _ptr(w),
                                 t, width, n_route, n_real, top, has_gate, c_float(scale), int(bool(sigmoid_scores)),
                                 int(bool(renorm)), _stream()), "moe_route")
    return w


def scale_blocks(t, weights, n_blocks, ff, tail) -> torch.Tensor:
    """In place: block e (``ff`` columns) of every row of ``t`` times weights[row][e]; the last ``tail`` columns
    times weights[row][n_blocks]."""
    _dev(t, weights)
    _need(t.dim() == 2 and t.dtype in DT and t.shape[1] == n_blocks * ff + tail, "scale_blocks: [T, blocks * ff + tail]")
    _need(weights.dtype == torch.float32 and weights.shape == (t.shape[0], n_blocks + int(tail > 0)), "scale_blocks: a weight for every block")
    _check(hybrid().li_scale_blocks(_ptr(t), DT[t.dtype], _ptr(weights), t.shape[0], n_blocks, ff, tail, _stream()), "scale_blocks")
    return t


def moe_buckets(weights, n_experts: int):
    """For each of the first ``n_experts`` columns of ``weights`` (float32 [T, cols]) the tokens whose weight is
    not zero, ascending: int32 [n_experts, T] on the device and the counts as a list.  Waits for the device."""
    _dev(weights)
    _need(weights.dtype == torch.float32 and weights.dim() == 2 and weights.shape[1] >= n_experts, "moe_buckets: float32 [T, >= experts]")
    t = weights.shape[0]
    idx = torch.empty((n_experts, t), dtype=torch.int32, device=weights.device)
    counts = torch.empty((n_experts,), dtype=torch.int32, device=weights.device)
    _check(hybrid().li_moe_buckets(_ptr(weights), weights.shape[1], t, n_experts, _ptr(idx), _ptr(counts), _stream()), "moe_buckets")
    return idx, counts.tolist()


def gather_rows(h, idx, n: int) -> torch.Tensor:
    """out[r] = h[idx[r]] for the first ``n`` entries of ``idx`` (int32, contiguous)."""
    _dev(h, idx)
    _need(h.dim() == 2 and h.dtype in DT and idx.dtype == torch.int32 and idx.numel() >= n, "gather_rows: rows and int32 indices")
    out = torch.empty((n, h.shape[1]), dtype=h.dtype, device=h.device)
    _check(hybrid().li_gather_rows(_ptr(h), DT[h.dtype], _ptr(idx), _ptr(out), n, h.shape[1], _stream()), "gather_rows")
    return out


def scatter_add_rows(residual, y, idx, weights, col: int) -> None:
    """residual[idx[r]] += weights[idx[r]][col] * y[r] for every row of ``y`` (``idx`` None: row r itself; ``col`` None:
    the rows are added as they are); no row may be named twice."""
    _dev(residual, y, idx, weights)
    n, width = y.shape
    _need(residual.dtype == torch.float32 and y.dtype == torch.float32 and residual.shape[1] == width, "scatter_add_rows: float32 rows of one width")
    col = -1 if col is None else col
    _need(weights.dtype == torch.float32 and weights.dim() == 2 and weights.shape[0] == residual.shape[0] and -1 <= col < weights.shape[1],
          "scatter_add_rows: a weight for every row of the residual")
    _need(idx is None and n == residual.shape[0] or idx is not None and idx.dtype == torch.int32 and idx.numel() >= n,
          "scatter_add_rows: int32 indices for every row of y")
    _drop_row_stats(residual)
    _check(hybrid().li_scatter_add_rows(_ptr(residual), _ptr(y), _ptr(idx), _ptr(weights), weights.shape[1], col, n, width,
                                        _stream()), "scatter_add_rows")


def copy_rows(x: torch.Tensor) -> torch.Tensor:
    """A copy of ``x`` in memory of its own (one device-to-device copy on the current stream)."""
    return x.clone()


# ---------------------------------------------------------------------------
# latent attention, the matrix-memory recurrence, a bigram embedding, the depth-weighted residual stream
# (csrc/latent.hip, in the hybrid library)
# ---------------------------------------------------------------------------
def _seq_arrays(ctx, n_tokens):
    """(seq_slot, seq_qstart, seq_qlen) of a step; the last two None for a step of one token a sequence."""
    _i32(ctx.seq_slot, ctx.n_seqs, "sequence slots")
    qstart, qlen = getattr(ctx, "seq_qstart", None), getattr(ctx, "seq_qlen", None)
    _need((qstart is None) == (qlen is None) and (qstart is not None or n_tokens == ctx.n_seqs),
          "per-sequence starts and lengths, or one token a sequence")
    return ctx.seq_slot, qstart, qlen


def embed_bigram(table, bigram, ctx, prev_state, scale: float, mul_prev: int, mul_cur: int, out=None) -> torch.Tensor:
    """x[t] = table[token] * scale + bigram[(previous token * mul_prev + token * mul_cur) mod buckets], buckets =
    rows of ``bigram`` - 1; a sequence's first token takes the last row.  ``prev_state`` int32 [slots]: the token
    before the first one that a sequence brings to this step; left at the sequence's last token of the step."""
    _dev(table, bigram, prev_state, out)
    n, (vocab, d) = ctx.n_tokens, table.shape
    _need(table.dim() == 2 and bigram.dim() == 2 and bigram.shape[1] == d and bigram.shape[0] >= 2 and table.dtype == bigram.dtype
          and table.dtype in DT, "embed_bigram: two float tables of one width and type")
    _i32(ctx.token_ids, n, "tokens")
    _i32(ctx.pos, n, "positions")
    _i32(ctx.tok_slot, n, "slots")
    _need(prev_state.dtype == torch.int32 and prev_state.dim() == 1, "embed_bigram: int32 [slots] previous tokens")
    seq_slot, qstart, qlen = _seq_arrays(ctx, n)
    if out is None:
        out = torch.empty((n, d), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (n, d), "embed_bigram out: float32 [T, d]")
    _drop_row_stats(out)
    _check(hybrid().li_embed_bigram(_ptr(table), _ptr(bigram), DT[table.dtype], _ptr(ctx.token_ids), _ptr(ctx.pos),
                                    _ptr(ctx.tok_slot), _ptr(seq_slot), _ptr(qstart), _ptr(qlen), _ptr(prev_state), _ptr(out), n,
                                    ctx.n_seqs, d, c_float(scale), c_int64(mul_prev), c_int64(mul_cur), bigram.shape[0] - 1,
                                    _stream()), "embed_bigram")
    return out


def depth_average(history: torch.Tensor, n: int, weights: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = sum over j < n of weights[j] * history[j]; ``history`` float32 [runs, T, width], ``out`` float32 [T, width]
    (it may be a later row of ``history``)."""
    _dev(history, weights, out)
    _need(history.dtype == torch.float32 and history.dim() == 3 and 1 <= n <= history.shape[0], "depth_average: float32 [runs, T, width]")
    _need(weights.dtype == torch.float32 and weights.numel() >= n, "depth_average: a float32 weight for every term")
    _need(out.dtype == torch.float32 and tuple(out.shape) == tuple(history.shape[1:]), "depth_average out: float32 [T, width]")
    _drop_row_stats(out)
    _check(hybrid().li_depth_average(_ptr(history), c_int64(history.stride(0)), _ptr(weights), n, _ptr(out), c_int64(out.numel()),
                                     _stream()), "depth_average")
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap) in place (float32)."""
    _dev(x)
    _need(x.dtype == torch.float32 and cap > 0, "softcap: float32 values, a positive cap")
    _check(hybrid().li_softcap(_ptr(x), c_int64(x.numel()), c_float(cap), _stream()), "softcap")
    return x


def conv_add(rows, weight, history, ctx, out_dtype) -> torch.Tensor:
    """u + conv(u) for the float32 ``rows`` u [T, channels]: a causal convolution per channel over time, weight
    float32 [channels, taps] (last column: the current token), no bias, no activation; ``history`` float32
    [slots, taps - 1, channels] holds every sequence's last inputs and is brought up to date.  Returns ``out_dtype``."""
    _dev(rows, weight, history)
    _f32_rows(rows, "conv rows")
    t, channels = rows.shape
    taps = weight.shape[1]
    _need(weight.dtype == torch.float32 and weight.shape == (channels, taps) and 1 <= taps <= 16, "conv weight: float32 [channels, taps <= 16]")
    _need(history.dtype == torch.float32 and history.dim() == 3 and tuple(history.shape[1:]) == (max(taps - 1, 1), channels),
          "conv history: float32 [slots, taps - 1, channels]")
    _i32(ctx.pos, t, "positions")
    _i32(ctx.tok_slot, t, "slots")
    seq_slot, qstart, qlen = _seq_arrays(ctx, t)
    out = torch.empty((t, channels), dtype=out_dtype, device=rows.device)
    _check(hybrid().li_conv_add(_ptr(rows), channels, 0, _ptr(weight), None, _ptr(history), _ptr(ctx.pos), _ptr(ctx.tok_slot),
                                _ptr(seq_slot), _ptr(qstart), _ptr(qlen), _ptr(out), DT[out_dtype], t, ctx.n_seqs, channels, taps,
                                _stream()), "conv_add")
    return out


def latent_store(proj, q_col, kv_col, norm_weight, eps, inv_freq, rot, pos, tok_slot, kv, n_heads, d, rd, r) -> torch.Tensor:
    """From the float32 rows of latent attention's input product (from column ``q_col`` every head's [d unrotated | rd
    rotated] query dimensions, from ``kv_col`` [latent r | rotated key part rd]): the latent divided by its root mean
    square, times ``norm_weight`` [r]; the rotated parts turned by position (the first ``rot`` of their rd dimensions
    in pairs (2i, 2i + 1), angle pos * inv_freq[i]); the key [latent | rotated part] (zeros up to the next multiple
    of 16) and the value (the latent) into the pages.  Returns q [T, H, KW] in the cache's type with every head's
    rotated part from column r on; the first r columns are left for ``head_linear``."""
    _dev(proj, norm_weight, inv_freq, pos, tok_slot)
    _f32_rows(proj, "latent_store rows")
    t = proj.shape[0]
    kw = padded_map_dim(r + rd)
    _need(q_col >= 0 and kv_col >= 0 and max(q_col + n_heads * (d + rd), kv_col + r + rd) <= proj.shape[1], "latent_store: columns beyond the rows")
    _need(norm_weight.dtype == torch.float32 and norm_weight.shape == (r,), "latent norm weight: float32 [r]")
    _need(0 <= rot <= rd and rot % 2 == 0, "latent_store: an even number of rotated dimensions within rd")
    if rot:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() >= rot // 2, "inv_freq: float32 [rot / 2]")
    _i32(pos, t, "positions")
    _i32(tok_slot, t, "slots")
    k_pages, v_pages, page_stride, page_table = _map_pages_check(kv, 1, kw, r)
    q = torch.empty((t, n_heads, kw), dtype=k_pages.dtype, device=proj.device)
    _check(hybrid().li_latent_store(_ptr(proj), proj.shape[1], q_col, kv_col, _ptr(norm_weight), c_float(eps), _ptr(inv_freq), rot,
                                    _ptr(pos), _ptr(tok_slot), _ptr(q), _ptr(k_pages), _ptr(v_pages), c_int64(page_stride),
                                    _ptr(page_table), page_table.shape[1], DT[k_pages.dtype], t, n_heads, d, rd, r, _stream()),
           "latent_store")
    return q


def head_linear(x, x_col, x_head_stride, w, out, out_col, out_head_stride, gate=None, gate_col=0) -> torch.Tensor:
    """A product per head: out[t, out_col + h * out_head_stride + j] = sum over i of w[h, j, i] * x[t, x_col + h *
    x_head_stride + i], ``w`` [H, n_out, n_in] in the model's type (a 16-bit model runs it on the matrix cores, a float32
    input as the sum of two 16-bit numbers), ``x`` [T, ...] float32 or of that type, ``out``
    [T, ...] of that type (both may be wider rows in which a head's part lies).  ``gate`` (float32 rows): the result
    is multiplied by sigmoid(gate[t, gate_col + h * n_out + j]).  Sums are float32."""
    _dev(x, w, out, gate)
    x2, o2 = x.view(x.shape[0], -1), out.view(out.shape[0], -1)
    t = x2.shape[0]
    _need(w.dim() == 3 and w.dtype in DT and x2.dtype in (torch.float32, w.dtype) and o2.dtype == w.dtype and o2.shape[0] == t,
          "head_linear: weights [H, n_out, n_in], rows of their type (or float32 in)")
    H, n_out, n_in = w.shape
    _need(x_col >= 0 and x_col + (H - 1) * x_head_stride + n_in <= x2.shape[1], "head_linear: input columns beyond the rows")
    _need(out_col >= 0 and out_col + (H - 1) * out_head_stride + n_out <= o2.shape[1], "head_linear: output columns beyond the rows")
    if gate is not None:
        _f32_rows(gate, "head_linear gate")
        _need(gate.shape[0] == t and gate_col >= 0 and gate_col + H * n_out <= gate.shape[1], "head_linear: gate columns beyond the rows")
    _need(n_in <= 960, "head_linear: up to 960 inputs a head")
    _drop_row_stats(out)
    _check(hybrid().li_head_linear(c_void_p(x2.data_ptr() + x_col * x2.element_size()), DT[x2.dtype], c_int64(x2.shape[1]),
                                   x_head_stride, _ptr(w), DT[w.dtype], c_void_p(o2.data_ptr() + out_col * o2.element_size()),
                                   c_int64(o2.shape[1]), out_head_stride,
                                   c_void_p(gate.data_ptr() + 4 * gate_col) if gate is not None else None,
                                   c_int64(gate.shape[1] if gate is not None else 0), t, H, n_in, n_out, _stream()), "head_linear")
    return out


def mlstm_scan(proj, q_col, k_col, v_col, i_col, f_col, i_bias, f_bias, cap, q_scale, state, norm_state, ctx, heads, d, dv,
               segments=None) -> torch.Tensor:
    """The matrix-memory recurrence in float32 over the tokens of a step.  q, k [heads, d], v [heads, dv] and the two raw
    gates [heads] are columns of the float32 rows ``proj``; with i = cap tanh((gi + i_bias) / cap), f = logsigmoid(cap
    tanh((gf + f_bias) / cap)):  m <- max(f + m, i);  S <- exp(f + m_old - m) S + exp(i - m) k v^T, n likewise with k;
    y = S^T q / (max(|n . q|, exp(-m)) + 1e-6), q times ``q_scale``.  ``state`` float32 [slots, heads, d, dv] and
    ``norm_state`` float32 [slots, heads, d + 1] (n, then m) are read and left up to date.  ``segments``
    (``ssm_segments``): the tokens run in segments side by side, each twice (first for what it adds to the state, then,
    from the state before it, for y); None: every sequence token by token in order.  Returns y float32 [T, heads * dv]."""
    _dev(proj, i_bias, f_bias, state, norm_state)
    _f32_rows(proj, "mlstm projections")
    t = proj.shape[0]
    _need(1 <= d <= 256 and dv >= 1 and cap > 0, "mlstm: keys up to 256 wide, a positive cap")
    _need(max(q_col + heads * d, k_col + heads * d, v_col + heads * dv, i_col + heads, f_col + heads) <= proj.shape[1]
          and min(q_col, k_col, v_col, i_col, f_col) >= 0, "mlstm: columns beyond the rows")
    for b in (i_bias, f_bias):
        _need(b is None or (b.dtype == torch.float32 and b.shape == (heads,)), "mlstm: float32 [heads] gate biases")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == (heads, d, dv), "mlstm state: float32 [slots, heads, d, dv]")
    _need(norm_state.dtype == torch.float32 and tuple(norm_state.shape[1:]) == (heads, d + 1) and norm_state.shape[0] == state.shape[0],
          "mlstm normaliser state: float32 [slots, heads, d + 1]")
    seq_slot, qstart, qlen = _seq_arrays(ctx, t)
    dev = proj.device
    # (keys more than 128 wide: two waves share a head's rows and add their halves of y)
    y = (torch.zeros if d > 128 else torch.empty)((t, heads * dv), dtype=torch.float32, device=dev)
    coef = torch.empty((t, heads, 3), dtype=torch.float32, device=dev)
    fresh = seg = None
    if segments is None:
        fresh = torch.empty((ctx.n_seqs, heads, d + 1), dtype=torch.float32, device=dev)
        tail = (None, None, None, None, None, 0, None, None, None)
    else:
        _need(qstart is not None, "mlstm in segments: per-sequence starts and lengths")
        k = segments["n"]
        for name, n in (("seg_seq", k), ("seg_t0", k), ("seg_n", k), ("seq_seg0", ctx.n_seqs), ("seq_nseg", ctx.n_seqs)):
            _i32(segments[name], n, "mlstm " + name)
        seg = (torch.empty((k, heads, d, dv), dtype=torch.float32, device=dev), torch.empty((k, heads, d), dtype=torch.float32, device=dev),
               torch.empty((k, heads), dtype=torch.float32, device=dev))
        tail = (_ptr(segments["seg_seq"]), _ptr(segments["seg_t0"]), _ptr(segments["seg_n"]), _ptr(segments["seq_seg0"]),
                _ptr(segments["seq_nseg"]), k, _ptr(seg[0]), _ptr(seg[1]), _ptr(seg[2]))
    _check(hybrid().li_mlstm_scan(_ptr(proj), proj.shape[1], q_col, k_col, v_col, i_col, f_col, _ptr(i_bias), _ptr(f_bias),
                                  c_float(cap), c_float(q_scale), _ptr(state), _ptr(norm_state), _ptr(fresh), _ptr(coef),
                                  _ptr(seq_slot), _ptr(qstart), _ptr(qlen), _ptr(y), t, ctx.n_seqs, heads, d, dv, *tail, _stream()),
           "mlstm_scan")
    return y


def gated_head_norm(y, weight, gate_rows, gate_col, heads, eps, out_dtype) -> torch.Tensor:
    """Every head's part of a float32 row [heads * dv] divided by its own root mean square, then times ``weight``
    [heads * dv] (None: none) and sigmoid of columns gate_col .. of the float32 ``gate_rows`` (None: no gate)."""
    _dev(y, weight, gate_rows)
    _f32_rows(y, "head norm rows")
    t, n = y.shape
    _need(heads >= 1 and n % heads == 0, "head norm: equal heads")
    _need(weight is None or (weight.dtype == torch.float32 and weight.shape == (n,)), "head norm weight: float32 [heads * dv]")
    if gate_rows is not None:
        _f32_rows(gate_rows, "head norm gate")
        _need(gate_rows.shape[0] == t and gate_col >= 0 and gate_col + n <= gate_rows.shape[1], "head norm: gate columns beyond the rows")
    out = torch.empty((t, n), dtype=out_dtype, device=y.device)
    _check(hybrid().li_gated_head_norm(_ptr(y), _ptr(weight),
                                       c_void_p(gate_rows.data_ptr() + 4 * gate_col) if gate_rows is not None else None,
                                       c_int64(gate_rows.shape[1] if gate_rows is not None else 0), _ptr(out), DT[out_dtype], t,
                                       heads, n // heads, c_float(eps), _stream()), "gated_head_norm")
    return out


def expert_act(z, weights, n_blocks, ff, tail, kind: str, on_input: bool, out_dtype, idx=None, col=None) -> torch.Tensor:
    """The hidden rows of experts side by side (``z`` float32 [rows, n_blocks * ff + tail], the sums of the up
    products) through the activation ``kind`` with the routing weight: block e of row r takes weights[r][e], the
    tail weights[r][n_blocks]; ``idx`` (int32): row r of ``z`` is token idx[r]; ``col``: every block takes that
    column (the rows of one expert).  ``on_input``: act(weight * z), the weight on the expert's input; else weight *
    act(z).  ``weights`` None: the plain activation."""
    _dev(z, weights, idx)
    _f32_rows(z, "expert rows")
    rows = z.shape[0]
    _need(kind in ACTIVATIONS and z.shape[1] == n_blocks * ff + tail, "expert_act: [rows, blocks * ff + tail], a known activation")
    wcols = 0
    if weights is not None:
        _need(weights.dtype == torch.float32 and weights.dim() == 2, "expert_act: float32 weights [tokens, columns]")
        wcols = weights.shape[1]
        _need(wcols >= (n_blocks + int(tail > 0) if col is None else col + 1), "expert_act: a weight for every block")
        if idx is None:
            _need(weights.shape[0] == rows, "expert_act: a row of weights for every row")
        else:
            _i32(idx, rows, "expert_act rows' tokens")
    out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
    _check(hybrid().li_expert_act(_ptr(z), _ptr(weights), wcols, _ptr(idx), -1 if col is None else col, _ptr(out), DT[out_dtype],
                                  rows, n_blocks, ff, tail, ACTIVATIONS[kind], int(bool(on_input)), _stream()), "expert_act")
    return out


# ---------------------------------------------------------------------------
# sub-layers between two norms, softmax attention with a sink, a gate a head and a rotation of half-paired dimensions
# or a bias by distance, clamped gated feed-forwards, experts by table (csrc/gated.hip, in the hybrid library)
# ---------------------------------------------------------------------------
def add_bias(rows, col0: int, bias) -> torch.Tensor:
    """rows[:, col0 : col0 + len(bias)] += bias, in place (float32 rows)."""
    _dev(rows, bias)
    _f32_rows(rows, "add_bias rows")
    _need(bias.dtype == torch.float32 and bias.dim() == 1 and bias.is_contiguous() and 0 <= col0 and col0 + bias.numel() <= rows.shape[1],
          "add_bias: a float32 vector within the rows")
    _drop_row_stats(rows)
    _check(hybrid().li_add_bias(_ptr(rows), rows.shape[1], col0, _ptr(bias), rows.shape[0], bias.numel(), _stream()), "add_bias")
    return rows


def scale_values(x: torch.Tensor, s: float) -> torch.Tensor:
    """x <- x * s in place (float32, contiguous)."""
    _dev(x)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "scale_values: contiguous float32 values")
    _check(hybrid().li_scale_values(_ptr(x), c_int64(x.numel()), c_float(s), _stream()), "scale_values")
    return x


def conv_history(rows, col0, channels, taps, history, ctx) -> None:
    """Brings ``history`` (float32 [slots, taps - 1, channels]: every sequence's last inputs of a causal convolution) up
    to date with the step's ``rows`` (float32, the channels from column ``col0`` on); for a kernel that convolves on the
    way to something else and only reads the history."""
    _dev(rows, history)
    _f32_rows(rows, "conv rows")
    _need(1 <= taps <= 16 and 0 <= col0 and col0 + channels <= rows.shape[1], "conv history: columns within the rows, up to 16 taps")
    _need(history.dtype == torch.float32 and history.dim() == 3 and tuple(history.shape[1:]) == (max(taps - 1, 1), channels),
          "conv history: float32 [slots, taps - 1, channels]")
    seq_slot, qstart, qlen = _seq_arrays(ctx, rows.shape[0])
    _check(hybrid().li_conv_history(_ptr(rows), rows.shape[1], col0, _ptr(history), _ptr(seq_slot), _ptr(qstart), _ptr(qlen),
                                    ctx.n_seqs, channels, taps, _stream()), "conv_history")


def rot_store(rows, q_col, k_col, v_col, inv_freq, rot, pos, tok_slot, kv, n_heads, n_kv_store, d, dv, q_dtype=None,
              conv=None) -> torch.Tensor:
    """From float32 rows with a token's q heads [H, d] from column ``q_col``, k heads [G, d] from ``k_col`` and values
    [G, dv] from ``v_col`` (it may equal ``k_col``: the values are the keys before their rotation): q and k turned by
    position in their first ``rot`` dimensions, dimension i paired with i + rot / 2, angle pos * inv_freq[i]; k and v
    into the pages in matrix-operand order (one map of keys, padded to a multiple of 16).  ``n_kv_store`` 0: nothing
    is stored (``kv`` may be None, ``q_dtype`` says q's type).  ``conv`` (weight float32 [channels, taps], history float32
    [slots, taps - 1, channels]): column c of the rows is channel c of a causal convolution over time that everything
    read passes first (the last tap is the token's own; inputs before the step's first token of a sequence come from
    the history, which is only read: ``conv_history`` brings it up to date afterwards).  Returns q [T, H, DP] in the
    cache's type."""
    _dev(rows, inv_freq, pos, tok_slot)
    _f32_rows(rows, "rot_store rows")
    t = rows.shape[0]
    dp = padded_map_dim(d)
    _need(0 <= rot <= d and rot % 2 == 0, "rot_store: an even number of rotated dimensions within the head")
    if rot:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() >= rot // 2, "inv_freq: float32 [rot / 2]")
    _need(q_col >= 0 and q_col + n_heads * d <= rows.shape[1], "rot_store: q columns beyond the rows")
    _i32(pos, t, "positions")
    _i32(tok_slot, t, "slots")
    if n_kv_store:
        _need(min(k_col, v_col) >= 0 and k_col + n_kv_store * d <= rows.shape[1] and v_col + n_kv_store * dv <= rows.shape[1],
              "rot_store: k or v columns beyond the rows")
        k_pages, v_pages, page_stride, page_table = _map_pages_check(kv, n_kv_store, dp, dv)
        q_dtype, max_pages = k_pages.dtype, page_table.shape[1]
    else:
        k_pages = v_pages = page_table = None
        page_stride = max_pages = 0
        _need(q_dtype in DT, "rot_store: q's type")
    conv_w = hist = None
    taps = channels = 0
    if conv is not None:
        conv_w, hist = conv
        _dev(conv_w, hist)
        channels, taps = conv_w.shape
        _need(conv_w.dtype == torch.float32 and conv_w.is_contiguous() and 1 <= taps <= 16 and channels <= rows.shape[1],
              "rot_store: conv weight float32 [channels, taps <= 16] for the first columns of the rows")
        _need(hist.dtype == torch.float32 and hist.dim() == 3 and tuple(hist.shape[1:]) == (max(taps - 1, 1), channels),
              "rot_store: conv history float32 [slots, taps - 1, channels]")
    q = torch.empty((t, n_heads, dp), dtype=q_dtype, device=rows.device)
    _check(hybrid().li_rot_store(_ptr(rows), rows.shape[1], q_col, k_col, v_col, _ptr(inv_freq), rot, _ptr(pos), _ptr(tok_slot),
                                 _ptr(q), _ptr(k_pages), _ptr(v_pages), c_int64(page_stride), _ptr(page_table), max_pages,
                                 DT[q_dtype], t, n_heads, n_kv_store, d, dv, _ptr(conv_w), taps, _ptr(hist), channels,
                                 _stream()), "rot_store")
    return q


def rmsnorm_add(x, y, weight, eps: float, bias=None, next_norm=None) -> torch.Tensor:
    """x += (y + bias) / sqrt(mean((y + bias)^2) + eps) * weight, row by row, in place (all float32).  ``next_norm``
    (weight float32 [width], eps, dtype): the RMS norm that reads the finished rows next is taken in the same pass and
    left for it (``prepared_rmsnorm`` finds it as long as nothing else writes into ``x``)."""
    _dev(x, y, weight, bias)
    _f32_rows(x, "rmsnorm_add x")
    _f32_rows(y, "rmsnorm_add y")
    width = x.shape[1]
    _need(y.shape == x.shape and weight.dtype == torch.float32 and weight.shape == (width,), "rmsnorm_add: rows of one shape, a float32 weight")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (width,)), "rmsnorm_add: a float32 bias")
    _drop_row_stats(x)
    nw = normed = None
    n_eps, n_dt = 0.0, torch.float32
    if next_norm is not None:
        nw, n_eps, n_dt = next_norm
        _dev(nw)
        _need(nw.dtype == torch.float32 and nw.shape == (width,) and n_dt in DT, "rmsnorm_add: the next norm's float32 weight and type")
        normed = torch.empty(x.shape, dtype=n_dt, device=x.device)
    _check(hybrid().li_rmsnorm_add(_ptr(x), _ptr(y), _ptr(bias), _ptr(weight), c_float(eps), x.shape[0], width, _ptr(nw),
                                   c_float(n_eps), _ptr(normed), DT[n_dt], _stream()), "rmsnorm_add")
    if normed is not None:
        x._li_normed = (normed, nw, float(n_eps), x._version)
    return x


def table_route(token_ids, table, n_experts: int, gate_logits=None, has_gate: int = 0) -> torch.Tensor:
    """Routing weights of experts that a table assigns: row ``table[token]`` (int32 [vocab, top]) names a token's experts,
    each of weight 1 / top.  Returns float32 [T, n_experts (+ 1)], 0 where not named; ``has_gate`` 1: the last column is
    sigmoid(gate_logits[t]) (float32 [T]), 2: it is 1."""
    _dev(token_ids, table, gate_logits)
    t = token_ids.shape[0]
    _i32(token_ids, t, "token ids")
    _need(table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous() and 1 <= table.shape[1] <= n_experts,
          "table_route: int32 [vocab, top]")
    _need(has_gate != 1 or (gate_logits is not None and gate_logits.dtype == torch.float32 and gate_logits.numel() == t
                            and gate_logits.is_contiguous()), "table_route: a float32 gate logit for every token")
    w = torch.empty((t, n_experts + int(bool(has_gate))), dtype=torch.float32, device=token_ids.device)
    _check(hybrid().li_table_route(_ptr(token_ids), _ptr(table), table.shape[1], n_experts, _ptr(gate_logits), int(has_gate),
                                   _ptr(w), t, _stream()), "table_route")
    return w
