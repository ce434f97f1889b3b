"""The kernels as Python functions over torch tensors that live on the GPU.

Every function here launches hand-written gfx950 code from ``liblucciola_hip.so`` on the
current HIP stream; there is no other implementation behind these names.  Loading fails loudly
if the library cannot be built or opened.  Parts call these through the module
(``ops.gemm(...)``), never by importing the names.
"""
from __future__ import annotations

import ctypes
import heapq
import threading
from dataclasses import dataclass, replace
from typing import Optional

import numpy as np
import torch

from ..csrc import build as _build

_lib = None

DT_F32, DT_BF16 = 0, 1

# argument kinds: p pointer, i int, f float
_ARG = {"p": ctypes.c_void_p, "i": ctypes.c_int, "f": ctypes.c_float, "q": ctypes.c_longlong}
_SIGNATURES = {
    "lc_embedding": "ppipiiifp",
    "lc_rmsnorm": "ppppfpiiiipiip",
    "lc_rmsnorm_act": "ppfpiiip",
    "lc_gemm_generic": "pipipiiiipp",
    "lc_gemm_bf16": "pppiiiiipp",
    "lc_gemm_bf16_supported": "iii",
    "lc_gemm_bf16_kblock": "",
    "lc_gemm_bf16_force_tile": "i",
    "lc_gemm_bf16_force_skinny": "i",
    "lc_gemm_bf16_even_rows": "i",
    "lc_gemm_bf16_runs": "i",
    "lc_gemm_bf16_small_partials": "i",
    "lc_gemm_bf16_force_shares": "i",
    "lc_gemm_bf16_skew": "i",
    "lc_gemm_bf16_residual_pieces": "iii",
    "lc_gemm_bf16_piece_stride": "i",
    "lc_gemm_bf16_shares": "iii",
    "lc_gemm_bf16_tile": "iiii",
    "lc_gemm_bf16_partials": "pppiiip",
    "lc_gemm_bf16_residual": "ppppppiiip",
    "lc_gemm_bf16_scaled_rows": "pppiiiipifp",
    "lc_gemm_bf16_scaled_rows_supported": "iii",
    "lc_qk_norm_rope_write": "piiiiippfppipppiip",
    "lc_attention_generic": "pipppipppiiiiiifipp",
    "lc_attention_generic_rows": "i",
    "lc_attn_bf16_supported": "iiii",
    "lc_attn_page_granule": "",
    "lc_gemm_bf16_runs_ring_ok": "",
    "lc_attn_decode_splits": "iii",
    "lc_attn_decode_waves": "i",
    "lc_attn_decode_deep": "i",
    "lc_attn_decode_deep_ok": "i",
    "lc_attn_decode_by_items": "iiiq",
    "lc_attn_decode_force_splits": "i",
    "lc_attn_decode_bf16": "pipppppppip" + "iiiiii" + "f" + "iii" + "ippfpii" + "pii" + "p",
    "lc_attn_decode_takes_shares": "ii",
    "lc_gemm_bf16_sum_shares": "ppiiiip",
    "lc_attn_prefill_bf16": "pippppp" + "iiiiii" + "f" + "i" + "ipfpi" + "ipp" + "p",
    "lc_attn_prefill_splits": "iiii",
    "lc_attn_prefill_wide": "i",
    "lc_attn_prefill_prepares_q": "ii",
    "lc_swiglu": "ppiiip",
    "lc_sample": "pppppiip",
    "lc_sample_workspace": "i",
    "lc_feed_tokens": "pppiip",
}


class KernelError(RuntimeError):
    pass


def register_signatures(signatures) -> None:
    """Entry points of the kernel library beyond the ones listed above, ``{name: kinds}`` with one
    letter per argument (p pointer, i int, q 64-bit int, f float; they return an int, 0 for success): a part
    that brings kernels of its own (a source file added to ``csrc``) declares them here and
    launches them with :func:`call`; no table in this file has to know them."""
    for name, kinds in signatures.items():
        bad = [c for c in kinds if c not in _ARG]
        if bad:
            raise KernelError(f"entry point {name}: unknown argument kinds {bad} (p, i, q or f)")
        if _SIGNATURES.get(name, kinds) != kinds:
            raise KernelError(f"entry point {name} is already declared as '{_SIGNATURES[name]}'")
        if _lib is not None:
            _declare(_lib, name, kinds)
        _SIGNATURES[name] = kinds


def _declare(lib, name: str, kinds: str) -> None:
    fn = getattr(lib, name, None)
    if fn is None:
        raise KernelError(f"the kernel library lacks the entry point {name}")
    fn.restype = ctypes.c_int
    fn.argtypes = [_ARG[c] for c in kinds]


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DT_F32
    if t.dtype == torch.bfloat16:
        return DT_BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


def library():
    """The loaded kernel library (built at the first call if there is no current build)."""
    global _lib
    if _lib is None:
        path = _build.library_path(build_if_needed=True)
        try:
            lib = ctypes.CDLL(path)
        except OSError as exc:
            raise KernelError(f"cannot load the kernel library {path}: {exc}") from exc
        lib.lc_last_error.restype = ctypes.c_char_p
        lib.lc_gemm_bf16_workspace.restype = ctypes.c_longlong
        lib.lc_gemm_bf16_workspace.argtypes = [ctypes.c_int] * 3
        lib.lc_gemm_generic_workspace.restype = ctypes.c_longlong
        lib.lc_gemm_generic_workspace.argtypes = [ctypes.c_int] * 3
        lib.lc_attention_generic_workspace.restype = ctypes.c_longlong
        lib.lc_attention_generic_workspace.argtypes = [ctypes.c_int] * 5
        for name, sig in _SIGNATURES.items():
            _declare(lib, name, sig)
        if lib.lc_attn_page_granule() != ATTENTION_PAGE_GRANULE:
            raise KernelError(f"the attention kernels of {path} are built for pages of "
                              f"{lib.lc_attn_page_granule()} tokens, this module for {ATTENTION_PAGE_GRANULE}")
        _lib = lib
    return _lib


def library_file() -> str:
    library()
    return _build.library_path(build_if_needed=False)


def _call(name: str, *args) -> None:
    lib = library()
    fn = getattr(lib, name)
    rc = fn(*args)
    if rc != 0:
        raise KernelError(lib.lc_last_error().decode("utf-8", "replace"))


def call(name: str, *args) -> None:
    """Launch a declared entry point (see :func:`register_signatures`); raises KernelError with
    the library's message if it reports a failure.  ``ptr(tensor)`` and ``stream()`` make the
    pointer and stream arguments."""
    _call(name, *args)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    if t is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


# torch's own fast path to the current stream's handle (what its compiled kernels use); the
# public route builds a Stream object per call, a third of the host's time in an eager step
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> ctypes.c_void_p:
    if _raw_stream is not None and _raw_device is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t: torch.Tensor, what: str, dtype=None, dim: Optional[int] = None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{what}: tensor must be on the GPU (is on {t.device})")
    if not t.is_contiguous():
        raise KernelError(f"{what}: tensor must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{what}: expected {dtype}, got {t.dtype}")
    if dim is not None and t.dim() != dim:
        raise KernelError(f"{what}: expected {dim} dimensions, got shape {tuple(t.shape)}")


ptr, stream = _ptr, _stream       # public names, for parts that bring kernels of their own

_c_int, _c_float = ctypes.c_int, ctypes.c_float

_said = set()


def _say_once(key, message: str) -> None:
    """A line on stderr the first time a slow path is taken for these sizes."""
    if key not in _said:
        _said.add(key)
        import sys
        print(f"[lucciola_amd] {message}", file=sys.stderr, flush=True)


# ------------------------------------------------------------------------------ embedding
def embedding(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, H] rows of ``table`` [V, H] picked by int32 ``ids`` [T], times ``scale``."""
    _need(ids, "embedding ids", torch.int32, 1)
    _need(table, "embedding table", None, 2)
    T, (V, H) = ids.shape[0], table.shape
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _call("lc_embedding", _ptr(ids), _ptr(table), _c_int(_dt(table)), _ptr(out), _c_int(T),
          _c_int(H), _c_int(V), _c_float(scale), _stream())
    return out


# ------------------------------------------------------------------------------ norms
# Steps of up to 16 rows (decode) are bound by the number of kernels they start.  There the
# norm between two products need not be a kernel of its own: the product before it can add its
# result to the residual stream and leave the sums of squares (a PendingProduct completed by
# ``rmsnorm(..., scaled=True)``), and the product after it can apply the rows' factors to its
# sums (it is given ScaledRows).  Both are only ever handed to code that asks for them; anyone
# else gets tensors.
@dataclass
class PendingProduct:
    """``x . w^T`` that has not been computed yet: a branch's last product, waiting to be
    added to the residual stream by the kernel that computes it."""

    x: torch.Tensor
    w: torch.Tensor
    out_dtype: torch.dtype

    def value(self) -> torch.Tensor:
        return gemm(self.x, self.w, self.out_dtype)


@dataclass
class ScaledRows:
    """The normed residual stream short of each row's factor: ``x`` = bf16(h * weight) [T, n];
    ``pieces`` [count, T rounded up to a power of two] float32 hold pieces of the rows' sums of
    squares (row t at [piece, t]); the factor of row t is rsqrt(sum of its pieces / n + eps)."""

    x: torch.Tensor
    pieces: torch.Tensor
    count: int
    eps: float
    h: torch.Tensor            # the stream and the weight, for whoever needs the rows themselves
    weight: torch.Tensor

    def value(self) -> torch.Tensor:
        return rmsnorm(self.h, None, self.weight, self.eps, self.x.dtype)


@dataclass
class ProductShares:
    """``x . w^T`` as the float32 shares [S, M, N] of a product that was cut along K: their sum
    in this order, rounded to ``out_dtype``, is the product.  Handed only to code that asked for
    it (``gemm(..., shares=True)``) and sums the shares itself, which saves the kernel that
    would."""

    partials: torch.Tensor
    out_dtype: torch.dtype

    @property
    def shape(self):
        return self.partials.shape[1:]

    def value(self) -> torch.Tensor:
        S, M, N = self.partials.shape
        out = torch.empty((M, N), dtype=self.out_dtype, device=self.partials.device)
        _call("lc_gemm_bf16_sum_shares", _ptr(self.partials), _ptr(out), _c_int(_dt(out)), _c_int(M),
              _c_int(N), _c_int(S), _stream())
        return out


def value(t):
    """The tensor that ``t`` stands for (``t`` itself if it is one)."""
    return t.value() if isinstance(t, (PendingProduct, ScaledRows, ProductShares)) else t


def rmsnorm(h: torch.Tensor, delta, weight: torch.Tensor, eps: float,
            out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, scaled: bool = False):
    """RMSNorm of the float32 residual stream ``h`` [T, n], with the pending branch output
    ``delta`` [T, n] (a tensor or a PendingProduct) added first.

    Without ``rows``: ``h += delta`` in place and every row is normed.  With ``rows`` (int32
    [R]): only those rows are normed (``h`` stays as it is) and the result is [R, n].
    ``scaled``: the caller also takes ScaledRows, and gets them where that saves a kernel.
    """
    _need(h, "rmsnorm h", torch.float32, 2)
    _need(weight, "rmsnorm weight", torch.float32, 1)
    T, n = h.shape
    if weight.shape[0] != n:
        raise KernelError(f"rmsnorm: weight has {weight.shape[0]} entries for rows of {n}")
    scaled = (scaled and rows is None and out_dtype == torch.bfloat16 and T > 0
              and bool(library().lc_gemm_bf16_scaled_rows_supported(T, 16, n)))
    if isinstance(delta, PendingProduct):
        M, K = delta.x.shape
        pieces = (library().lc_gemm_bf16_residual_pieces(M, n, K)
                  if scaled and delta.w.shape[0] == n and M == T else 0)
        if pieces:
            xg = torch.empty((T, n), dtype=torch.bfloat16, device=h.device)
            parts = torch.empty((pieces, library().lc_gemm_bf16_piece_stride(T)), dtype=torch.float32,
                                device=h.device)
            _call("lc_gemm_bf16_residual", _ptr(delta.x), _ptr(delta.w), _ptr(h), _ptr(weight),
                  _ptr(xg), _ptr(parts), _c_int(M), _c_int(n), _c_int(K), _stream())
            return ScaledRows(xg, parts, pieces, float(eps), h, weight)
        shares = library().lc_gemm_bf16_shares(M, n, K) if (delta.w.shape[0] == n and M == T) else 0
        if shares:
            # the product is cut along K anyway: its shares are summed in the norm kernel
            partials = torch.empty((shares, T, n), dtype=torch.float32, device=h.device)
            _call("lc_gemm_bf16_partials", _ptr(delta.x), _ptr(delta.w), _ptr(partials), _c_int(M),
                  _c_int(n), _c_int(K), _stream())
            delta = partials
        else:
            shares = 0
            delta = delta.value()
    else:
        shares = 0
    if delta is not None and not shares:
        _need(delta, "rmsnorm delta", out_dtype, 2)
        if tuple(delta.shape) != (T, n):
            raise KernelError(f"rmsnorm: delta {tuple(delta.shape)} does not match h {(T, n)}")
    if rows is not None:
        _need(rows, "rmsnorm rows", torch.int32, 1)
    R = T if rows is None else rows.shape[0]
    out = torch.empty((R, n), dtype=out_dtype, device=h.device)
    parts = (torch.empty((1, library().lc_gemm_bf16_piece_stride(T)), dtype=torch.float32, device=h.device)
             if scaled else None)
    _call("lc_rmsnorm", _ptr(h), _ptr(delta), _ptr(rows), _ptr(weight), _c_float(eps), _ptr(out),
          _c_int(_dt(out)), _c_int(R), _c_int(n),
          _c_int(1 if (rows is None and delta is not None) else 0), _ptr(parts), _c_int(shares),
          _c_int(T), _stream())
    return ScaledRows(out, parts, 1, float(eps), h, weight) if scaled else out


def rmsnorm_act(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm over the last dimension of an activation tensor."""
    _need(x, "rmsnorm_act x")
    _need(weight, "rmsnorm_act weight", torch.float32, 1)
    n = x.shape[-1]
    if weight.shape[0] != n:
        raise KernelError(f"rmsnorm_act: weight has {weight.shape[0]} entries for rows of {n}")
    out = torch.empty_like(x)
    _call("lc_rmsnorm_act", _ptr(x), _ptr(weight), _c_float(eps), _ptr(out), _c_int(_dt(x)),
          _c_int(x.numel() // n), _c_int(n), _stream())
    return out


# ------------------------------------------------------------------------------ products
def _scaled_product(x: "ScaledRows", w: torch.Tensor, epilogue: int) -> Optional[torch.Tensor]:
    """``x`` with its rows' factors times ``w`` transposed in one kernel, or None if there is
    no such kernel for these operands."""
    M, K = x.x.shape
    N = w.shape[0]
    if not (w.dtype == torch.bfloat16 and x.x.dtype == torch.bfloat16 and w.shape[1] == K
            and x.count <= 512 and library().lc_gemm_bf16_scaled_rows_supported(M, N, K)):
        return None
    out = torch.empty((M, N // 2 if epilogue else N), dtype=torch.bfloat16, device=w.device)
    _call("lc_gemm_bf16_scaled_rows", _ptr(x.x), _ptr(w), _ptr(out), _c_int(M), _c_int(N),
          _c_int(K), _c_int(epilogue), _ptr(x.pieces), _c_int(x.count), _c_float(x.eps), _stream())
    return out


def gemm(x, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None, defer: bool = False,
         shares: bool = False):
    """``x`` [M, K] times ``w`` [N, K] transposed -> [M, N]; float32 accumulation.

    ``x`` may be ScaledRows.  ``defer``: the result is a branch's output that goes to the
    residual stream; where the kernel that computes it can add it there itself, a
    PendingProduct comes back instead of a tensor.  ``shares``: the caller sums the shares of
    a product that is cut along K itself; where this one is, ProductShares come back."""
    if isinstance(x, ScaledRows):
        if out_dtype in (None, torch.bfloat16) and not defer:
            out = _scaled_product(x, w, 0)
            if out is not None:
                return out
        x = x.value()
    _need(x, "gemm x", None, 2)
    _need(w, "gemm w", None, 2)
    M, K = x.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: x is [{M}, {K}] but w is [{N}, {K2}]")
    out_dtype = out_dtype or x.dtype
    if (defer and out_dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (library().lc_gemm_bf16_residual_pieces(M, N, K) or library().lc_gemm_bf16_shares(M, N, K))):
        return PendingProduct(x, w, out_dtype)
    if shares and out_dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        count = library().lc_gemm_bf16_shares(M, N, K)
        if count:
            partials = torch.empty((count, M, N), dtype=torch.float32, device=x.device)
            _call("lc_gemm_bf16_partials", _ptr(x), _ptr(w), _ptr(partials), _c_int(M), _c_int(N),
                  _c_int(K), _stream())
            return ProductShares(partials, out_dtype)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return out
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and _fast_gemm_ok(M, N, K)):
        _call("lc_gemm_bf16", _ptr(x), _ptr(w), _ptr(out), _c_int(_dt(out)), _c_int(M), _c_int(N),
              _c_int(K), 0, _ptr(_gemm_workspace(M, N, K, x.device)), _stream())
    else:
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and N * K >= 1 << 22:
            _say_once(("gemm", N, K),
                      f"a bfloat16 product with w [{N}, {K}] has no matrix-core kernel (K must be a multiple "
                      f"of {library().lc_gemm_bf16_kblock()}): the general kernel runs, correct and many times slower")
        words = library().lc_gemm_generic_workspace(M, N, K)
        workspace = torch.empty((words,), dtype=torch.float32, device=x.device) if words else None
        _call("lc_gemm_generic", _ptr(x), _c_int(_dt(x)), _ptr(w), _c_int(_dt(w)), _ptr(out),
              _c_int(_dt(out)), _c_int(M), _c_int(N), _c_int(K), _ptr(workspace), _stream())
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Stack gate and up weights [I, H] as blocks of 8 gate rows followed by their 8 up rows
    (the layout ``gemm_swiglu`` wants); I must be a multiple of 8."""
    I, H = gate.shape
    return torch.stack([gate.view(I // 8, 8, H), up.view(I // 8, 8, H)], dim=1).reshape(2 * I, H).contiguous()


def gemm_swiglu_supported(x_dtype, w: torch.Tensor, K: int) -> bool:
    return (x_dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.shape[0] % 16 == 0
            and _fast_gemm_ok(64, w.shape[0], K))


def gemm_swiglu(x: torch.Tensor, w_interleaved: torch.Tensor) -> torch.Tensor:
    """``silu(x . gate^T) * (x . up^T)`` in one kernel, with gate and up interleaved by
    :func:`interleave_gate_up`; bfloat16 only.  [M, K] x [2 I, K] -> [M, I].  ``x`` may be
    ScaledRows."""
    if isinstance(x, ScaledRows):
        out = _scaled_product(x, w_interleaved, 1) if w_interleaved.shape[0] % 16 == 0 else None
        if out is not None:
            return out
        x = x.value()
    _need(x, "gemm_swiglu x", torch.bfloat16, 2)
    _need(w_interleaved, "gemm_swiglu w", torch.bfloat16, 2)
    M, K = x.shape
    N, K2 = w_interleaved.shape
    if K != K2 or N % 16:
        raise KernelError(f"gemm_swiglu: x is [{M}, {K}], w is [{N}, {K2}] (rows must come in 16s)")
    out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=x.device)
    if M:
        _call("lc_gemm_bf16", _ptr(x), _ptr(w_interleaved), _ptr(out), DT_BF16, M, N, K, 1,
              _ptr(_gemm_workspace(M, N, K, x.device)), _stream())
    return out


def _gemm_workspace(M: int, N: int, K: int, device) -> Optional[torch.Tensor]:
    """Float32 scratch for the products that cut K into shares (None when none is needed)."""
    words = library().lc_gemm_bf16_workspace(M, N, K)
    return torch.empty((words,), dtype=torch.float32, device=device) if words else None


def force_gemm_tile(tile: int) -> None:
    """Make the tiled bfloat16 product use one tile shape for every size (0: 64x128, 1: 128x128,
    2: 256x128, 3: 256x192, 4: 256x256, 5: 192x128, 6: 192x256, 7: 64x64, 8: 64x96, 9: 192x320, 10: 64x224,
    11: 64x128 in one round, 12: 64x160; -1: choose by size again).  For tests and tuning."""
    _call("lc_gemm_bf16_force_tile", _c_int(tile))


def gemm_even_rows(on: bool) -> None:
    """Whether the bfloat16 product of up to 16 rows may cut N into work items of fewer than 16
    rows so that every CU gets the same number (on by default).  For tests and tuning."""
    _call("lc_gemm_bf16_even_rows", _c_int(1 if on else 0))


def gemm_runs(mode) -> None:
    """Whether the bfloat16 product of up to 16 rows reads w in runs of 1 KB through LDS: where K
    is a multiple of 512 and w is large enough to gain (1 or True, the default), wherever K is
    a multiple of 512 (2), never (0 or False).  For tests and tuning."""
    _call("lc_gemm_bf16_runs", _c_int(int(mode)))


def force_gemm_skinny(shape: int) -> None:
    """Make the bfloat16 product of up to 16 rows use one shape of its kernel (0: deep unroll,
    1: plain, 2: two row tiles a workgroup, 3: several tiles a workgroup with x in registers;
    -1: choose by size again).  For tests and tuning."""
    _call("lc_gemm_bf16_force_skinny", _c_int(shape))


def _fast_gemm_ok(M: int, N: int, K: int) -> bool:
    return bool(library().lc_gemm_bf16_supported(M, N, K))


# ------------------------------------------------------------------------------ attention
def qk_norm_rope_write(qkv: torch.Tensor, nh: int, nkv: int, d: int,
                       q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                       eps: float, positions: Optional[torch.Tensor],
                       rope_table: Optional[torch.Tensor],
                       k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                       slots: Optional[torch.Tensor], page_size: int, skip_q: bool = False) -> None:
    """In place on ``qkv`` [T, (nh + 2 nkv) d]: per-head RMSNorm of q and k (if weights are
    given), rotation by ``rope_table`` [positions, rot] (cos | sin halves) at each token's
    position, and the write of k and v into their cache slot ``slots`` [T]
    (page * page_size + offset; negative: no write).  Key cache [pages, nkv, page_size, d],
    value cache [pages, nkv, d, page_size].  ``skip_q``: q is left raw (the attention kernels
    prepare it themselves)."""
    _need(qkv, "qkv", None, 2)
    T = qkv.shape[0]
    if qkv.shape[1] != (nh + 2 * nkv) * d:
        raise KernelError(f"qkv has {qkv.shape[1]} columns, expected {(nh + 2 * nkv) * d}")
    rot = 0
    if rope_table is not None:
        _need(rope_table, "rope table", torch.float32, 2)
        _need(positions, "positions", torch.int32, 1)
        rot = rope_table.shape[1]
        if positions.shape[0] != T:
            raise KernelError("positions do not match the tokens")
    for wt, name in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if wt is not None:
            _need(wt, name, torch.float32, 1)
            if wt.shape[0] != d:
                raise KernelError(f"{name} has {wt.shape[0]} entries for head size {d}")
    if k_cache is not None and slots is not None:
        _need(k_cache, "k cache", qkv.dtype, 4)
        _need(v_cache, "v cache", qkv.dtype, 4)
        _need(slots, "slots", torch.int32, 1)
        _check_caches(k_cache, v_cache, nkv, page_size, d)
        if slots.shape[0] != T:
            raise KernelError("slots do not match the tokens")
    else:
        k_cache = v_cache = slots = None
    _call("lc_qk_norm_rope_write", _ptr(qkv), _c_int(_dt(qkv)), _c_int(T), _c_int(nh), _c_int(nkv),
          _c_int(d), _ptr(q_weight), _ptr(k_weight), _c_float(eps), _ptr(positions),
          _ptr(rope_table), _c_int(rot), _ptr(k_cache), _ptr(v_cache), _ptr(slots),
          _c_int(page_size), _c_int(nh if skip_q else 0), _stream())


def _check_caches(k_cache, v_cache, nkv, page_size, d) -> None:
    if tuple(k_cache.shape[1:]) != (nkv, page_size, d):
        raise KernelError(f"key cache shape {tuple(k_cache.shape)} does not fit "
                          f"[pages, {nkv}, {page_size}, {d}]")
    if tuple(v_cache.shape) != (k_cache.shape[0], nkv, d, page_size):
        raise KernelError(f"value cache shape {tuple(v_cache.shape)} does not fit "
                          f"[{k_cache.shape[0]}, {nkv}, {d}, {page_size}] (values are transposed "
                          f"inside a page)")


@dataclass
class AttentionBatch:
    """What attention needs to know of a step's batch, for one group of cache pages.

    All tensors are int32 on the GPU.  ``tok_req[t]`` is the row of ``block_table`` that token
    t belongs to; ``positions[t]`` its absolute position; ``block_table`` [R, max_blocks] maps
    position // page_size to a page.  ``q_start`` [R + 1] are the requests' token offsets in
    the batch, ``ctx_len`` [R] their cached lengths after this step.  ``decode_rows`` and
    ``prefill_tiles`` list the work of the decode and prefill kernels (None: not prepared).
    """

    tok_req: torch.Tensor
    positions: torch.Tensor
    block_table: torch.Tensor
    q_start: Optional[torch.Tensor] = None
    ctx_len: Optional[torch.Tensor] = None
    slots: Optional[torch.Tensor] = None
    num_decode: int = 0
    decode_rows: Optional[torch.Tensor] = None     # [ND, 4] of the length-1 portions: token row, request, position, its items
    decode_items: Optional[torch.Tensor] = None    # [NI, 8]: the rows' pages cut into work items by length (None: not prepared)
    prefill_tiles: Optional[torch.Tensor] = None   # [NT, 4]: request, first token row, rows, first position
    max_ctx: int = 0                               # longest cached length in the batch
    all_decode: bool = False
    even_lengths: bool = False                     # the longest decoding request is within a tenth of the mean length
    decode_longest: int = 0                        # tokens of the longest decoding request, and of all of them
    decode_total: int = 0


class _Switch(threading.local):
    on = True


_decode_by_items = _Switch()     # per thread, like the library's own switches


def decode_by_items(on):
    """Whether the decode kernel takes the planner's list of work items: True where the library
    says it pays (the default), False never, "always" wherever there is a list (tests and
    tuning); returns the setting before."""
    before = _decode_by_items.on
    _decode_by_items.on = on if on == "always" else bool(on)
    return before


PREFILL_TILE = 64               # query rows of one work item of the prefill attention kernel
ATTENTION_PLAN = "paged_attention"


def plan_attention(layout):
    """The work lists of the attention kernels for one step's batch (a planner in the sense of
    ``Part.batch_planner``): the portions of length one, which the decode kernel serves, four
    numbers each (token row, request, position, and where its work items lie: all a workgroup
    needs to know of its token in one load, not one look-up after the other), the same rows' pages
    cut into work items by length (:func:`_decode_items`), which the kernel takes instead where
    few requests hold most of the keys, and the tiles of up to PREFILL_TILE query rows that the longer portions are
    cut into, four numbers each (request, first token row, rows, first position).  The tiles
    that see the most keys come first: the kernel's workgroups start in this order, and whoever
    is done takes the longest that is left (the order changes no tile's result).  The decoding
    rows likewise come longest request first."""
    R, q_start, first = layout.num_requests, layout.q_start, layout.first_position
    if layout.single:
        singles = np.arange(R, dtype=np.int64)
        tiles = np.zeros((0, 4), dtype=np.int32)
    else:
        singles = np.asarray([r for r in range(R) if q_start[r + 1] - q_start[r] == 1], dtype=np.int64)
        tile_list = []
        for r in range(R):
            n = q_start[r + 1] - q_start[r]
            if n == 1:
                continue
            for t0 in range(0, n, PREFILL_TILE):
                tile_list.append((r, q_start[r] + t0, min(PREFILL_TILE, n - t0), first[r] + t0))
        tile_list.sort(key=lambda t: -(t[3] + t[2]))
        tiles = np.asarray(tile_list, dtype=np.int32).reshape(-1, 4)
    # lengths after this step of the requests that decode: a hint for the decode kernel (how
    # it lays its work out, never what it computes); "graph_hint" below keeps a captured step
    # to the batches whose hints are its own
    lengths = np.asarray(first, dtype=np.int64)[singles] + 1
    decode = np.zeros((singles.size, 4), dtype=np.int32)
    decode[:, 0] = np.asarray(q_start, dtype=np.int64)[singles]
    decode[:, 1] = singles
    decode[:, 2] = lengths - 1
    even = bool(lengths.size) and int(lengths.max()) * int(lengths.size) <= 1.1 * int(lengths.sum())
    if lengths.size > 1 and int(lengths.max()) != int(lengths.min()):
        # the decode kernel's workgroups start in the order of this list: the longest requests first,
        # so that none of them starts late and runs on alone at the end (64 requests of 16 to 2,200
        # tokens: 58 instead of 70 us a layer; the order changes no token's result)
        decode = decode[np.argsort(-lengths, kind="stable")]
    items = _decode_items(decode, lengths[np.argsort(-lengths, kind="stable")] if lengths.size > 1 else lengths)
    # (whether the list pays, the kernel's library says from the longest and the total length)
    longest, total = (int(lengths.max()), int(lengths.sum())) if lengths.size else (0, 0)
    # what a captured step must share with the batches it is replayed for: the classes of lengths
    # between which the decode kernel's launch changes (even; up to a quarter above the mean;
    # up to three times the mean; beyond: the thresholds of lc_attn_decode_by_items)
    spread = longest * int(lengths.size)
    hint = (even, 0 if spread * 4 <= total * 5 else 1 if spread < total * 3 else 2)
    return ({"decode_rows": decode, "decode_items": items, "prefill_tiles": tiles},
            {"num_decode": int(singles.size), "all_decode": int(singles.size) == R, "even_lengths": even,
             "decode_longest": longest, "decode_total": total, "graph_hint": hint})


ITEM_PAGES_MIN = 8       # kernel pages of the smallest work item that a request is cut into
ITEM_SHARES_MOST = 32    # items of one request at most (the join kernel takes up to 64)


def decode_item_count(num_decode: int) -> int:
    """Work items that the planner makes for a step with ``num_decode`` single tokens: a number
    that follows from the count alone, so that steps of one make-up have lists of one size (a
    captured step is replayed with the next step's list in the same buffer)."""
    return max(num_decode + num_decode // 2, min(64, 8 * num_decode)) if num_decode else 0


def _decode_items(decode: np.ndarray, lengths: np.ndarray) -> np.ndarray:
    """The decode rows' pages (of ATTENTION_PAGE_GRANULE tokens) cut into ``decode_item_count``
    work items so that the largest item is as small as may be: every row one item, the spare ones
    to whichever row has the largest items then (at most ITEM_SHARES_MOST a row, none smaller than
    ITEM_PAGES_MIN pages).  Eight numbers an item: token row, request, position, row, first page,
    end page, the row's number of items, 0; a row's items are neighbours; items that are left over
    have no shares and do nothing.  Writes each row's first item and number of items into
    ``decode[:, 3]``.  ``lengths`` in the order of ``decode``."""
    nd = int(decode.shape[0])
    total = decode_item_count(nd)
    items = np.zeros((total, 8), dtype=np.int32)
    if nd == 0:
        return items
    lengths = np.asarray(lengths, dtype=np.int64)
    pages = (lengths + ATTENTION_PAGE_GRANULE - 1) // ATTENTION_PAGE_GRANULE
    shares = np.ones(nd, dtype=np.int64)
    # lengths so even that no launcher would take the list: every row its one item, no search
    uneven = int(lengths.max()) * nd * 4 > int(lengths.sum()) * 5
    spare = total - nd
    if uneven and spare > 0:
        most = np.minimum(ITEM_SHARES_MOST, np.maximum(1, pages // ITEM_PAGES_MIN))
        heap = [(-int(pages[r]), r) for r in np.nonzero(most > 1)[0].tolist()]
        heapq.heapify(heap)
        while spare > 0 and heap:
            _, r = heapq.heappop(heap)
            shares[r] += 1
            spare -= 1
            if shares[r] < most[r]:
                heapq.heappush(heap, (-int((pages[r] + shares[r] - 1) // shares[r]), r))
    first = np.cumsum(shares) - shares
    decode[:, 3] = first | (shares << 20)
    used = int(shares.sum())
    row = np.repeat(np.arange(nd, dtype=np.int64), shares)
    nth = np.arange(used, dtype=np.int64) - first[row]        # which of its row's items
    n, k = pages[row], shares[row]                            # sizes that differ by one page at most, none empty
    items[:used, 0:3] = decode[row, 0:3]
    items[:used, 3] = row
    items[:used, 4] = nth * n // k
    items[:used, 5] = (nth + 1) * n // k
    items[:used, 6] = k
    return items


# Tokens of a cache page as the matrix-core attention kernels index it: a page of a multiple of
# it reaches them as so many pages of this size.  The kernels say the same number
# (lc_attn_page_granule), which is checked when the library is loaded; a model can be described
# and its cache laid out without loading it.
ATTENTION_PAGE_GRANULE = 16


def attention_page_granule() -> int:
    return ATTENTION_PAGE_GRANULE


def attention_batch(batch, pages, plan=None) -> AttentionBatch:
    """The attention kernels' record of a step: from the step's batch (``engine.batch.StepBatch``:
    tok_req, positions, q_offsets, ctx_len, max_ctx), a page group's view of it (``PagesView``:
    block table, slots) and the work lists of ``plan`` (made by :func:`plan_attention`; None:
    without, and only the generic kernel can run).  Made once a step and page group, kept in
    ``pages.made``."""
    done = pages.made.get(ATTENTION_PLAN)
    if done is None:
        done = AttentionBatch(tok_req=batch.tok_req, positions=batch.positions,
                              block_table=pages.block_table, q_start=batch.q_offsets,
                              ctx_len=batch.ctx_len, slots=pages.slots, max_ctx=batch.max_ctx)
        if plan is not None:
            done = replace(done, decode_rows=plan.arrays["decode_rows"],
                           decode_items=plan.arrays.get("decode_items"),
                           decode_longest=plan.info.get("decode_longest", 0),
                           decode_total=plan.info.get("decode_total", 0),
                           prefill_tiles=plan.arrays["prefill_tiles"],
                           num_decode=plan.info["num_decode"], all_decode=plan.info["all_decode"],
                           even_lengths=plan.info["even_lengths"])
        pages.made[ATTENTION_PLAN] = done
    return done


@dataclass
class QKPrologue:
    """What has to happen to the raw q, k, v of a step before attention: RMSNorm of every q and
    k head (weights may be None), rotary embedding (table may be None), and the write of k and
    v to the cache slots (``slots`` None: no write, another site owns the cache)."""

    q_weight: Optional[torch.Tensor]
    k_weight: Optional[torch.Tensor]
    eps: float
    rope_table: Optional[torch.Tensor]
    slots: Optional[torch.Tensor]


def attention_takes_shares(batch: AttentionBatch, T: int, nh: int, nkv: int, d: int, page_size: int,
                           dtype: torch.dtype, rot: int) -> bool:
    """Whether ``attention`` can take the raw q, k, v of this step as ProductShares: a step of
    single tokens in bfloat16, whose decode kernel prepares whole heads of 128 itself and sums
    the shares as it reads them."""
    lib = library()
    return bool(dtype == torch.bfloat16 and batch.decode_rows is not None
                and batch.prefill_tiles is not None and batch.num_decode == T and T > 0
                and lib.lc_attn_bf16_supported(nh, nkv, d, page_size)
                and lib.lc_attn_decode_takes_shares(d, rot))


def attention(qkv, batch: AttentionBatch, k_cache: torch.Tensor,
              v_cache: torch.Tensor, nh: int, nkv: int, d: int, page_size: int, scale: float,
              window: int = 0, prologue: Optional[QKPrologue] = None) -> torch.Tensor:
    """Causal attention of the q heads in ``qkv`` [T, (nh + 2 nkv) d] over the cached keys and
    values -> [T, nh d].  Without ``prologue`` the step's own keys and values have been written
    already and q is ready; with it, ``qkv`` is raw, and what is left raw in it afterwards is
    not defined (q stays raw where the attention kernels prepare it on the fly)."""
    shares = None
    if isinstance(qkv, ProductShares):
        # asked for by a caller who had attention_takes_shares say yes; anything else gets the sum
        rope0 = prologue.rope_table if prologue is not None else None
        if (prologue is not None and qkv.out_dtype == torch.bfloat16
                and attention_takes_shares(batch, qkv.shape[0], nh, nkv, d, page_size, qkv.out_dtype,
                                           rope0.shape[1] if rope0 is not None else 0)
                and (prologue.q_weight is None) == (prologue.k_weight is None)):
            shares = qkv.partials
            qkv = torch.empty((0, shares.shape[2]), dtype=torch.bfloat16, device=shares.device)
        else:
            qkv = qkv.value()
    _need(qkv, "qkv", None, 2)
    _need(k_cache, "k cache", qkv.dtype, 4)
    _need(v_cache, "v cache", qkv.dtype, 4)
    T = qkv.shape[0] if shares is None else shares.shape[1]
    out = torch.empty((T, nh * d), dtype=qkv.dtype, device=qkv.device)
    if T == 0:
        return out
    _need(batch.tok_req, "tok_req", torch.int32, 1)
    _need(batch.positions, "positions", torch.int32, 1)
    _need(batch.block_table, "block table", torch.int32, 2)
    _check_caches(k_cache, v_cache, nkv, page_size, d)
    lib = library()
    fast = (qkv.dtype == torch.bfloat16 and batch.decode_rows is not None
            and batch.prefill_tiles is not None and lib.lc_attn_bf16_supported(nh, nkv, d, page_size))
    if qkv.dtype == torch.bfloat16 and not fast:
        _say_once(("attention", nh, nkv, d, page_size),
                  f"bfloat16 attention with {nh} heads, {nkv} kv heads of {d} and pages of {page_size} tokens has no "
                  "matrix-core kernel (heads of 32, 64, 96 or 128, pages of a multiple of 16 tokens, at most 16 heads a kv head): "
                  "the general kernel runs, correct and many times slower")
    # who prepares q, k, v (norm, rotation, cache write) when they arrive raw: a step of single
    # tokens does it all inside the decode kernel; otherwise a kernel of its own does k and v,
    # and q too unless both attention kernels can prepare their q themselves
    rope = prologue.rope_table if prologue is not None else None
    if rope is not None:
        _need(rope, "rotary table", torch.float32, 2)
    rot = rope.shape[1] if rope is not None else 0
    all_in_decode = fast and prologue is not None and batch.num_decode == T
    own_q = (fast and prologue is not None and not all_in_decode
             and (prologue.q_weight is None) == (prologue.k_weight is None)
             and bool(lib.lc_attn_prefill_prepares_q(d, rot)))
    if prologue is not None and not all_in_decode:
        qk_norm_rope_write(qkv, nh, nkv, d, prologue.q_weight, prologue.k_weight, prologue.eps,
                           batch.positions, prologue.rope_table, k_cache, v_cache, prologue.slots,
                           page_size, skip_q=own_q)
    in_kernel = all_in_decode or own_q
    if fast:
        mb = batch.block_table.shape[1]
        nd = batch.num_decode
        if nd > 0:
            # requests of unequal length: the planner's list of work items, which cuts the long ones
            # into more shares than the short ones; else every request into the same number
            items = None
            if batch.decode_items is not None and _decode_by_items.on is not False and (
                    _decode_by_items.on == "always"
                    or lib.lc_attn_decode_by_items(nd, nkv, batch.decode_longest, batch.decode_total)):
                items = batch.decode_items
            splits = 1 if items is not None else lib.lc_attn_decode_splits(nd, nkv, batch.max_ctx)
            part_o = part_ml = None
            parts = items.shape[0] if items is not None else (nd * splits if splits > 1 else 0)
            if parts:
                part_o = torch.empty((parts * nh * d,), dtype=torch.float32, device=qkv.device)
                part_ml = torch.empty((parts * nh * 2,), dtype=torch.float32, device=qkv.device)
            _call("lc_attn_decode_bf16", _ptr(qkv if shares is None else None), qkv.shape[1], _ptr(k_cache), _ptr(v_cache),
                  _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(batch.decode_rows),
                  _ptr(items), items.shape[0] if items is not None else 0,
                  _ptr(batch.block_table), mb, nd, nh,
                  nkv, d, page_size, scale, window, splits, 1 if batch.even_lengths else 0,
                  1 if in_kernel else 0,
                  _ptr(prologue.q_weight if in_kernel else None),
                  _ptr(prologue.k_weight if in_kernel else None),
                  _c_float(prologue.eps if in_kernel else 0.0), _ptr(rope if in_kernel else None),
                  rot if in_kernel else 0,
                  1 if all_in_decode and prologue.slots is not None else 0,
                  _ptr(shares), shares.shape[0] if shares is not None else 0,
                  shares.shape[1] if shares is not None else 0, _stream())
        nt = batch.prefill_tiles.shape[0]
        if nt > 0:
            pf_splits = lib.lc_attn_prefill_splits(nt, nh, nkv, batch.max_ctx)
            pf_o = pf_ml = None
            if pf_splits > 1:      # few tiles after a long history: the keys are shared out
                pf_o = torch.empty((T * nh * pf_splits * d,), dtype=torch.float32, device=qkv.device)
                pf_ml = torch.empty((T * nh * pf_splits * 2,), dtype=torch.float32, device=qkv.device)
            _call("lc_attn_prefill_bf16", _ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache),
                  _ptr(out), _ptr(batch.prefill_tiles), _ptr(batch.block_table), mb, nt, nh, nkv, d,
                  page_size, scale, window, 1 if own_q else 0,
                  _ptr(prologue.q_weight if own_q else None),
                  _c_float(prologue.eps if own_q else 0.0), _ptr(rope if own_q else None),
                  rot if own_q else 0, pf_splits, _ptr(pf_o), _ptr(pf_ml), _stream())
        return out
    words = lib.lc_attention_generic_workspace(T, nh, nkv, batch.block_table.shape[1], page_size)
    workspace = torch.empty((words,), dtype=torch.float32, device=qkv.device) if words else None
    _call("lc_attention_generic", _ptr(qkv), _c_int(qkv.shape[1]), _ptr(k_cache), _ptr(v_cache),
          _ptr(out), _c_int(_dt(qkv)), _ptr(batch.tok_req), _ptr(batch.positions),
          _ptr(batch.block_table), _c_int(batch.block_table.shape[1]), _c_int(T), _c_int(nh),
          _c_int(nkv), _c_int(d), _c_int(page_size), _c_float(scale), _c_int(window),
          _ptr(workspace), _stream())
    return out


# ------------------------------------------------------------------------------ feed-forward
def swiglu(gu: torch.Tensor) -> torch.Tensor:
    """``gu`` [T, 2 I] (gate columns, then up columns) -> silu(gate) * up, [T, I]."""
    _need(gu, "swiglu input", None, 2)
    T, two_i = gu.shape
    if two_i % 2:
        raise KernelError("swiglu: the input needs an even number of columns")
    out = torch.empty((T, two_i // 2), dtype=gu.dtype, device=gu.device)
    _call("lc_swiglu", _ptr(gu), _ptr(out), _c_int(_dt(gu)), _c_int(T), _c_int(two_i // 2), _stream())
    return out


# ------------------------------------------------------------------------------ sampling
def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Token ids (int32 [R]) from float32 ``logits`` [R, V]: greedy where the row's temperature
    is <= 0 (or none is given), else inverse-CDF sampling of softmax(logits / temperature) with
    the row's uniform number in [0, 1)."""
    _need(logits, "logits", torch.float32, 2)
    R, V = logits.shape
    if temperature is not None:
        _need(temperature, "temperature", torch.float32, 1)
        _need(uniform, "uniform", torch.float32, 1)
        if temperature.shape[0] != R or uniform.shape[0] != R:
            raise KernelError("sample: one temperature and one uniform number per row")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    workspace = torch.empty((max(1, library().lc_sample_workspace(R)),), dtype=torch.float32,
                            device=logits.device)
    _call("lc_sample", _ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(out), _ptr(workspace),
          _c_int(R), _c_int(V), _stream())
    return out


def feed_tokens(ids: torch.Tensor, source: torch.Tensor, sampled: torch.Tensor) -> None:
    """``ids[i] = sampled[source[i]]`` wherever ``source[i] >= 0`` (all int32, on the device):
    what an earlier step sampled becomes a later step's input without passing the host."""
    _need(ids, "fed ids", torch.int32, 1)
    _need(source, "feed source", torch.int32, 1)
    _need(sampled, "sampled ids", torch.int32, 1)
    if source.shape[0] != ids.shape[0]:
        raise KernelError("feed_tokens: one source row per id")
    _call("lc_feed_tokens", _ptr(ids), _ptr(source), _ptr(sampled), _c_int(ids.shape[0]),
          _c_int(sampled.shape[0]), _stream())
