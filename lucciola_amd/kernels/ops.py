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
    "lc_rmsnorm_act": "pqpfpiiip",
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
    "lc_dynamic_tanh": "pppppfpiiiip",
    "lc_stream_add": "ppippiip",
    "lc_activation": "piiffqp",
    "lc_scale": "pfqp",
    "lc_token_shift": "pippppppiip",
    "lc_rms_shift": "ppipffppppppiiip",
    "lc_gemm_grouped": "piqqpipiqqiiiipppiiipqqp",
    "lc_gemm_grouped_fast": "i",
    "lc_gemm_grouped_takes_tile": "iii",
    "lc_latent_prepare": "pqpiqiiiiipfppiipppp",
    "lc_latent_attention": "piiiiippppiifippp",
    "lc_latent_bf16_supported": "ii",
    "lc_latent_bf16_splits": "ii",
    "lc_latent_attention_bf16": "piiiippiipiifippippp",
    "lc_moe_max_experts": "",
    "lc_moe_route": "piiiifppp",
    "lc_moe_route_sigmoid": "ppiiiiifppp",
    "lc_lightning_prepare": "piiiiipppp",
    "lc_lightning_readout": "ppiipfiipip",
    "lc_moe_lists": "piiiippppp",
    "lc_moe_combine": "pppiiipip",
    "lc_layer_norm": "ppifppfpppfpiiiiip",
    "lc_embedding_sinusoid": "pppippiiifp",
    "lc_gated_activation": "ppiiiip",
    "lc_head_norm_write": "piiiiiiippfpppppiip",
    "lc_general_delta_prepare": "piiiipppffppp",
    "lc_gated_delta_prepare": "piiiiiippippfpppppp",
    "lc_conv_tail_update": "piipiiippip",
    "lc_delta_scan": "pippipppiiiiip",
    "lc_head_gate_norm": "ppiipifiiiipip",
    "lc_moe_route_logits": "pipiiippp",
    "lc_moe_combine_shared": "pppiiipipiipip",
    "lc_gated_activation_weighted": "ppippiiip",
    "lc_masked_attention": "pppi" + "ppp" + "ii" + "i" + "iiiii" + "f" + "ii" + "ppp" + "f" + "i" + "ff" + "pii" + "pp",
    "lc_attention_prepare": "p" + "iiiiiii" + "pip" + "ppp" + "pip" + "if" + "ppp" + "i" + "pip",
    "lc_attention_prepare_pairs": "i",
    "lc_masked_attention_bf16_supported": "iiii",
    "lc_masked_attention_bf16": "ppp" + "pi" + "pii" + "iiiii" + "f" + "ii" + "ppp" + "f" + "i" + "ff" + "pii" + "ppiiip",
    "lc_masked_attention_bf16_staged": "i",
    "lc_masked_attention_bf16_workspace": "iiiiii",
    "lc_state_space_prepare": "piiiiii" + "ppi" + "ppp" + "ppp" + "pp" + "p",
    "lc_state_space_readout": "pppiipiipifipip",
    "lc_scaled_sum": "pifpifpqp",
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
    return t.value() if isinstance(t, (PendingProduct, ScaledRows, ProductShares, NormedBranch)) else t


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


def rmsnorm_act(x: torch.Tensor, weight: torch.Tensor, eps: float, column: Optional[int] = None) -> torch.Tensor:
    """RMSNorm over the last dimension of an activation tensor.  With ``column``: over the columns
    ``column`` .. ``column`` + len(weight) of the 2-D ``x`` alone -> [rows, len(weight)]."""
    _need(x, "rmsnorm_act x")
    _need(weight, "rmsnorm_act weight", torch.float32, 1)
    n = weight.shape[0]
    if column is not None:
        if x.dim() != 2 or column < 0 or column + n > x.shape[1]:
            raise KernelError(f"rmsnorm_act: columns {column}..{column + n} of {tuple(x.shape)}")
        out = torch.empty((x.shape[0], n), dtype=x.dtype, device=x.device)
        _call("lc_rmsnorm_act", ctypes.c_void_p(x.data_ptr() + column * x.element_size()), x.shape[1], _ptr(weight),
              _c_float(eps), _ptr(out), _c_int(_dt(x)), _c_int(x.shape[0]), _c_int(n), _stream())
        return out
    if x.shape[-1] != n:
        raise KernelError(f"rmsnorm_act: weight has {weight.shape[0]} entries for rows of {x.shape[-1]}")
    out = torch.empty_like(x)
    _call("lc_rmsnorm_act", _ptr(x), n, _ptr(weight), _c_float(eps), _ptr(out), _c_int(_dt(x)),
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


# ------------------------------------------------------------------------------ other norms, other feed-forwards
ACTIVATIONS = {"gelu_tanh": 1, "relu_squared": 2, "xielu": 5}     # xielu takes two numbers (``params``)
_EPILOGUE_GATE, _EPILOGUE_GROUP_GATE = 3, 4
_EPILOGUES = {"gelu_tanh": 1, "relu_squared": 2}                    # what a grouped product can apply itself


def dynamic_tanh(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor,
                 alpha: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``tanh(alpha v) * weight + bias`` of the float32 residual stream ``h`` [T, n] with the pending
    branch output ``delta`` added first (v = h + delta).  Without ``rows``: ``h += delta`` in place and
    every row is normed; with ``rows`` (int32 [R]): only those rows, ``h`` stays as it is."""
    _need(h, "dynamic_tanh h", torch.float32, 2)
    _need(weight, "dynamic_tanh weight", torch.float32, 1)
    _need(bias, "dynamic_tanh bias", torch.float32, 1)
    T, n = h.shape
    if weight.shape[0] != n or bias.shape[0] != n:
        raise KernelError(f"dynamic_tanh: weight and bias must have {n} entries")
    if delta is not None:
        _need(delta, "dynamic_tanh delta", out_dtype, 2)
        if tuple(delta.shape) != (T, n):
            raise KernelError(f"dynamic_tanh: delta {tuple(delta.shape)} does not match h {(T, n)}")
    if rows is not None:
        _need(rows, "dynamic_tanh rows", torch.int32, 1)
    R = T if rows is None else rows.shape[0]
    out = torch.empty((R, n), dtype=out_dtype, device=h.device)
    _call("lc_dynamic_tanh", _ptr(h), _ptr(delta), _ptr(rows), _ptr(weight), _ptr(bias), float(alpha), _ptr(out),
          _dt(out), R, n, 1 if (rows is None and delta is not None) else 0, _stream())
    return out


def stream_add(h: torch.Tensor, delta: Optional[torch.Tensor], vector: torch.Tensor,
               more: Optional[torch.Tensor] = None) -> None:
    """``h[t] += delta[t] (+ more[t]) + vector`` for every row of the float32 residual stream ``h`` [T, n];
    ``more`` float32 [T, n]."""
    _need(h, "stream_add h", torch.float32, 2)
    _need(vector, "stream_add vector", torch.float32, 1)
    T, n = h.shape
    if vector.shape[0] != n:
        raise KernelError(f"stream_add: a vector of {vector.shape[0]} entries for rows of {n}")
    if delta is not None:
        _need(delta, "stream_add delta", None, 2)
        if tuple(delta.shape) != (T, n):
            raise KernelError(f"stream_add: delta {tuple(delta.shape)} does not match h {(T, n)}")
    if more is not None:
        _need(more, "stream_add more", torch.float32, 2)
        if tuple(more.shape) != (T, n):
            raise KernelError(f"stream_add: more {tuple(more.shape)} does not match h {(T, n)}")
    _call("lc_stream_add", _ptr(h), _ptr(delta), _dt(delta) if delta is not None else DT_F32, _ptr(more), _ptr(vector),
          T, n, _stream())


def activation(x: torch.Tensor, kind: str, params=(0.0, 0.0)) -> torch.Tensor:
    """``x`` through one of ACTIVATIONS, in place; returns ``x``.  ``params``: the two numbers of "xielu"
    (z > 0: a z^2 + z/2; z <= 0: b (e^z - 1 - z) + z/2)."""
    _need(x, "activation x")
    _call("lc_activation", _ptr(x), _dt(x), ACTIVATIONS[kind], float(params[0]), float(params[1]), x.numel(), _stream())
    return x


def gemm_act(x, w: torch.Tensor, kind: str, out_dtype: torch.dtype, params=(0.0, 0.0)) -> torch.Tensor:
    """``act(x . w^T)``: the first product of a two-matrix feed-forward with its activation."""
    return activation(gemm(x, w, out_dtype), kind, params)


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """float32 ``x`` times ``factor``, in place; returns ``x``."""
    _need(x, "scale_ x", torch.float32)
    _call("lc_scale", _ptr(x), float(factor), x.numel(), _stream())
    return x


def _check_shift(T: int, n: int, mix, state, tok_req, q_offsets, slot_ids, what: str) -> None:
    _need(mix, f"{what} mix", torch.float32, 1)
    _need(state, f"{what} state", torch.float32, 2)
    _need(tok_req, "tok_req", torch.int32, 1)
    _need(q_offsets, "q_offsets", torch.int32, 1)
    _need(slot_ids, "slot_ids", torch.int32, 1)
    if mix.shape[0] != n or state.shape[1] != n or tok_req.shape[0] != T or q_offsets.shape[0] != slot_ids.shape[0] + 1:
        raise KernelError(f"{what}: mix, state or the request lists do not fit {T} rows of {n}")


def token_shift(x: torch.Tensor, mix: torch.Tensor, state: torch.Tensor, tok_req: torch.Tensor,
                q_offsets: torch.Tensor, slot_ids: torch.Tensor) -> torch.Tensor:
    """``y[t] = x[t] + (x[t - 1] - x[t]) * mix`` within every request; the row before a request's first token
    of the step is ``state[slot]`` (float32 [slots, n]), which then takes the request's last row."""
    _need(x, "token_shift x", None, 2)
    T, n = x.shape
    _check_shift(T, n, mix, state, tok_req, q_offsets, slot_ids, "token_shift")
    y = torch.empty_like(x)
    _call("lc_token_shift", _ptr(x), _dt(x), _ptr(mix), _ptr(state), _ptr(tok_req), _ptr(q_offsets), _ptr(slot_ids),
          _ptr(y), T, n, _stream())
    return y


def rms_shift(h: torch.Tensor, delta, gain: float, eps: float, mix: torch.Tensor, state: torch.Tensor,
              tok_req: torch.Tensor, q_offsets: torch.Tensor, slot_ids: torch.Tensor, out_dtype: torch.dtype):
    """The residual addition, an RMS norm with one number as its weight and the token shift in one kernel:
    v = h + delta; u = v / sqrt(mean(v^2) + eps) * gain; y[t] = u[t] + (u[t - 1] - u[t]) * mix, the row before
    a request's first token of the step being ``state[slot]``, which then takes the request's last u (float32).
    Returns (v float32 [T, n], a new tensor; y [T, n] of ``out_dtype``)."""
    _need(h, "rms_shift h", torch.float32, 2)
    T, n = h.shape
    delta = value(delta)
    if delta is not None:
        _need(delta, "rms_shift delta", None, 2)
        if tuple(delta.shape) != (T, n):
            raise KernelError(f"rms_shift: delta {tuple(delta.shape)} does not match h {(T, n)}")
    _check_shift(T, n, mix, state, tok_req, q_offsets, slot_ids, "rms_shift")
    h_out = torch.empty_like(h)
    y = torch.empty((T, n), dtype=out_dtype, device=h.device)
    _call("lc_rms_shift", _ptr(h), _ptr(delta), _dt(delta) if delta is not None else DT_F32, _ptr(h_out), float(gain),
          float(eps), _ptr(mix), _ptr(state), _ptr(tok_req), _ptr(q_offsets), _ptr(slot_ids), _ptr(y), _dt(y), T, n,
          _stream())
    return h_out, y


@dataclass
class Strided:
    """Equal stretches of the columns of a 2-D tensor, one per group: group g owns the columns
    ``column + g * group`` onwards (the heads side by side in a row of projections)."""

    tensor: torch.Tensor
    column: int
    group: int

    def pointer(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(self.tensor.data_ptr() + self.column * self.tensor.element_size())


def _check_strided(s: Strided, what: str, rows: int, groups: int, width: int, dtype=None) -> None:
    _need(s.tensor, what, dtype, 2)
    if s.tensor.shape[0] < rows or s.column < 0 or s.column + (groups - 1) * s.group + width > s.tensor.shape[1]:
        raise KernelError(f"{what}: {groups} groups of {width} columns from column {s.column}, {s.group} apart, "
                          f"and {rows} rows do not fit {tuple(s.tensor.shape)}")


def _grouped_tile(rows: int, N: int, groups: int, x: torch.Tensor, w: torch.Tensor) -> int:
    """Rows of a grouped product's tiles, for ``rows`` rows a group: 16 for a step of few tokens, 128
    (by 128 columns) where the operands take the bfloat16 kernel and there are so many rows and
    columns that even tiles of that size are several to a CU (measured: 2,048 rows, 16 heads and 128
    or 512 columns are faster in tiles of 64 x 64, which are four times as many)."""
    if rows <= 16:
        return 16
    if (-(-rows // 128)) * (-(-N // 128)) * groups >= 2048 and library().lc_gemm_grouped_takes_tile(128, _dt(x), _dt(w)):
        return 128
    return 64


def grouped_gemm(x: Strided, w: torch.Tensor, out: Strided, rows: int, gate: Optional[Strided] = None,
                 activation: Optional[str] = None, gate_per_group: bool = False) -> None:
    """For every group g: ``out_g = x_g . w[g]^T`` over the first ``rows`` rows, with ``w`` [G, N, K], x_g
    the K columns of group g of ``x`` and out_g the N columns of group g of ``out`` (a product per
    head over all tokens, in one launch).  With ``gate``: the result times sigmoid of the gate's
    entry at the same row and column of its group; ``gate_per_group``: the gate has ONE entry per row and
    group (a number per token and head).  True 32-bit arithmetic whatever the types."""
    _need(w, "grouped_gemm w", None, 3)
    G, N, K = w.shape
    _check_strided(x, "grouped_gemm x", rows, G, K)
    _check_strided(out, "grouped_gemm out", rows, G, N)
    epilogue = _EPILOGUES[activation] if activation else 0
    if gate is not None:
        if activation:
            raise KernelError("grouped_gemm: a gate or an activation, not both")
        _check_strided(gate, "grouped_gemm gate", rows, G, 1 if gate_per_group else N, x.tensor.dtype)
        epilogue = _EPILOGUE_GROUP_GATE if gate_per_group else _EPILOGUE_GATE
    if rows == 0:
        return
    _call("lc_gemm_grouped", x.pointer(), _dt(x.tensor), x.tensor.shape[1], x.group, _ptr(w), _dt(w),
          out.pointer(), _dt(out.tensor), out.tensor.shape[1], out.group, rows, N, K, G, None, None, None, 0,
          _grouped_tile(rows, N, G, x.tensor, w), epilogue, gate.pointer() if gate is not None else None,
          gate.tensor.shape[1] if gate is not None else 0, gate.group if gate is not None else 0, _stream())


def grouped_gemm_matrix_cores(on: bool) -> bool:
    """Whether grouped products of bfloat16 operands may take the bfloat16 matrix instruction (the
    default) or always run as true 32-bit products; for tests and tuning.  Returns the setting before."""
    return bool(library().lc_gemm_grouped_fast(1 if on else 0))


# ------------------------------------------------------------------------------ latent attention
def latent_prepare(proj: torch.Tensor, heads: int, dim: int, rot: int, rank: int, norm_weight: torch.Tensor,
                   eps: float, positions: torch.Tensor, rope_table: Optional[torch.Tensor], pairing: str,
                   cache: torch.Tensor, slots: Optional[torch.Tensor], qa: torch.Tensor,
                   q: Optional[torch.Tensor] = None, kv_column: Optional[int] = None) -> None:
    """What latent attention does to a step's projections ``proj`` [T, heads (dim + rot) + rank + rot
    (+ more)] before it attends: the ``rank`` entries behind the q heads, divided by their root mean
    square and times ``norm_weight``, and the ``rot`` entries behind them, rotated at the token's
    position, go to the token's row of ``cache`` [pages, page, rank + rot] (``slots`` [T]: page *
    page size + offset; negative or None: no write); every head's ``rot`` query entries, rotated,
    go to ``qa`` [T, heads (rank + rot)] behind the head's ``rank`` entries (which a product fills).
    ``rope_table`` [positions, rd] holds cosines, then sines; the first rd entries of a part are
    rotated, as pairs (2i, 2i + 1) (``pairing`` "interleaved") or (i, i + rd/2) ("half").
    With ``q`` [T, heads (dim + rot)] the heads' queries come from that tensor (a product of their own) and
    ``proj`` holds [rank | rot | ...] from ``kv_column`` on."""
    _need(proj, "latent_prepare proj", None, 2)
    T = proj.shape[0]
    if q is None:
        q, kv_column = proj, heads * (dim + rot)
    else:
        _need(q, "latent_prepare q", proj.dtype, 2)
        kv_column = int(kv_column or 0)
        if q.shape[0] != T or q.shape[1] < heads * (dim + rot):
            raise KernelError(f"latent_prepare: q {tuple(q.shape)} does not hold {heads} heads of {dim} + {rot}")
    _need(norm_weight, "latent norm weight", torch.float32, 1)
    if norm_weight.shape[0] != rank:
        raise KernelError(f"latent_prepare: norm weight has {norm_weight.shape[0]} entries for a latent of {rank}")
    _need(qa, "latent_prepare qa", proj.dtype, 2)
    if tuple(qa.shape) != (T, heads * (rank + rot)):
        raise KernelError(f"latent_prepare: qa {tuple(qa.shape)} is not [{T}, {heads * (rank + rot)}]")
    if proj.shape[1] < kv_column + rank + rot:
        raise KernelError(f"latent_prepare: rows of {proj.shape[1]} entries are too short")
    rd = 0
    if rope_table is not None and rot:
        _need(rope_table, "rope table", torch.float32, 2)
        _need(positions, "positions", torch.int32, 1)
        rd = rope_table.shape[1]
        if positions.shape[0] != T or rd > rot or rd % 2:
            raise KernelError("latent_prepare: positions or rotary table do not fit")
    else:
        rope_table = None
    if slots is not None:
        _need(cache, "latent cache", proj.dtype, 3)
        _need(slots, "slots", torch.int32, 1)
        if cache.shape[2] != rank + rot or slots.shape[0] != T:
            raise KernelError(f"latent_prepare: cache rows of {cache.shape[2]} entries, expected {rank + rot}")
    _call("lc_latent_prepare", _ptr(q), q.shape[1], ctypes.c_void_p(proj.data_ptr() + kv_column * proj.element_size()),
          _dt(proj), proj.shape[1], T, heads, dim, rot, rank, _ptr(norm_weight),
          float(eps), _ptr(positions), _ptr(rope_table), rd, 1 if pairing == "interleaved" else 0,
          _ptr(cache if slots is not None else None), _ptr(slots), _ptr(qa), _stream())


class _LatentSwitch(threading.local):
    on = True


_latent_fast = _LatentSwitch()      # per thread, like the library's own switches


def latent_matrix_cores(on: bool) -> bool:
    """Whether bfloat16 latent attention may run on the matrix-core kernel (tests run both); returns
    the setting before."""
    before = _latent_fast.on
    _latent_fast.on = bool(on)
    return before


LATENT_PLAN = "latent_attention"
LATENT_TILE = 16                # tokens of one work item of the matrix-core latent attention kernel


def plan_latent_attention(layout):
    """The work list of the matrix-core latent attention kernel for one step's batch (a planner in the
    sense of ``Part.batch_planner``): every request's tokens of this step cut into tiles of up to
    LATENT_TILE, four numbers each (first token row, tokens, request, first position); a request
    that brings one token is a tile of one token, which the kernel serves head by head."""
    tiles = []
    for r in range(layout.num_requests):
        first, n = layout.q_start[r], layout.q_start[r + 1] - layout.q_start[r]
        for t0 in range(0, n, LATENT_TILE):
            tiles.append((first + t0, min(LATENT_TILE, n - t0), r, layout.first_position[r] + t0))
    # the tiles that see the most keys first: the kernel's workgroups start in this order, and whoever
    # is done takes the longest that is left (the order changes no tile's result)
    tiles.sort(key=lambda t: -(t[3] + t[1]))
    return ({"tiles": np.asarray(tiles, dtype=np.int32).reshape(-1, 4)},
            {"any_portion": any(t[1] > 1 for t in tiles), "any_lone": any(t[1] == 1 for t in tiles),
             "num_tiles": len(tiles)})


def latent_attention(qa: torch.Tensor, heads: int, rank: int, rot: int, tok_req: torch.Tensor,
                     positions: torch.Tensor, block_table: torch.Tensor, cache: torch.Tensor, page_size: int,
                     scale: float, window: int = 0, plan=None, max_ctx: int = 0,
                     sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention in the latent's space: queries ``qa`` [T, heads (rank + rot)] against the cached
    rows [c | k_r] of the token's request (``cache`` [pages, page, rank + rot], ``block_table`` [R,
    blocks]), weights softmax(q . row * scale) over the positions j <= p (and j > p - window), result
    the weighted sum of the rows' first ``rank`` entries -> [T, heads rank].  ``sink`` float32 [heads]: the
    softmax's denominator of head h holds one more term, exp(sink[h]) (not scaled, no row)."""
    _need(qa, "latent_attention qa", None, 2)
    if sink is not None:
        _need(sink, "latent_attention sink", torch.float32, 1)
        if sink.shape[0] != heads:
            raise KernelError(f"latent_attention: {sink.shape[0]} sinks for {heads} heads")
    _need(cache, "latent cache", qa.dtype, 3)
    T = qa.shape[0]
    if qa.shape[1] != heads * (rank + rot) or cache.shape[2] != rank + rot or cache.shape[1] != page_size:
        raise KernelError(f"latent_attention: qa {tuple(qa.shape)} or cache {tuple(cache.shape)} do not fit "
                          f"{heads} heads of {rank} + {rot} and pages of {page_size}")
    _need(tok_req, "tok_req", torch.int32, 1)
    _need(positions, "positions", torch.int32, 1)
    _need(block_table, "block table", torch.int32, 2)
    if tok_req.shape[0] != T or positions.shape[0] != T:
        raise KernelError("latent_attention: one request and one position per token")
    out = torch.empty((T, heads * rank), dtype=qa.dtype, device=qa.device)
    if T == 0:
        return out
    lib = library()
    if (qa.dtype == torch.bfloat16 and plan is not None and _latent_fast.on
            and lib.lc_latent_bf16_supported(rank, rot)):
        # the matrix-core kernel, over the planner's tiles; few tiles: their keys are shared out
        tiles, any_portion = plan.arrays["tiles"], plan.info["any_portion"]
        workgroups = tiles.shape[0] * (-(-heads // 4) if any_portion else -(-heads // 64))
        most = block_table.shape[1] * page_size if max_ctx <= 0 else max_ctx
        splits = lib.lc_latent_bf16_splits(workgroups, min(most, window) if window > 0 else most)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty((T * heads * splits * rank,), dtype=torch.float32, device=qa.device)
            part_ml = torch.empty((T * heads * splits * 2,), dtype=torch.float32, device=qa.device)
        _call("lc_latent_attention_bf16", _ptr(qa), T, heads, rank, rot, _ptr(cache), _ptr(tiles), tiles.shape[0],
              1 if any_portion else 0, _ptr(block_table), block_table.shape[1], page_size, float(scale), int(window),
              _ptr(sink), _ptr(out), splits, _ptr(part_o), _ptr(part_ml), _stream())
        return out
    if qa.dtype == torch.bfloat16 and plan is not None and _latent_fast.on and rank * heads >= 1024:
        _say_once(("latent attention", rank, rot),
                  f"bfloat16 latent attention with a latent of {rank} and {rot} rotated entries has no matrix-core "
                  "kernel (a latent of a multiple of 16 up to 512, rows of a multiple of 8 up to 576, at most 128 rotated entries): the general "
                  "kernel runs, correct and many times slower")
    _call("lc_latent_attention", _ptr(qa), _dt(qa), T, heads, rank, rot, _ptr(cache), _ptr(tok_req),
          _ptr(positions), _ptr(block_table), block_table.shape[1], page_size, float(scale), int(window),
          _ptr(sink), _ptr(out), _stream())
    return out


# ------------------------------------------------------------------------------ routed experts
@dataclass
class Routing:
    """A step's routing, all on the device: ``ids`` and ``weights`` [T, top] (the chosen experts, best
    first, and what their outputs count); the (token, choice) pairs sorted by expert: ``row_start``
    and ``tile_start`` [E + 1], ``sorted_token`` [T top] and ``entry_row`` [T top]."""

    ids: torch.Tensor
    weights: torch.Tensor
    row_start: torch.Tensor
    tile_start: torch.Tensor
    sorted_token: torch.Tensor
    entry_row: torch.Tensor
    experts: int
    tile: int                   # rows of a tile of the sorted rows: what tile_start counts
    max_tiles: int


def moe_route(logits: torch.Tensor, top: int, renormalise: bool = True, eps: float = 1e-20,
              large_tiles: bool = False) -> Routing:
    """From the router's float32 ``logits`` [T, E]: softmax over all experts, the ``top`` largest scores of
    every token, divided by their sum + ``eps`` where ``renormalise``, and the lists that sort the
    (token, choice) pairs by expert for :func:`moe_experts`.  ``large_tiles``: the experts' products will
    take tiles of 128 rows (:func:`moe_large_tiles` says whether they do)."""
    _need(logits, "router logits", torch.float32, 2)
    T, E = logits.shape
    dev = logits.device
    ids = torch.empty((T, top), dtype=torch.int32, device=dev)
    weights = torch.empty((T, top), dtype=torch.float32, device=dev)
    _call("lc_moe_route", _ptr(logits), T, E, top, 1 if renormalise else 0, float(eps), _ptr(ids), _ptr(weights),
          _stream())
    # few rows an expert: tiles of 16 rows; many, and the caller's products take them: of 128; else of 64
    tile = 16 if T * top <= 16 * E else 128 if (large_tiles and T * top >= 192 * E) else 64
    lists = torch.empty((2 * (E + 1) + 2 * T * top,), dtype=torch.int32, device=dev)
    row_start, tile_start = lists[:E + 1], lists[E + 1:2 * (E + 1)]
    sorted_token, entry_row = lists[2 * (E + 1):2 * (E + 1) + T * top], lists[2 * (E + 1) + T * top:]
    _call("lc_moe_lists", _ptr(ids), T, top, E, tile, _ptr(row_start), _ptr(tile_start), _ptr(sorted_token),
          _ptr(entry_row), _stream())
    return Routing(ids, weights, row_start, tile_start, sorted_token, entry_row, E, tile, (T * top) // tile + E)


def moe_route_sigmoid(logits: torch.Tensor, top: int, correction: Optional[torch.Tensor] = None, groups: int = 1,
                      keep: int = 1, scale: float = 1.0, large_tiles: bool = False) -> Routing:
    """As :func:`moe_route`, with scores s = sigmoid(logits): the ``top`` largest of s + ``correction`` [E] are
    chosen (the lower index wins a tie) and weigh s * ``scale``, not renormalised.  ``groups`` > 1: the experts
    form that many equal groups of neighbours, a group ranks by the sum of its two largest s + correction, and
    only experts of the ``keep`` best groups can be chosen."""
    _need(logits, "router logits", torch.float32, 2)
    T, E = logits.shape
    if correction is not None:
        _need(correction, "router correction", torch.float32, 1)
        if correction.shape[0] != E:
            raise KernelError(f"moe_route_sigmoid: a correction of {correction.shape[0]} entries for {E} experts")
    dev = logits.device
    ids = torch.empty((T, top), dtype=torch.int32, device=dev)
    weights = torch.empty((T, top), dtype=torch.float32, device=dev)
    _call("lc_moe_route_sigmoid", _ptr(logits), _ptr(correction), T, E, top, int(groups), int(keep), float(scale),
          _ptr(ids), _ptr(weights), _stream())
    tile = 16 if T * top <= 16 * E else 128 if (large_tiles and T * top >= 192 * E) else 64
    lists = torch.empty((2 * (E + 1) + 2 * T * top,), dtype=torch.int32, device=dev)
    row_start, tile_start = lists[:E + 1], lists[E + 1:2 * (E + 1)]
    sorted_token, entry_row = lists[2 * (E + 1):2 * (E + 1) + T * top], lists[2 * (E + 1) + T * top:]
    _call("lc_moe_lists", _ptr(ids), T, top, E, tile, _ptr(row_start), _ptr(tile_start), _ptr(sorted_token),
          _ptr(entry_row), _stream())
    return Routing(ids, weights, row_start, tile_start, sorted_token, entry_row, E, tile, (T * top) // tile + E)


def moe_large_tiles(x_dtype: torch.dtype, up: torch.Tensor, down: torch.Tensor) -> bool:
    """Whether both of the experts' products (weights ``up`` [E, I, H], ``down`` [E, H, I]) can run in tiles
    of 128 rows: bfloat16 operands whose rows are whole 16-byte pieces, 128 columns at least."""
    if x_dtype != torch.bfloat16 or up.dtype != torch.bfloat16 or down.dtype != torch.bfloat16:
        return False
    (_, I, H) = up.shape
    return bool(I % 8 == 0 and H % 8 == 0 and I >= 128 and H >= 128
                and library().lc_gemm_grouped_takes_tile(128, DT_BF16, DT_BF16))


def moe_experts(x: torch.Tensor, w: torch.Tensor, routing: Routing, out_dtype: torch.dtype,
                activation: Optional[str] = None, gather: bool = False) -> torch.Tensor:
    """One of the experts' two products over the sorted rows: sorted row m, which belongs to expert e,
    becomes ``act(x[m] . w[e]^T)`` with ``w`` [E, N, K]; ``gather``: ``x`` has a row per token and sorted
    row m reads its token's.  -> [T top, N]"""
    _need(x, "moe_experts x", None, 2)
    _need(w, "moe_experts w", None, 3)
    E, N, K = w.shape
    rows = routing.sorted_token.shape[0]
    if E != routing.experts or x.shape[1] != K or (not gather and x.shape[0] != rows):
        raise KernelError(f"moe_experts: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit the routing")
    out = torch.empty((rows, N), dtype=out_dtype, device=x.device)
    if rows:
        _call("lc_gemm_grouped", _ptr(x), _dt(x), K, 0, _ptr(w), _dt(w), _ptr(out), _dt(out), N, 0, rows, N, K, E,
              _ptr(routing.sorted_token if gather else None), _ptr(routing.row_start), _ptr(routing.tile_start),
              routing.max_tiles, routing.tile, _EPILOGUES[activation] if activation else 0,
              None, 0, 0, _stream())
    return out


def moe_combine(y: torch.Tensor, routing: Routing, out_dtype: torch.dtype) -> torch.Tensor:
    """``out[t] = sum_k weights[t, k] * y[row of token t's k-th choice]`` from float32 ``y`` [T top, n]."""
    _need(y, "moe_combine y", torch.float32, 2)
    T, top = routing.ids.shape
    if y.shape[0] != T * top:
        raise KernelError(f"moe_combine: {y.shape[0]} rows for {T} tokens of {top} choices")
    out = torch.empty((T, y.shape[1]), dtype=out_dtype, device=y.device)
    _call("lc_moe_combine", _ptr(y), _ptr(routing.weights), _ptr(routing.entry_row), T, top, y.shape[1], _ptr(out),
          _dt(out), _stream())
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


# ------------------------------------------------------------------------------ layer norm, position vector
@dataclass
class NormedBranch:
    """A branch's output ``x`` [T, n] that is to pass a layer norm (``weight``, ``bias``, ``eps``)
    before it is added to the residual stream.  :func:`layer_norm` takes it as the stream's pending
    addition and does both in its kernel; anyone else gets the normed tensor from ``value()``."""

    x: torch.Tensor
    weight: torch.Tensor
    bias: torch.Tensor
    eps: float

    def value(self) -> torch.Tensor:
        return layer_norm_act(self.x, self.weight, self.bias, self.eps)


def layer_norm(h: torch.Tensor, delta, weight: torch.Tensor, bias: torch.Tensor, eps: float,
               out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, branch_scale: float = 1.0) -> torch.Tensor:
    """Layer norm ``(v - mean) / sqrt(var + eps) * weight + bias`` of the float32 residual stream ``h``
    [T, n] with the pending addition ``delta`` taken in first (v = h + branch_scale delta); ``delta`` may be a
    :class:`NormedBranch`, which is normed with its own weights before it is added.  Without ``rows``:
    ``h`` becomes v in place and every row is normed; with ``rows`` (int32 [R]): only those rows, ``h``
    stays as it is."""
    _need(h, "layer_norm h", torch.float32, 2)
    _need(weight, "layer_norm weight", torch.float32, 1)
    _need(bias, "layer_norm bias", torch.float32, 1)
    T, n = h.shape
    if weight.shape[0] != n or bias.shape[0] != n:
        raise KernelError(f"layer_norm: weight and bias must have {n} entries")
    post_w = post_b = None
    post_eps = 0.0
    if isinstance(delta, NormedBranch):
        post_w, post_b, post_eps = delta.weight, delta.bias, delta.eps
        _need(post_w, "layer_norm branch weight", torch.float32, 1)
        _need(post_b, "layer_norm branch bias", torch.float32, 1)
        if post_w.shape[0] != n or post_b.shape[0] != n:
            raise KernelError(f"layer_norm: the branch's weight and bias must have {n} entries")
        delta = delta.x
    delta = value(delta)
    if delta is not None:
        _need(delta, "layer_norm delta", None, 2)
        if tuple(delta.shape) != (T, n):
            raise KernelError(f"layer_norm: delta {tuple(delta.shape)} does not match h {(T, n)}")
    if rows is not None:
        _need(rows, "layer_norm rows", torch.int32, 1)
    R = T if rows is None else rows.shape[0]
    out = torch.empty((R, n), dtype=out_dtype, device=h.device)
    if R:
        _call("lc_layer_norm", _ptr(h), _ptr(delta), _dt(delta) if delta is not None else DT_F32, float(branch_scale),
              _ptr(post_w),
              _ptr(post_b), float(post_eps), _ptr(rows), _ptr(weight), _ptr(bias), float(eps), _ptr(out), _dt(out),
              R, n, 1 if (rows is None and delta is not None) else 0, T, _stream())
    return out


def layer_norm_act(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    """Layer norm over the last dimension of an activation tensor, in its dtype."""
    _need(x, "layer_norm_act x")
    _need(weight, "layer_norm_act weight", torch.float32, 1)
    _need(bias, "layer_norm_act bias", torch.float32, 1)
    n = x.shape[-1]
    if weight.shape[0] != n or bias.shape[0] != n:
        raise KernelError(f"layer_norm_act: weight and bias must have {n} entries")
    out = torch.empty_like(x)
    rows = x.numel() // n
    if rows:
        _call("lc_layer_norm", None, _ptr(x), _dt(x), 1.0, _ptr(weight), _ptr(bias), float(eps), None, None, None,
              0.0, _ptr(out), _dt(out), rows, n, 0, rows, _stream())
    return out


def embedding_sinusoid(ids: torch.Tensor, table: torch.Tensor, positions: torch.Tensor,
                       frequencies: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, H]: row ``ids[t]`` of ``table`` times ``scale`` plus the position vector of
    ``positions[t]``: entry 2i is sin(p f_i), entry 2i + 1 cos(p f_i), ``frequencies`` float32 [ceil(H/2)]."""
    _need(ids, "embedding ids", torch.int32, 1)
    _need(positions, "embedding positions", torch.int32, 1)
    _need(table, "embedding table", None, 2)
    _need(frequencies, "embedding frequencies", torch.float32, 1)
    T, (V, H) = ids.shape[0], table.shape
    if positions.shape[0] != T or frequencies.shape[0] != (H + 1) // 2:
        raise KernelError("embedding_sinusoid: one position per id and one frequency per pair of entries")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    if T:
        _call("lc_embedding_sinusoid", _ptr(ids), _ptr(positions), _ptr(table), _dt(table), _ptr(frequencies),
              _ptr(out), T, H, V, float(scale), _stream())
    return out


# ------------------------------------------------------------------------------ gated activations
GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def gated_activation(gu: torch.Tensor, kind: str) -> torch.Tensor:
    """``gu`` [T, 2 I] (gate columns, then up columns) -> act(gate) * up, [T, I]; float32 arithmetic."""
    _need(gu, "gated_activation input", None, 2)
    T, two_i = gu.shape
    if two_i % 2:
        raise KernelError("gated_activation: the input needs an even number of columns")
    out = torch.empty((T, two_i // 2), dtype=gu.dtype, device=gu.device)
    if T:
        _call("lc_gated_activation", _ptr(gu), _ptr(out), _dt(gu), T, two_i // 2, GATE_ACTIVATIONS[kind], _stream())
    return out


def gated_activation_weighted(gu: torch.Tensor, kind: str, routing: "Routing") -> torch.Tensor:
    """As :func:`gated_activation` over the experts' sorted rows, each row's gate and up entries first times
    the weight of its (token, choice) pair: ``act(w gate) * (w up)``, which is what a gated expert makes of
    w times its input."""
    _need(gu, "gated_activation_weighted input", None, 2)
    rows, two_i = gu.shape
    if two_i % 2 or rows != routing.entry_row.shape[0]:
        raise KernelError("gated_activation_weighted: the rows do not fit the routing")
    out = torch.empty((rows, two_i // 2), dtype=gu.dtype, device=gu.device)
    if rows:
        _call("lc_gated_activation_weighted", _ptr(gu), _ptr(out), _dt(gu), _ptr(routing.weights),
              _ptr(routing.entry_row), rows, two_i // 2, GATE_ACTIVATIONS[kind], _stream())
    return out


# ------------------------------------------------------------------------------ attention with heads in slots
def attention_head_slot(size: int) -> int:
    """The head size that the cache and the attention kernels use for heads of up to ``size`` entries:
    the next size the matrix-core kernels are built for, else the next multiple of 16."""
    for slot in (32, 64, 96, 128):
        if size <= slot:
            return slot
    if size > 256:
        raise KernelError(f"attention: heads of {size} entries are above the kernels' 256")
    return -(-size // 16) * 16


def head_norm_write(proj: torch.Tensor, nh: int, nkv: int, d: int, dv: int, slot: int,
                    q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                    head_scale: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_size: int) -> torch.Tensor:
    """From the raw projections ``proj`` [T, nh d + nkv d + nkv dv] (queries, keys, values; ``nkv`` = 0:
    queries only): every q and k head divided by its root mean square over its ``d`` entries (eps
    inside the root) and multiplied by its weight [d] (None: no norm), q head h also by
    ``head_scale[h]``.  Returns q as [T, nh slot] (zeros behind the d entries); k and v go to the
    cache slot ``slots[t]`` (negative: no write) as heads of ``slot`` entries, zeros behind theirs:
    keys [pages, nkv, page_size, slot], values [pages, nkv, slot, page_size]."""
    _need(proj, "head_norm_write proj", None, 2)
    T = proj.shape[0]
    if proj.shape[1] != nh * d + nkv * (d + dv):
        raise KernelError(f"head_norm_write: proj has {proj.shape[1]} columns, expected {nh * d + nkv * (d + dv)}")
    if d > slot or dv > slot:
        raise KernelError(f"head_norm_write: heads of {d}/{dv} do not fit a slot of {slot}")
    for wt, name in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if wt is not None:
            _need(wt, name, torch.float32, 1)
            if wt.shape[0] != d:
                raise KernelError(f"{name} has {wt.shape[0]} entries for head size {d}")
    if head_scale is not None:
        _need(head_scale, "head scale", torch.float32, 1)
        if head_scale.shape[0] != nh:
            raise KernelError(f"head scale has {head_scale.shape[0]} entries for {nh} heads")
    if nkv and slots is not None and k_cache is not None:
        _need(k_cache, "k cache", proj.dtype, 4)
        _need(v_cache, "v cache", proj.dtype, 4)
        _need(slots, "slots", torch.int32, 1)
        _check_caches(k_cache, v_cache, nkv, page_size, slot)
        if slots.shape[0] != T:
            raise KernelError("slots do not match the tokens")
    else:
        k_cache = v_cache = slots = None
    q = torch.empty((T, nh * slot), dtype=proj.dtype, device=proj.device)
    if T:
        _call("lc_head_norm_write", _ptr(proj), _dt(proj), T, nh, nkv, d, dv, slot, _ptr(q_weight), _ptr(k_weight),
              float(eps), _ptr(head_scale), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(slots), page_size,
              k_cache.shape[0] if k_cache is not None else 0, _stream())
    return q


# ------------------------------------------------------------------------------ delta rules
DELTA_MAX_KEY = 256        # key channels of a head that the scan kernel holds (16 a lane, 16 lanes a column)
CONV_MAX_TAPS = 16


def check_delta_sizes(what: str, key_dim: int, value_dim: int, taps: int = 1) -> None:
    if not 1 <= key_dim <= DELTA_MAX_KEY:
        raise KernelError(f"{what}: a head's {key_dim} key channels are outside the scan kernel's 1..{DELTA_MAX_KEY}")
    if value_dim < 1:
        raise KernelError(f"{what}: a head needs value channels")
    if not 1 <= taps <= CONV_MAX_TAPS:
        raise KernelError(f"{what}: {taps} taps are outside the convolution kernel's 1..{CONV_MAX_TAPS}")


def general_delta_prepare(proj: torch.Tensor, heads: int, dim: int, inner: int, decay_out: torch.Tensor,
                          decay_bias: torch.Tensor, removal_bias: torch.Tensor, unit_eps: float,
                          decay_scale: float):
    """The scan's inputs of the generalized delta rule from the float32 projections ``proj``
    [T, 5 n + inner], n = heads dim: columns r | k | v | gate | removal | decay_in.
    decay = exp(-decay_scale sigmoid(decay_out tanh(decay_in) + decay_bias)), a = sigmoid(removal +
    removal_bias), u = k / sqrt(sum k^2 + unit_eps) per head.  Returns ``coef`` float32 [5, T, n]
    (decay, probe = u, removal = a u, write = k, read = r) and ``v`` float32 [T, n]."""
    _need(proj, "general_delta proj", torch.float32, 2)
    n = heads * dim
    T = proj.shape[0]
    if proj.shape[1] != 5 * n + inner:
        raise KernelError(f"general_delta_prepare: proj has {proj.shape[1]} columns, expected {5 * n + inner}")
    _need(decay_out, "decay_out", torch.float32, 2)
    _need(decay_bias, "decay_bias", torch.float32, 1)
    _need(removal_bias, "removal_bias", torch.float32, 1)
    if tuple(decay_out.shape) != (n, inner) or decay_bias.shape[0] != n or removal_bias.shape[0] != n:
        raise KernelError("general_delta_prepare: the decay's and the removal's tensors do not fit the heads")
    coef = torch.empty((5, T, n), dtype=torch.float32, device=proj.device)
    v = torch.empty((T, n), dtype=torch.float32, device=proj.device)
    if T:
        _call("lc_general_delta_prepare", _ptr(proj), T, heads, dim, inner, _ptr(decay_out), _ptr(decay_bias),
              _ptr(removal_bias), float(unit_eps), float(decay_scale), _ptr(coef), _ptr(v), _stream())
    return coef, v


def gated_delta_prepare(proj: torch.Tensor, tail: torch.Tensor, taps: torch.Tensor, rate_log: torch.Tensor,
                        rate_bias: torch.Tensor, heads: int, kv_heads: int, key_dim: int, value_dim: int,
                        num_taps: int, unit_eps: float, tok_req: torch.Tensor, q_offsets: torch.Tensor,
                        slot_ids: torch.Tensor):
    """The scan's inputs of the gated delta rule from the float32 projections ``proj`` [T, C + nv + 2
    heads]: columns q | k | v (the C = 2 kv_heads key_dim + heads value_dim channels that pass the
    convolutions) | gate | beta | rate.  Channel c of token t becomes silu(sum_j taps[c, K - 1 - j] x[t -
    j, c]); inputs from before the step come from ``tail`` [slots, K - 1, C] (the request's last K - 1
    inputs, oldest first), zeros before the sequence's start.  q and k are made unit vectors per head
    (q also times key_dim^-1/2); g = exp(-exp(rate_log) softplus(rate + rate_bias)), beta = sigmoid(beta).
    Returns ``coef`` float32 [5, T, heads key_dim] (decay = g, probe = g k, removal = beta k, write = beta k,
    read = q) and ``v`` float32 [T, heads value_dim]."""
    _need(proj, "gated_delta proj", torch.float32, 2)
    T = proj.shape[0]
    C = 2 * kv_heads * key_dim + heads * value_dim
    if proj.shape[1] != C + heads * value_dim + 2 * heads:
        raise KernelError(f"gated_delta_prepare: proj has {proj.shape[1]} columns, expected "
                          f"{C + heads * value_dim + 2 * heads}")
    _need(taps, "conv taps", torch.float32, 2)
    _need(tail, "conv tail", torch.float32, 3)
    if tuple(taps.shape) != (C, num_taps) or tuple(tail.shape[1:]) != (num_taps - 1, C):
        raise KernelError("gated_delta_prepare: taps or tail do not fit the channels")
    _need(rate_log, "rate_log", torch.float32, 1)
    _need(rate_bias, "rate_bias", torch.float32, 1)
    _need(tok_req, "tok_req", torch.int32, 1)
    _need(q_offsets, "q_offsets", torch.int32, 1)
    _need(slot_ids, "slot_ids", torch.int32, 1)
    if rate_log.shape[0] != heads or rate_bias.shape[0] != heads or tok_req.shape[0] != T:
        raise KernelError("gated_delta_prepare: per-head vectors or the token map do not fit")
    coef = torch.empty((5, T, heads * key_dim), dtype=torch.float32, device=proj.device)
    v = torch.empty((T, heads * value_dim), dtype=torch.float32, device=proj.device)
    if T:
        _call("lc_gated_delta_prepare", _ptr(proj), T, heads, kv_heads, key_dim, value_dim, num_taps, _ptr(taps),
              _ptr(tail), tail.shape[0], _ptr(rate_log), _ptr(rate_bias), float(unit_eps), _ptr(tok_req),
              _ptr(q_offsets), _ptr(slot_ids), _ptr(coef), _ptr(v), _stream())
    return coef, v


def conv_tail_update(proj: torch.Tensor, tail: torch.Tensor, channels: int, num_taps: int,
                     q_offsets: torch.Tensor, slot_ids: torch.Tensor, num_requests: int) -> None:
    """After a step: ``tail`` [slots, K - 1, C] of every request of the batch becomes the last K - 1
    rows of (its old tail, then the first ``channels`` columns of the request's rows of ``proj``)."""
    _need(proj, "conv_tail_update proj", torch.float32, 2)
    _need(tail, "conv tail", torch.float32, 3)
    if num_taps <= 1 or num_requests == 0:
        return
    if tuple(tail.shape[1:]) != (num_taps - 1, channels) or proj.shape[1] < channels:
        raise KernelError("conv_tail_update: the tail does not fit the channels")
    if q_offsets.shape[0] != num_requests + 1 or slot_ids.shape[0] != num_requests:
        raise KernelError("conv_tail_update: the request lists do not fit")
    _call("lc_conv_tail_update", _ptr(proj), proj.shape[1], proj.shape[0], _ptr(tail), tail.shape[0], channels,
          num_taps, _ptr(q_offsets), _ptr(slot_ids), num_requests, _stream())


def delta_scan(coef: torch.Tensor, v: torch.Tensor, state: torch.Tensor, q_offsets: torch.Tensor,
               slot_ids: torch.Tensor, num_requests: int, heads: int, key_dim: int, value_dim: int) -> torch.Tensor:
    """The delta-rule recurrence over every request's tokens in order, per head:
    ``S <- diag(decay) S - removal (probe^T S) + write v^T`` (the probe meets S as the last token left it, before the decay), ``o = S^T read``.
    ``coef`` float32 [5, T, heads key_dim] holds decay, probe, removal, write, read, or, for the recurrence
    without a removal term, [3, T, heads key_dim]: decay, write, read; ``v`` float32
    [T, heads value_dim]; ``state`` float32 [slots, heads, value_dim, key_dim] (S transposed: a value
    channel's key rows lie in a row) is read at the request's slot before its first token of the step
    and written after its last.  -> float32 [T, heads value_dim]."""
    _need(coef, "delta_scan coef", torch.float32, 3)
    _need(v, "delta_scan v", torch.float32, 2)
    _need(state, "delta_scan state", torch.float32, 4)
    T = v.shape[0]
    if coef.shape[0] not in (5, 3) or tuple(coef.shape[1:]) != (T, heads * key_dim) or v.shape[1] != heads * value_dim:
        raise KernelError("delta_scan: coef or v do not fit the heads")
    if tuple(state.shape[1:]) != (heads, value_dim, key_dim):
        raise KernelError(f"delta_scan: state {tuple(state.shape)} does not fit [slots, {heads}, {value_dim}, {key_dim}]")
    _need(q_offsets, "q_offsets", torch.int32, 1)
    _need(slot_ids, "slot_ids", torch.int32, 1)
    if q_offsets.shape[0] != num_requests + 1 or slot_ids.shape[0] != num_requests:
        raise KernelError("delta_scan: the request lists do not fit")
    check_delta_sizes("delta_scan", key_dim, value_dim)
    out = torch.empty((T, heads * value_dim), dtype=torch.float32, device=v.device)
    if T:
        _call("lc_delta_scan", _ptr(coef), coef.shape[0], _ptr(v), _ptr(state), state.shape[0], _ptr(out), _ptr(q_offsets),
              _ptr(slot_ids), num_requests, T, heads, key_dim, value_dim, _stream())
    return out


HEAD_GATES = {"sigmoid": 0, "silu": 1}


def head_gate_norm(o: torch.Tensor, gates: torch.Tensor, gate_column: int, weight: torch.Tensor,
                   weight_per_head: bool, eps: float, gate: str, heads: int, dim: int,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Every head of float32 ``o`` [T, heads dim] divided by its root mean square (eps inside the root),
    times ``weight`` ([heads dim] where ``weight_per_head``, else [dim] for all heads), times
    ``gate``(g) with g the float32 columns ``gate_column`` .. + heads dim of ``gates``.  -> [T, heads dim]."""
    _need(o, "head_gate_norm o", torch.float32, 2)
    _need(gates, "head_gate_norm gates", torch.float32, 2)
    _need(weight, "head_gate_norm weight", torch.float32, 1)
    T, n = o.shape
    if n != heads * dim or gates.shape[0] != T or gate_column + n > gates.shape[1]:
        raise KernelError("head_gate_norm: o or the gates do not fit the heads")
    if weight.shape[0] != (n if weight_per_head else dim):
        raise KernelError("head_gate_norm: the weight does not fit the heads")
    out = torch.empty((T, n), dtype=out_dtype, device=o.device)
    if T:
        _call("lc_head_gate_norm", _ptr(o), _ptr(gates), gates.shape[1], gate_column, _ptr(weight),
              1 if weight_per_head else 0, float(eps), HEAD_GATES[gate], T, heads, dim, _ptr(out), _dt(out), _stream())
    return out


# ------------------------------------------------------------------------------ routing by logits, shared expert
def moe_route_logits(logits: torch.Tensor, experts: int, top: int, bias: Optional[torch.Tensor] = None,
                     large_tiles: bool = False) -> Routing:
    """As :func:`moe_route`, from the first ``experts`` columns of float32 ``logits`` [T, >= experts] with
    ``bias`` [experts] added: the ``top`` largest logits are chosen (the lower index wins a tie) and
    weigh as the softmax over the chosen logits alone."""
    _need(logits, "router logits", torch.float32, 2)
    T, cols = logits.shape
    E = experts
    if cols < E:
        raise KernelError(f"moe_route_logits: {cols} columns for {E} experts")
    if bias is not None:
        _need(bias, "router bias", torch.float32, 1)
        if bias.shape[0] != E:
            raise KernelError(f"moe_route_logits: a bias of {bias.shape[0]} entries for {E} experts")
    dev = logits.device
    ids = torch.empty((T, top), dtype=torch.int32, device=dev)
    weights = torch.empty((T, top), dtype=torch.float32, device=dev)
    _call("lc_moe_route_logits", _ptr(logits), cols, _ptr(bias), T, E, top, _ptr(ids), _ptr(weights), _stream())
    tile = 16 if T * top <= 16 * E else 128 if (large_tiles and T * top >= 192 * E) else 64
    lists = torch.empty((2 * (E + 1) + 2 * T * top,), dtype=torch.int32, device=dev)
    row_start, tile_start = lists[:E + 1], lists[E + 1:2 * (E + 1)]
    sorted_token, entry_row = lists[2 * (E + 1):2 * (E + 1) + T * top], lists[2 * (E + 1) + T * top:]
    _call("lc_moe_lists", _ptr(ids), T, top, E, tile, _ptr(row_start), _ptr(tile_start), _ptr(sorted_token),
          _ptr(entry_row), _stream())
    return Routing(ids, weights, row_start, tile_start, sorted_token, entry_row, E, tile, (T * top) // tile + E)


def moe_combine_shared(y: torch.Tensor, routing: Routing, shared: Optional[torch.Tensor],
                       gates: Optional[torch.Tensor], gate_column: int, out_dtype: torch.dtype,
                       weighted: bool = True) -> torch.Tensor:
    """:func:`moe_combine` plus ``sigmoid(gates[t, gate_column]) * shared[t]`` (``gates`` float32; without
    ``gates`` the shared rows count as they are, without ``shared`` there are none).  Not ``weighted``: every
    choice counts 1 (the weights have been applied on the experts' way in)."""
    _need(y, "moe_combine_shared y", torch.float32, 2)
    T, top = routing.ids.shape
    n = y.shape[1]
    if shared is not None:
        _need(shared, "moe_combine_shared shared", None, 2)
    if gates is not None:
        _need(gates, "moe_combine_shared gates", torch.float32, 2)
        if shared is None or gates.shape[0] != T or not 0 <= gate_column < gates.shape[1]:
            raise KernelError("moe_combine_shared: the gates do not fit the rows")
    if y.shape[0] != T * top or (shared is not None and tuple(shared.shape) != (T, n)):
        raise KernelError("moe_combine_shared: the operands do not fit the routing")
    out = torch.empty((T, n), dtype=out_dtype, device=y.device)
    if T:
        _call("lc_moe_combine_shared", _ptr(y), _ptr(routing.weights if weighted else None), _ptr(routing.entry_row),
              T, top, n, _ptr(shared), _dt(shared) if shared is not None else DT_F32, _ptr(gates),
              gates.shape[1] if gates is not None else 0, gate_column, _ptr(out), _dt(out), _stream())
    return out


# ------------------------------------------------------------------------------ lightning attention
def lightning_prepare(proj: torch.Tensor, heads: int, key_dim: int, value_dim: int, decay: torch.Tensor):
    """The scan's inputs of lightning attention from the float32 projections ``proj`` [T, >= heads (2 key_dim
    + value_dim)]: columns q | k | v.  Returns ``coef`` float32 [3, T, heads key_dim] (decay = ``decay``[head]
    in every channel, write = silu(k), read = silu(q): no removal term) and ``v`` = silu(v) float32
    [T, heads value_dim]."""
    _need(proj, "lightning proj", torch.float32, 2)
    _need(decay, "lightning decay", torch.float32, 1)
    T = proj.shape[0]
    if proj.shape[1] < heads * (2 * key_dim + value_dim) or decay.shape[0] != heads:
        raise KernelError(f"lightning_prepare: proj {tuple(proj.shape)} or decay do not fit {heads} heads")
    coef = torch.empty((3, T, heads * key_dim), dtype=torch.float32, device=proj.device)
    v = torch.empty((T, heads * value_dim), dtype=torch.float32, device=proj.device)
    if T:
        _call("lc_lightning_prepare", _ptr(proj), proj.shape[1], T, heads, key_dim, value_dim, _ptr(decay), _ptr(coef),
              _ptr(v), _stream())
    return coef, v


def lightning_readout(o: torch.Tensor, gates: torch.Tensor, gate_column: int, weight: torch.Tensor, eps: float,
                      out_dtype: torch.dtype) -> torch.Tensor:
    """Every row of float32 ``o`` [T, n] (all heads side by side) divided by its root mean square (eps inside
    the root), times ``weight`` [n], times sigmoid(g) with g the float32 columns ``gate_column`` .. + n of
    ``gates``.  -> [T, n] of ``out_dtype``."""
    _need(o, "lightning_readout o", torch.float32, 2)
    _need(gates, "lightning_readout gates", torch.float32, 2)
    _need(weight, "lightning_readout weight", torch.float32, 1)
    T, n = o.shape
    if gates.shape[0] != T or gate_column < 0 or gate_column + n > gates.shape[1] or weight.shape[0] != n:
        raise KernelError("lightning_readout: the gates or the weight do not fit the rows")
    out = torch.empty((T, n), dtype=out_dtype, device=o.device)
    if T:
        _call("lc_lightning_readout", _ptr(o), _ptr(gates), gates.shape[1], gate_column, _ptr(weight), float(eps), T, n,
              _ptr(out), _dt(out), _stream())
    return out


# ------------------------------------------------------------------------------ masked attention
MASKED_ATTENTION_MAX = 256      # entries of a key head and of a value head at most
SHORT_CONV_MAX_TAPS = 16


class _MaskedSwitch(threading.local):
    on = True


_masked_fast = _MaskedSwitch()


class _MaskedSplits(threading.local):
    forced = 0


_masked_splits = _MaskedSplits()


def masked_attention_force_splits(count: int) -> int:
    """Tests and tuning: over how many workgroups a lone token's keys are shared out at most where a step allows
    it (0: by the step's size; for the calling thread).  Returns the setting before."""
    before = _masked_splits.forced
    _masked_splits.forced = int(count)
    return before


def masked_attention_matrix_cores(on: bool) -> bool:
    """Tests and tuning: whether :func:`masked_attention` may take the matrix-core kernel (for the calling
    thread).  Returns the setting before."""
    before = _masked_fast.on
    _masked_fast.on = bool(on)
    return before


def attention_prepare_pairs(on: bool) -> bool:
    """Tests: whether :func:`attention_prepare` without the unit norm may take the kernel with a thread per pair of
    entries (for the calling thread).  Returns the setting before."""
    return bool(library().lc_attention_prepare_pairs(1 if on else 0))


def masked_attention_staged(on: bool) -> bool:
    """Tests and tuning: whether tiles of several tokens may take the matrix-core kernel that stages keys and values
    in LDS (for the calling thread).  Returns the setting before."""
    return bool(library().lc_masked_attention_bf16_staged(1 if on else 0))


def masked_attention_on_matrix_cores(dtype: torch.dtype, d: int, dv: int, page_size: int, maps: int) -> bool:
    """Whether the matrix-core kernel serves these sizes: bfloat16, key heads of a multiple of 8 up to 128 entries,
    value heads of a multiple of 16 up to 128, pages of a multiple of 16 tokens."""
    return dtype == torch.bfloat16 and bool(library().lc_masked_attention_bf16_supported(int(d), int(dv), int(page_size),
                                                                                        int(maps)))


def attention_prepare(proj: torch.Tensor, nq: int, nk: int, nv: int, d: int, dv: int, out_dtype: torch.dtype,
                      k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                      rows: Optional[torch.Tensor], taps: Optional[torch.Tensor] = None,
                      tail: Optional[torch.Tensor] = None, tok_req: Optional[torch.Tensor] = None,
                      q_offsets: Optional[torch.Tensor] = None, slot_ids: Optional[torch.Tensor] = None,
                      table: Optional[torch.Tensor] = None, rot: int = 0,
                      positions: Optional[torch.Tensor] = None, unit_eps: Optional[float] = None) -> torch.Tensor:
    """q, k and v of a step from the first (nq + nk) d + nv dv columns of the float32 projections ``proj`` (q heads
    | k heads | v heads).  ``taps`` float32 [columns, K]: every column first passes a causal convolution over time whose
    inputs from before the step come from ``tail`` float32 [slots, K - 1, columns] (the request's last K - 1
    inputs, oldest first).  ``table`` float32 [positions, rot] (cosines | sines): entries 2i, 2i + 1 of the first
    ``rot`` of every q and k head are rotated by angle i of the token's position.  ``unit_eps``: every q and k
    head is divided by its root mean square.  Returns q [T, nq d] of ``out_dtype``; k and v go to place ``rows[t]``
    (page * page size + place in the page; where ``rows`` is given and not negative) of ``k_cache`` [pages, page,
    nk d] and ``v_cache`` [pages, nv dv, page]."""
    _need(proj, "attention_prepare proj", torch.float32, 2)
    T, cols = proj.shape
    C = (nq + nk) * d + nv * dv
    if cols < C:
        raise KernelError(f"attention_prepare: proj has {cols} columns, fewer than the heads' {C}")
    if max(d, dv) > MASKED_ATTENTION_MAX:
        raise KernelError(f"attention_prepare: heads of {d}/{dv} entries are above {MASKED_ATTENTION_MAX}")
    K = 0
    if taps is not None:
        _need(taps, "conv taps", torch.float32, 2)
        K = taps.shape[1]
        if taps.shape[0] != C or not 1 <= K <= SHORT_CONV_MAX_TAPS:
            raise KernelError(f"attention_prepare: taps {tuple(taps.shape)} do not fit {C} columns")
        for t, what in ((tok_req, "tok_req"), (q_offsets, "q_offsets"), (slot_ids, "slot_ids")):
            _need(t, what, torch.int32, 1)
        if K > 1:
            _need(tail, "conv tail", torch.float32, 3)
            if tuple(tail.shape[1:]) != (K - 1, C):
                raise KernelError("attention_prepare: the tail does not fit the taps")
    if table is not None:
        _need(table, "rotary table", torch.float32, 2)
        _need(positions, "positions", torch.int32, 1)
        if table.shape[1] != rot or rot % 2 or rot > d:
            raise KernelError(f"attention_prepare: a table of {table.shape[1]} columns for {rot} rotated entries of {d}")
    if rows is not None:
        _need(rows, "cache rows", torch.int32, 1)
        if k_cache is None or v_cache is None or k_cache.dtype != out_dtype or v_cache.dtype != out_dtype:
            raise KernelError("attention_prepare: the cache must have the queries' dtype")
        if k_cache.dim() != 3 or v_cache.dim() != 3 or k_cache.shape[2] != nk * d or v_cache.shape[1] != nv * dv \
                or v_cache.shape[2] != k_cache.shape[1] or v_cache.shape[0] != k_cache.shape[0]:
            raise KernelError("attention_prepare: the cache does not fit the heads")
    q = torch.empty((T, nq * d), dtype=out_dtype, device=proj.device)
    if T:
        _call("lc_attention_prepare", _ptr(proj), cols, T, nq, nk, nv, d, dv, _ptr(taps), K, _ptr(tail),
              _ptr(tok_req), _ptr(q_offsets), _ptr(slot_ids), _ptr(table), int(rot), _ptr(positions),
              0 if unit_eps is None else 1, float(unit_eps or 0.0), _ptr(q), _ptr(k_cache if rows is not None else None),
              _ptr(v_cache if rows is not None else None), _dt(q), _ptr(rows),
              k_cache.shape[1] if rows is not None else 0, _stream())
    return q


def masked_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, tok_req: torch.Tensor,
                     positions: torch.Tensor, block_table: torch.Tensor, page_size: int, heads: int, kv_heads: int,
                     maps: int, d: int, dv: int, scale: float, chunk: int = 0, window: int = 0,
                     r1: Optional[torch.Tensor] = None, r2: Optional[torch.Tensor] = None,
                     sink: Optional[torch.Tensor] = None, subtract: float = 0.0, unit_eps: Optional[float] = None,
                     out_scale: float = 1.0, gate: Optional[torch.Tensor] = None, gate_column: int = 0,
                     plan=None, max_ctx: int = 0) -> torch.Tensor:
    """Attention of every token of the batch over its request's cached keys lo .. p (p its position; lo the start
    of its chunk of ``chunk`` positions, of its window of ``window``, or 0), float32 arithmetic.  ``q`` [T, heads
    maps d]; ``k_cache`` [pages, page, kv_heads maps d], ``v_cache`` [pages, page, kv_heads dv].  Scores are
    ``scale`` (q . k) minus ``r1[h] ln(1 + r2[h] (p - j))`` where the bias is given; ``sink`` float32 [heads] adds
    exp(sink[h]) to the softmax's denominator.  ``maps`` = 2: a head's two maps over the same values are combined as
    a_0 - ``subtract`` a_1.  ``unit_eps``: the head's output is divided by its root mean square and multiplied by
    ``out_scale``.  ``gate`` float32 [T, >= gate_column + heads dv]: the output times sigmoid of those columns.
    ``plan``: the step's tiles (:func:`plan_latent_attention`: up to 16 tokens of one request each); with them,
    bfloat16 operands of sizes the matrix-core kernel takes (:func:`masked_attention_on_matrix_cores`) go there;
    ``max_ctx`` (the longest request of the step) lets a step of few lone tokens share every token's keys out over
    several workgroups.  -> [T, heads dv] in q's dtype."""
    _need(q, "masked_attention q", None, 2)
    T = q.shape[0]
    if q.shape[1] != heads * maps * d:
        raise KernelError(f"masked_attention: q has {q.shape[1]} columns, expected {heads * maps * d}")
    _need(k_cache, "masked_attention keys", q.dtype, 3)
    _need(v_cache, "masked_attention values", q.dtype, 3)
    if tuple(k_cache.shape[1:]) != (page_size, kv_heads * maps * d) or tuple(v_cache.shape[1:]) != (kv_heads * dv, page_size):
        raise KernelError(f"masked_attention: keys {tuple(k_cache.shape)} and values {tuple(v_cache.shape)} do not fit "
                          f"pages of {page_size} with rows of {kv_heads * maps * d} and {kv_heads * dv}")
    _need(tok_req, "tok_req", torch.int32, 1)
    _need(positions, "positions", torch.int32, 1)
    _need(block_table, "block_table", torch.int32, 2)
    for vec, what in ((r1, "r1"), (r2, "r2"), (sink, "sink")):
        if vec is not None:
            _need(vec, f"masked_attention {what}", torch.float32, 1)
            if vec.shape[0] != heads:
                raise KernelError(f"masked_attention: {what} has {vec.shape[0]} entries for {heads} heads")
    if gate is not None:
        _need(gate, "masked_attention gate", torch.float32, 2)
        if gate.shape[0] != T or gate_column < 0 or gate_column + heads * dv > gate.shape[1]:
            raise KernelError("masked_attention: the gate does not fit the rows")
    out = torch.empty((T, heads * dv), dtype=q.dtype, device=q.device)
    if T and plan is not None and _masked_fast.on and masked_attention_on_matrix_cores(q.dtype, d, dv, page_size, maps):
        tiles = plan.arrays["tiles"]
        # a step of lone tokens that leaves most of the card idle: every token's key blocks over several workgroups (a
        # workgroup a CU in all), a workgroup keeping two blocks a wave at least
        zsplits, shares = 1, None
        if not plan.info.get("any_portion", True) and max_ctx > 0:
            reach = min(int(chunk) or max_ctx, int(window) or max_ctx, max_ctx)
            zsplits = max(1, min(_masked_splits.forced or 256 // max(1, tiles.shape[0] * kv_heads), 16, reach // 256))
            if zsplits > 1:
                words = library().lc_masked_attention_bf16_workspace(tiles.shape[0], heads, kv_heads, maps, dv, zsplits)
                shares = torch.empty((words,), dtype=torch.float32, device=q.device)
        _call("lc_masked_attention_bf16", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(tiles), tiles.shape[0],
              _ptr(block_table), block_table.shape[1], int(page_size), heads, kv_heads, maps, d, dv, float(scale),
              int(chunk), int(window), _ptr(r1), _ptr(r2), _ptr(sink), float(subtract), 0 if unit_eps is None else 1,
              float(unit_eps or 0.0), float(out_scale), _ptr(gate), gate.shape[1] if gate is not None else 0,
              int(gate_column), _ptr(out), _ptr(shares), zsplits, 1 if plan.info.get("any_portion", True) else 0,
              1 if plan.info.get("any_lone", True) else 0, _stream())
    elif T:
        _call("lc_masked_attention", _ptr(q), _ptr(k_cache), _ptr(v_cache), _dt(q), _ptr(tok_req), _ptr(positions),
              _ptr(block_table), block_table.shape[1], int(page_size), T, heads, kv_heads, maps, d, dv, float(scale),
              int(chunk), int(window), _ptr(r1), _ptr(r2), _ptr(sink), float(subtract), 0 if unit_eps is None else 1,
              float(unit_eps or 0.0), float(out_scale), _ptr(gate), gate.shape[1] if gate is not None else 0,
              int(gate_column), _ptr(out), _stream())
    return out


# ------------------------------------------------------------------------------ the state-space mixer
def state_space_prepare(proj: torch.Tensor, heads: int, groups: int, state: int, value_dim: int, taps: torch.Tensor,
                        bias: torch.Tensor, tail: Optional[torch.Tensor], dt_bias: torch.Tensor, a_log: torch.Tensor,
                        tok_req: torch.Tensor, q_offsets: torch.Tensor, slot_ids: torch.Tensor):
    """The scan's inputs of the state-space mixer from the float32 projections ``proj`` [T, 2 heads value_dim + 2
    groups state + heads]: columns x | B | C | z | dt.  x, B and C pass the convolution ``taps`` [C, K] (+ ``bias``,
    then SiLU; inputs from before the step from ``tail`` [slots, K - 1, C]).  step = softplus(dt + dt_bias).
    Returns ``coef`` float32 [3, T, heads state] (decay = exp(-exp(a_log) step) in every channel, write = step B,
    read = C, each head with its group's B and C) and x float32 [T, heads value_dim]."""
    _need(proj, "state_space proj", torch.float32, 2)
    T = proj.shape[0]
    inner = heads * value_dim
    C = inner + 2 * groups * state
    if proj.shape[1] != C + inner + heads or heads % groups:
        raise KernelError(f"state_space_prepare: proj has {proj.shape[1]} columns, expected {C + inner + heads}")
    _need(taps, "conv taps", torch.float32, 2)
    _need(bias, "conv bias", torch.float32, 1)
    K = taps.shape[1]
    if taps.shape[0] != C or bias.shape[0] != C or not 1 <= K <= SHORT_CONV_MAX_TAPS:
        raise KernelError("state_space_prepare: taps or bias do not fit the channels")
    if K > 1:
        _need(tail, "conv tail", torch.float32, 3)
        if tuple(tail.shape[1:]) != (K - 1, C):
            raise KernelError("state_space_prepare: the tail does not fit the taps")
    for vec, what in ((dt_bias, "dt_bias"), (a_log, "a_log")):
        _need(vec, what, torch.float32, 1)
        if vec.shape[0] != heads:
            raise KernelError(f"state_space_prepare: {what} has {vec.shape[0]} entries for {heads} heads")
    for t, what in ((tok_req, "tok_req"), (q_offsets, "q_offsets"), (slot_ids, "slot_ids")):
        _need(t, what, torch.int32, 1)
    if tok_req.shape[0] != T:
        raise KernelError("state_space_prepare: the token map does not fit")
    coef = torch.empty((3, T, heads * state), dtype=torch.float32, device=proj.device)
    x = torch.empty((T, inner), dtype=torch.float32, device=proj.device)
    if T:
        _call("lc_state_space_prepare", _ptr(proj), proj.shape[1], T, heads, groups, state, value_dim, _ptr(taps),
              _ptr(bias), K, _ptr(tail if K > 1 else None), _ptr(dt_bias), _ptr(a_log), _ptr(tok_req), _ptr(q_offsets),
              _ptr(slot_ids), _ptr(coef), _ptr(x), _stream())
    return coef, x


def state_space_readout(o: torch.Tensor, x: torch.Tensor, gates: torch.Tensor, z_column: int, skip: torch.Tensor,
                        heads: int, value_dim: int, weight: torch.Tensor, parts: int, eps: float,
                        out_dtype: torch.dtype) -> torch.Tensor:
    """``(o + skip[head] x) silu(z)`` with z the float32 columns ``z_column`` .. + n of ``gates``, the row divided by
    its root mean square in ``parts`` equal parts (eps inside the root), times ``weight`` [n].  -> [T, n]."""
    _need(o, "state_space_readout o", torch.float32, 2)
    _need(x, "state_space_readout x", torch.float32, 2)
    _need(gates, "state_space_readout gates", torch.float32, 2)
    _need(skip, "state_space_readout skip", torch.float32, 1)
    _need(weight, "state_space_readout weight", torch.float32, 1)
    T, n = o.shape
    if n != heads * value_dim or tuple(x.shape) != (T, n) or gates.shape[0] != T or z_column < 0 \
            or z_column + n > gates.shape[1] or skip.shape[0] != heads or weight.shape[0] != n or parts < 1 or n % parts:
        raise KernelError("state_space_readout: the operands do not fit the heads")
    out = torch.empty((T, n), dtype=out_dtype, device=o.device)
    if T:
        _call("lc_state_space_readout", _ptr(o), _ptr(x), _ptr(gates), gates.shape[1], int(z_column), _ptr(skip), heads,
              value_dim, _ptr(weight), int(parts), float(eps), T, _ptr(out), _dt(out), _stream())
    return out


def scaled_sum(a, a_scale: float, b, b_scale: float) -> torch.Tensor:
    """``a_scale a + b_scale b`` as float32 (two branches that a layer adds to its stream as one)."""
    a, b = value(a), value(b)
    _need(a, "scaled_sum a", None, 2)
    _need(b, "scaled_sum b", None, 2)
    if a.shape != b.shape:
        raise KernelError(f"scaled_sum: {tuple(a.shape)} and {tuple(b.shape)} differ")
    out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    if out.numel():
        _call("lc_scaled_sum", _ptr(a), _dt(a), float(a_scale), _ptr(b), _dt(b), float(b_scale), _ptr(out),
              out.numel(), _stream())
    return out
