"""Checked Python entry points of the HIP kernels.

Every function here validates shapes, dtypes, devices and strides on the host before it
launches anything: a kernel is never handed operands that its indexing does not expect.
There is no other implementation behind these functions: without a GPU, or when the
kernels cannot be compiled, they raise.  Kernels run on torch's current stream, so a
step can be captured into a HIP graph.
"""
from __future__ import annotations

import os
from ctypes import c_float, c_int, c_longlong, c_void_p
from dataclasses import dataclass
from typing import Optional

import torch

from .csrc import build as _build

PAGE = _build.header_constant("BN_PAGE")                         # tokens per cache page: defined once, in csrc/common.h
F32_FOLD_KEYS = _build.header_constant("BN_F32_FOLD_KEYS")       # a float32 cache's keys are summed in runs of this many
SPLIT_MIN_PAGES = _build.header_constant("BN_SPLIT_MIN_PAGES")   # shortest run of pages that decode attention splits off
_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "elementwise": {
        "bn_embed_gather": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p],
        "bn_softcap": [c_void_p, c_longlong, c_float, c_void_p],
        "bn_gather_rows": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "bn_add_rmsnorm": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_residual_add": [c_int, c_void_p, c_void_p, c_longlong, c_void_p],
        "bn_add_rmsnorm_parts": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_float, c_void_p],
        "bn_residual_add_parts": [c_void_p, c_void_p, c_int, c_longlong, c_void_p],
        "bn_add_rmsnorm_parts_pieces": [c_int],
        "bn_add_rmsnorm_parts_wide": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_float,
                                      c_void_p],
        "bn_swiglu": [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "bn_sum_deferred": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
        "bn_swiglu_scaled": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_bias_add": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    },
    "rope_kv": {
        "bn_v_transposed_write": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                  c_int, c_void_p],
        "bn_rope_kv_write": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                             c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "bn_rope_kv_write_tiles": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                   c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p],
    },
    "attn_rows": {
        "bn_attn_rows_key_tile": [c_int, c_int],
        "bn_attn_rows": [c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                         c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                         c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p],
    },
    "attn_mfma": {
        "bn_attn_mfma_supports": [c_int],
        "bn_attn_mfma_prompt_tokens": [c_int, c_int],
        "bn_attn_mfma_scaled": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_attn_mfma": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                         c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p,
                         c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p],
    },
    "gemm_tiled": {
        "bn_gemm_tiled": [c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                          c_void_p],
    },
    "gemm_mfma": {
        "bn_gemm_mfma_supports": [c_int, c_int, c_int, c_int, c_int],
        "bn_gemm_mfma": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_int, c_void_p],
    },
    "skinny_gemm": {
        "bn_skinny_gemm_supports": [c_int, c_int, c_int, c_int, c_int],
        "bn_skinny_gemm": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_int, c_int, c_void_p],
        "bn_skinny_gemm_fused_tile_cols": [c_int],
        "bn_skinny_gemm_fused_tiles": [c_int, c_int],
        "bn_skinny_gemm_fused": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_void_p, c_int, c_int, c_float, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                 c_int, c_void_p],
    },
    "splitk_gemm": {
        "bn_splitk_gemm_supports": [c_int, c_int, c_int, c_int, c_int, c_int],
        "bn_splitk_gemm_splits": [c_int, c_int, c_int],
        "bn_splitk_gemm": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "bn_splitk_gemm_swiglu": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                  c_int, c_float, c_int, c_void_p],
    },
    "sampling": {
        "bn_argmax": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
        "bn_repeat_penalty": [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p],
        "bn_sample": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p],
        "bn_sample_wide": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p],
    },
}
_fns = {}


def _fn(lib: str, name: str):
    f = _fns.get(name)
    if f is None:
        handle = _build.load(lib)
        f = getattr(handle, name)
        f.argtypes = _SIGNATURES[lib][name]
        f.restype = c_int
        _fns[name] = f
    return f


_gpu_seen = False


def require_gpu() -> None:
    global _gpu_seen
    if _gpu_seen:                      # asked before every launch: a GPU that was there stays
        return
    if not torch.cuda.is_available():
        raise KernelError("no GPU: the kernels of this library are HIP code for gfx950 and there is "
                          "no CPU implementation behind them")
    _gpu_seen = True


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (it changes under a graph capture, so it is asked for at every launch; the
    raw query costs a fraction of building a torch.cuda.Stream object)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(rc: int, what: str) -> None:
    if rc == 0:
        return
    if rc == -1:
        raise KernelError(f"{what}: the kernel refuses these sizes or this alignment")
    if rc == -2:
        raise KernelError(f"{what}: unsupported dtype")
    raise KernelError(f"{what}: HIP error {rc}")


def _dev(t: torch.Tensor, name: str, dtype=None, dims=None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a GPU tensor")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if dims is not None and t.dim() != dims:
        raise KernelError(f"{name}: expected {dims} dimensions, got shape {tuple(t.shape)}")


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{name}: expected a 2-D tensor with contiguous rows, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _code(dtype) -> int:
    if dtype not in _DT:
        raise KernelError(f"unsupported dtype {dtype}")
    return _DT[dtype]


# The gate's activation of a gated feed-forward, out = act(gate) * up (BN_ACT_* of csrc/common.h): every kernel that
# ends in a gated unit takes the kind as an argument.
ACTIVATIONS = {"silu": _build.header_constant("BN_ACT_SILU"), "gelu_tanh": _build.header_constant("BN_ACT_GELU_TANH"),
               "relu2": _build.header_constant("BN_ACT_RELU2")}


def _act(name: str) -> int:
    if name not in ACTIVATIONS:
        raise KernelError(f"unknown gate activation {name!r}; the kernels take {sorted(ACTIVATIONS)}")
    return ACTIVATIONS[name]


# --------------------------------------------------------------------------------------
# row-wise kernels
# --------------------------------------------------------------------------------------

def embed_gather(table: torch.Tensor, tokens: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 rows of the embedding table for int32 token ids, times `scale` (an architecture's embedding
    multiplier; 1 changes no bit)."""
    require_gpu()
    _dev(table, "table", dims=2)
    _dev(tokens, "tokens", torch.int32, 1)
    if not table.is_contiguous() or not tokens.is_contiguous():
        raise KernelError("embed_gather: table and tokens must be contiguous")
    n, dim = tokens.numel(), table.shape[1]
    x = torch.empty((n, dim), dtype=torch.float32, device=table.device)
    _check(_fn("elementwise", "bn_embed_gather")(_code(table.dtype), x.data_ptr(), table.data_ptr(),
                                                 tokens.data_ptr(), n, dim, table.shape[0], float(scale), _stream()),
           "embed_gather")
    return x


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out_dtype) -> torch.Tensor:
    """The rows `rows` (int32) of the float32 stream x [T, D], in out_dtype: what an output matrix reads when the
    architecture puts no norm in front of it."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(rows, "rows", torch.int32, 1)
    if not x.is_contiguous() or not rows.is_contiguous():
        raise KernelError("gather_rows: x and rows must be contiguous")
    out = torch.empty((rows.numel(), x.shape[1]), dtype=out_dtype, device=x.device)
    if rows.numel():
        _check(_fn("elementwise", "bn_gather_rows")(_code(out_dtype), out.data_ptr(), x.data_ptr(), rows.data_ptr(), rows.numel(),
                                                    x.shape[1], _stream()), "gather_rows")
    return out


def softcap_(logits: torch.Tensor, cap: float) -> None:
    """In place: cap * tanh(logits / cap), float32 (an architecture's bound on its logits; cap > 0)."""
    require_gpu()
    _dev(logits, "logits", torch.float32)
    if not logits.is_contiguous() or not cap > 0:
        raise KernelError("softcap: contiguous float32 logits and a positive cap")
    if logits.numel():
        _check(_fn("elementwise", "bn_softcap")(logits.data_ptr(), logits.numel(), float(cap), _stream()), "softcap")


def add_rmsnorm(x: torch.Tensor, delta, weight: torch.Tensor, eps: float, out_dtype,
                rows=None) -> torch.Tensor:
    """x (float32, [T, D]) += delta (if given), and the RMS-normed rows in out_dtype.
    With `rows` (int32 indices) only those rows are normed and x is left as it is."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(weight, "weight", torch.float32, 1)
    T, D = x.shape
    if not x.is_contiguous() or weight.numel() != D or not weight.is_contiguous():
        raise KernelError(f"add_rmsnorm: x {tuple(x.shape)} must be contiguous and weight have {D} elements")
    parts = delta if isinstance(delta, PartialSums) else None
    if parts is not None:
        if parts.shape != x.shape:
            raise KernelError(f"add_rmsnorm: partial sums {tuple(parts.shape)} do not match x {tuple(x.shape)}")
    elif delta is not None:
        _dev(delta, "delta", out_dtype, 2)
        if delta.shape != x.shape or not delta.is_contiguous():
            raise KernelError(f"add_rmsnorm: delta {tuple(delta.shape)} does not match x {tuple(x.shape)}")
    n = T
    if rows is not None:
        _dev(rows, "rows", torch.int32, 1)
        if not rows.is_contiguous():
            raise KernelError("add_rmsnorm: rows must be contiguous")
        n = rows.numel()
    out = torch.empty((n, D), dtype=out_dtype, device=x.device)
    if n == 0:
        return out
    if parts is not None and rows is None and D % 4 == 0 and parts.slabs.shape[0] > 2 and T <= 65535:
        # many slabs: the sum over the whole chip first, then the norm (one workgroup a row would pull all of its slabs alone)
        ssq = torch.empty((T, _fn("elementwise", "bn_add_rmsnorm_parts_pieces")(D)), dtype=torch.float32, device=x.device)
        _check(_fn("elementwise", "bn_add_rmsnorm_parts_wide")(_code(out_dtype), x.data_ptr(), parts.slabs.data_ptr(),
                                                               parts.slabs.shape[0], T, weight.data_ptr(), out.data_ptr(),
                                                               ssq.data_ptr(), D, float(eps), _stream()), "add_rmsnorm")
        return out
    if parts is not None:
        _check(_fn("elementwise", "bn_add_rmsnorm_parts")(_code(out_dtype), x.data_ptr(), parts.slabs.data_ptr(),
                                                          parts.slabs.shape[0], T, weight.data_ptr(), out.data_ptr(),
                                                          rows.data_ptr() if rows is not None else None,
                                                          n, D, float(eps), _stream()), "add_rmsnorm")
        return out
    _check(_fn("elementwise", "bn_add_rmsnorm")(_code(out_dtype), x.data_ptr(),
                                                delta.data_ptr() if delta is not None else None,
                                                weight.data_ptr(), out.data_ptr(),
                                                rows.data_ptr() if rows is not None else None,
                                                n, D, float(eps), _stream()), "add_rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta) -> None:
    """x (float32) += delta (a tensor of x's shape, or PartialSums)."""
    require_gpu()
    _dev(x, "x", torch.float32)
    if isinstance(delta, PartialSums):
        if tuple(delta.shape) != tuple(x.shape) or not x.is_contiguous():
            raise KernelError("residual_add: partial sums do not match x, or x is not contiguous")
        _check(_fn("elementwise", "bn_residual_add_parts")(x.data_ptr(), delta.slabs.data_ptr(), delta.slabs.shape[0],
                                                           x.numel(), _stream()), "residual_add")
        return
    _dev(delta, "delta")
    if x.shape != delta.shape or not x.is_contiguous() or not delta.is_contiguous():
        raise KernelError("residual_add: shapes differ or tensors are not contiguous")
    _check(_fn("elementwise", "bn_residual_add")(_code(delta.dtype), x.data_ptr(), delta.data_ptr(),
                                                 x.numel(), _stream()), "residual_add")


def swiglu(gu: torch.Tensor, interleaved: bool = False, activation: str = "silu") -> torch.Tensor:
    """[T, 2F] (gate | up) -> act(gate) * up, [T, F].  interleaved: gate and up columns
    alternate in blocks of 8 (see interleave_gate_up).  activation: one of ACTIVATIONS."""
    require_gpu()
    _dev(gu, "gu", dims=2)
    if not gu.is_contiguous() or gu.shape[1] % 2:
        raise KernelError(f"swiglu: expected a contiguous [T, 2F] tensor, got {tuple(gu.shape)}")
    T, F = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((T, F), dtype=gu.dtype, device=gu.device)
    if interleaved and F % 8:
        raise KernelError("swiglu: the interleaved layout needs F to be a multiple of 8")
    _check(_fn("elementwise", "bn_swiglu")(_code(gu.dtype), out.data_ptr(), gu.data_ptr(), T, F, int(interleaved),
                                           _act(activation), _stream()), "swiglu")
    return out


def bias_add(y: torch.Tensor, bias: torch.Tensor) -> None:
    require_gpu()
    _dev(y, "y", dims=2)
    _dev(bias, "bias", torch.float32, 1)
    if not y.is_contiguous() or bias.numel() != y.shape[1] or not bias.is_contiguous():
        raise KernelError("bias_add: y must be contiguous [T, N] and bias have N elements")
    _check(_fn("elementwise", "bn_bias_add")(_code(y.dtype), y.data_ptr(), bias.data_ptr(), y.shape[0],
                                             y.shape[1], _stream()), "bias_add")


# --------------------------------------------------------------------------------------
# matrix products
# --------------------------------------------------------------------------------------

def _tiled(x, w, out_dtype):
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_fn("gemm_tiled", "bn_gemm_tiled")(_code(x.dtype), _code(out_dtype), x.data_ptr(), w.data_ptr(),
                                              y.data_ptr(), M, N, K, _rows(x, "x"), _rows(w, "w"), N,
                                              _stream()), "gemm_tiled")
    return y


def gemm_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype=None, glu8: bool = False, activation: str = "silu",
              width: int = 0) -> torch.Tensor:
    """The library-free bf16 product for many rows: y[M, N] = x[M, K] . w[N, K]^T on the matrix cores,
    or with glu8 act(gate) * up for w = gate and up rows interleaved in blocks of 8 ([2N, K]).
    width: the tile's rows of w (256, 192 or 128); 0 lets the kernel pick by the shape."""
    require_gpu()
    if width not in (0, 256, 192, 128):
        raise KernelError(f"gemm_mfma: the tile width is 256, 192, 128 or 0 (any), not {width}")
    _dev(x, "x", torch.bfloat16, 2)
    _dev(w, "w", torch.bfloat16, 2)
    M, K = x.shape
    rows = w.shape[0]
    if w.shape[1] != K or (glu8 and rows % 16):
        raise KernelError(f"gemm_mfma: x {tuple(x.shape)} and w {tuple(w.shape)} do not agree")
    N = rows // 2 if glu8 else rows
    out_dtype = out_dtype or torch.bfloat16
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return y
    _check(_fn("gemm_mfma", "bn_gemm_mfma")(_code(out_dtype), x.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K,
                                            _rows(x, "x"), _rows(w, "w"), N, int(glu8), _act(activation), int(width),
                                            _stream()),
           "gemm_mfma")
    return y


def gemm_mfma_supported(M: int, N: int, K: int, ldx: int, ldw: int) -> bool:
    """The conditions of bn_gemm_mfma_supports, checked here so that asking does not load (and at
    first use compile) a kernel that a model may never need."""
    return M >= 1 and N >= 1 and K >= 8 and K % 8 == 0 and ldx % 8 == 0 and ldw % 8 == 0 and ldx >= K and ldw >= K


SKINNY_ROWS = 16      # bf16 products with more rows than this go to the library


def skinny_supported(M: int, N: int, K: int, ldx: int, ldw: int) -> bool:
    return bool(_fn("skinny_gemm", "bn_skinny_gemm_supports")(M, N, K, ldx, ldw))


# --------------------------------------------------------------------------------------
# the streamed copy of a weight matrix
# --------------------------------------------------------------------------------------
STREAM_TILE_ROWS = _build.header_constant("BN_STREAM_TILE_ROWS")
STREAM_TILE_COLS = _build.header_constant("BN_STREAM_TILE_COLS")


@dataclass
class StreamedWeight:
    """A bf16 weight matrix [N, K] in the order in which the kernels that read it once per call load it (csrc/common.h):
    tiles of tile_rows (at most 16) rows x 32 columns, each the run of bytes that one load of a wave takes (lane r + 16 g:
    columns 8 g .. 8 g + 7 of row r), [ceil(N / tile_rows), ceil(K / 32), 32 tile_rows], rows past N and columns past K zero.
    A second copy beside the row-major matrix, which the products of many rows (the library's) and everything else keep
    reading: the kernels of up to 128 rows take it through their `streamed` argument and give the same result bit for
    bit, 5 to 15 % sooner.  The kernel of up to 16 rows gives a workgroup one row of tiles, so fewer than 16 rows a tile
    are chosen where that spreads the tiles more evenly over the CUs (stream_tile_rows)."""
    tiles: torch.Tensor
    N: int
    K: int
    tile_rows: int = STREAM_TILE_ROWS

    @property
    def k_tiles(self) -> int:
        return self.tiles.shape[1]

    def nbytes(self) -> int:
        return self.tiles.numel() * self.tiles.element_size()


def stream_tile_rows(N: int) -> int:
    """The rows per tile with which a matrix of N rows is best streamed: the columns that the fused product of up to 16
    rows gives a workgroup over the row-major matrix (16, or fewer when that leaves the busiest CU at least 15 % fewer
    columns: 12 for 6,144 rows on 256 CUs, 10 for 5,120)."""
    return int(_fn("skinny_gemm", "bn_skinny_gemm_fused_tile_cols")(int(N)))


def stream_copy(w: torch.Tensor, tile_rows: Optional[int] = None) -> StreamedWeight:
    """The streamed copy of w [N, K] (bf16, on the device; made there).  tile_rows None: stream_tile_rows(N); a matrix
    with gate and up rows interleaved in blocks of 8 needs 16."""
    require_gpu()
    _dev(w, "w", torch.bfloat16, 2)
    N, K = w.shape
    R, C = (stream_tile_rows(N) if tile_rows is None else int(tile_rows)), STREAM_TILE_COLS
    if not 1 <= R <= STREAM_TILE_ROWS:
        raise KernelError(f"stream_copy: a tile has 1 to {STREAM_TILE_ROWS} rows, not {R}")
    nt, kt = (N + R - 1) // R, (K + C - 1) // C
    if nt * R != N or kt * C != K:
        padded = torch.zeros((nt * R, kt * C), dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        w = padded
    # [nt, r, kt, g, 8] -> [nt, kt, g, r, 8]: lane r + 16 g of tile (nt, kt)
    tiles = w.view(nt, R, kt, C // 8, 8).permute(0, 2, 3, 1, 4).contiguous().view(nt, kt, R * C)
    return StreamedWeight(tiles, N, K, R)


def unstream(sw: StreamedWeight) -> torch.Tensor:
    """The row-major matrix [N, K] that a streamed copy holds."""
    R, C = sw.tile_rows, STREAM_TILE_COLS
    nt, kt = sw.tiles.shape[:2]
    return sw.tiles.view(nt, kt, C // 8, R, 8).permute(0, 3, 1, 2, 4).reshape(nt * R, kt * C)[:sw.N, :sw.K].contiguous()


def _weight_arg(w: torch.Tensor, streamed: Optional[StreamedWeight], what: str, need_rows: int = 0):
    """(pointer, row stride or tiles along K, rows per tile or 0) of the weights that a kernel is to read: the streamed
    copy if one is given (checked against w; need_rows: the only tile height the kernel takes, else w is read), else
    w itself."""
    if streamed is not None and need_rows and getattr(streamed, "tile_rows", 0) != need_rows:
        streamed = None
    if streamed is None:
        return w.data_ptr(), _rows(w, "w"), 0
    t = streamed.tiles
    R = streamed.tile_rows
    if (not isinstance(streamed, StreamedWeight) or (streamed.N, streamed.K) != tuple(w.shape) or t.device != w.device
            or t.dtype != torch.bfloat16 or not t.is_contiguous() or t.dim() != 3 or not 1 <= R <= STREAM_TILE_ROWS
            or tuple(t.shape) != ((streamed.N + R - 1) // R, (streamed.K + STREAM_TILE_COLS - 1) // STREAM_TILE_COLS,
                                  R * STREAM_TILE_COLS)):
        raise KernelError(f"{what}: the streamed copy does not belong to w {tuple(w.shape)}")
    return t.data_ptr(), t.shape[1], R


# bf16 products with many rows: the library's matrix product (as the reference hands its batched
# products to a library, src/gpu_cuda.cu:11571) unless this is False or BITNET_NO_LIBRARY is set;
# then this library's own matrix-core kernel (gemm_mfma) does them.
LIBRARY_PRODUCTS = os.environ.get("BITNET_NO_LIBRARY", "") in ("", "0")


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype=None, *, allow_library: Optional[bool] = None,
           streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """y[M, N] = x[M, K] . w[N, K]^T.  streamed: w's streamed copy, which the kernel of up to 16 rows reads instead.

    float32: the tiled kernel (plain fmaf, a fixed order of summation).
    bf16: up to 16 rows (one MFMA tile of activations) the matrix-core kernel that streams
    the weights once; above that the library's matrix product, which from 32 rows on is about
    twice as fast as the streaming kernel, with a bf16 or a float32 result (logits).  Without the
    library (allow_library False; None follows LIBRARY_PRODUCTS) the streaming kernel takes up to 64
    rows and the tiled matrix-core kernel (gemm_mfma) everything above; shapes that none of them
    takes (rows that are not 16-byte aligned) go to the plain tiled kernel."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(w, "w", x.dtype, 2)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"linear: x {tuple(x.shape)} and w {tuple(w.shape)} do not agree")
    out_dtype = out_dtype or x.dtype
    if allow_library is None:
        allow_library = LIBRARY_PRODUCTS
    if M == 0:
        return torch.empty((0, N), dtype=out_dtype, device=x.device)
    ldx, ldw = _rows(x, "x"), _rows(w, "w")
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise KernelError("linear: float32 inputs give float32 outputs")
        return _tiled(x, w, torch.float32)
    if x.dtype != torch.bfloat16:
        raise KernelError(f"linear: unsupported dtype {x.dtype}")
    aligned = (x.data_ptr() % 16 == 0) and (w.data_ptr() % 16 == 0)
    small = M <= SKINNY_ROWS or (M <= 64 and not allow_library)
    if small and aligned and skinny_supported(M, N, K, ldx, ldw):
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        wp, wl, tiled = _weight_arg(w, streamed if M <= SKINNY_ROWS else None, "linear")
        _check(_fn("skinny_gemm", "bn_skinny_gemm")(_code(out_dtype), x.data_ptr(), wp, y.data_ptr(),
                                                    M, N, K, ldx, wl, N, 0, 0, 0, tiled, _stream()), "skinny_gemm")
        return y
    if M > SKINNY_ROWS and allow_library:
        if out_dtype == torch.bfloat16:
            return torch.matmul(x, w.t())
        if out_dtype == torch.float32:
            return torch.mm(x, w.t(), out_dtype=torch.float32)
    if aligned and gemm_mfma_supported(M, N, K, ldx, ldw):
        return gemm_mfma(x, w, out_dtype)
    return _tiled(x, w, out_dtype)


def interleave_gate_up(w_gate: torch.Tensor, w_up: torch.Tensor) -> torch.Tensor:
    """[2F, K] with gate and up rows alternating in blocks of 8 (F a multiple of 8): rows
    16t..16t+7 are gate rows 8t..8t+7, rows 16t+8..16t+15 the up rows of the same columns.  A
    16-row tile of the decode kernel then holds both halves of 8 result columns."""
    F, K = w_gate.shape
    if F % 8 or w_up.shape != w_gate.shape:
        raise KernelError("interleave_gate_up: F must be a multiple of 8 and the shapes equal")
    return torch.stack([w_gate.reshape(F // 8, 8, K), w_up.reshape(F // 8, 8, K)], dim=1).reshape(2 * F, K).contiguous()


# The interleaved gate/up product with its SwiGLU epilogue in the kernel that stages the activations once per 64 or 112
# columns (splitk_gemm.hip).  Without the library it is the kernel of 17 to 128 rows.  With the library it takes the row
# counts at which it was measured faster than what else there is (the fused streaming kernel up to 16 rows, whose every
# workgroup stages all rows for its 16 columns; above that the library's product and the kernel of the gated unit) on
# matrices of at least STAGED_MIN_TILES_PER_CU column tiles per CU (smaller ones leave it too few waves): 13 to 16 rows,
# and up to 64 rows over a streamed copy of the weights (us at 16 / 32 / 64 rows, streamed: 8B 45.6 / 45.7 / 50.9 against
# 47.8 / 55.4 / 54.3; 13B 53.2 / 53.7 / 61.5 against 57.9 / 56.1 / 59.7; 70B 163 / 169 / 190 against 175 / 196 / 216;
# at a hidden size of 3,072 and below the others win by 5 to 15 %).
SWIGLU_STAGED_ROWS = (17, 128)
SWIGLU_STAGED_LIBRARY_ROWS = (13, 16)
SWIGLU_STAGED_STREAMED_ROWS = (13, 64)
STAGED_MIN_TILES_PER_CU = 6


_CUS = None


def _compute_units() -> int:
    global _CUS
    if _CUS is None:
        _CUS = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _CUS


def _staged_swiglu_rows(M: int, allow_library: bool, w_rows: int, streamed) -> bool:
    if not allow_library:
        lo, hi = SWIGLU_STAGED_ROWS
        return lo <= M <= hi
    lo, hi = SWIGLU_STAGED_STREAMED_ROWS if streamed is not None else SWIGLU_STAGED_LIBRARY_ROWS
    return lo <= M <= hi and w_rows // 16 >= STAGED_MIN_TILES_PER_CU * _compute_units()


def _staged_swiglu(x, w_gate_up, pre, activation, streamed=None):
    """The staged kernel's gate/up product with the gated unit (and a deferred norm's factor) in its epilogue; None if
    it does not take the shape."""
    M, K = x.shape
    F = w_gate_up.shape[0] // 2
    ldx = _rows(x, "x")
    wp, wl, tiled = _weight_arg(w_gate_up, streamed, "linear_swiglu", need_rows=STREAM_TILE_ROWS)
    if F % 8 or not _fn("splitk_gemm", "bn_splitk_gemm_supports")(M, 2 * F, K, ldx, wl, tiled):
        return None
    if pre is not None:          # what the kernel's passes over the parts of the sums of squares hold (SG_NORM_*)
        n = pre.slots.shape[1]
        per = min(64, 1 << max(0, n - 1).bit_length())
        if -(-M // (4 * (64 // per))) > 4 or -(-n // per) > 8:
            return None
    y = torch.empty((M, F), dtype=x.dtype, device=x.device)
    _check(_fn("splitk_gemm", "bn_splitk_gemm_swiglu")(
        x.data_ptr(), wp, y.data_ptr(), M, F, K, ldx, wl, F, _act(activation),
        pre.slots.data_ptr() if pre is not None else None, pre.slots.shape[1] if pre is not None else 0,
        pre.stream.shape[1] if pre is not None else 0, float(pre.eps) if pre is not None else 0.0, int(tiled != 0), _stream()),
        "splitk_gemm(glu)")
    return y


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, interleaved: bool = False, *,
                  allow_library: Optional[bool] = None, activation: str = "silu",
                  streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """act(x.Wg^T) * (x.Wu^T) for w_gate_up = [Wg; Wu] ([2F, K]), or the two interleaved in
    blocks of 8 rows (interleave_gate_up); act is silu unless `activation` names another of
    ACTIVATIONS.  The decode-sized bf16 case is one kernel, and so is the interleaved case without
    the library; every other case is the product followed by the gated-unit kernel."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(w_gate_up, "w_gate_up", x.dtype, 2)
    M, K = x.shape
    if w_gate_up.shape[0] % 2 or w_gate_up.shape[1] != K:
        raise KernelError(f"linear_swiglu: x {tuple(x.shape)} and w {tuple(w_gate_up.shape)} do not agree")
    F = w_gate_up.shape[0] // 2
    if interleaved and F % 8:
        raise KernelError("linear_swiglu: the interleaved layout needs F to be a multiple of 8")
    if allow_library is None:
        allow_library = LIBRARY_PRODUCTS
    if M == 0:
        return torch.empty((0, F), dtype=x.dtype, device=x.device)
    ldx, ldw = _rows(x, "x"), _rows(w_gate_up, "w_gate_up")
    aligned = x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0
    if x.dtype == torch.bfloat16 and interleaved and aligned and _staged_swiglu_rows(M, allow_library, 2 * F, streamed):
        y = _staged_swiglu(x, w_gate_up, None, activation, streamed)
        if y is not None:
            return y
    if (x.dtype == torch.bfloat16 and (M <= SKINNY_ROWS or (M <= 64 and not allow_library))
            and aligned and skinny_supported(M, F, K, ldx, ldw)):
        y = torch.empty((M, F), dtype=x.dtype, device=x.device)
        _check(_fn("skinny_gemm", "bn_skinny_gemm")(_code(x.dtype), x.data_ptr(), w_gate_up.data_ptr(),
                                                    y.data_ptr(), M, F, K, ldx, ldw, F, 2 if interleaved else 1, F,
                                                    _act(activation), 0, _stream()), "skinny_gemm(glu)")
        return y
    if (x.dtype == torch.bfloat16 and interleaved and not allow_library and aligned
            and gemm_mfma_supported(M, 2 * F, K, ldx, ldw)):
        return gemm_mfma(x, w_gate_up, x.dtype, glu8=True, activation=activation)
    return swiglu(linear(x, w_gate_up, allow_library=allow_library), interleaved, activation)


# --------------------------------------------------------------------------------------
# decode products with the neighbouring RMSNorm folded in
# --------------------------------------------------------------------------------------
# Set False (or BITNET_NO_FUSED_NORM=1) to keep every norm a kernel of its own.
SPLIT_SUMS = os.environ.get("BITNET_NO_SPLIT_SUMS", "") in ("", "0")
# Where a product that ends a part is left as partial sums (splitk_gemm) instead of going to the library: from 17 to 128
# rows when K is at least twice N, the shape of a feed-forward's last product.  Measured on nine layer shapes (hidden 2,048
# to 8,192) with the kernels of the next norm included: from 64 rows on it is 15 to 45 % faster than the library's product
# (8B: 36 us against 45 at 64 rows, 44 against 80 at 128; 70B: 119 against 148, 141 against 210); below 64 rows the two
# products are equal within a tenth, and the partial sums win by the kernel that they save: one kernel adds them to
# the stream and leaves the next norm to its consumer (sum_deferred), where the library's product needs the add and the
# norm.  Square products (an output projection) as well up to SPLIT_SUM_SQUARE_WIDTH columns: 12 + 5 us against 15 + 5 at
# 64 rows of the 8B shape; at widths of 5,120 and 8,192 whole decode steps were equal within the noise of a run or slower.
SPLIT_SUM_ROWS = (17, 128)
SPLIT_SUM_SQUARE_WIDTH = int(os.environ.get("BITNET_SPLIT_SQUARE_WIDTH", "4096"))


@dataclass
class PartialSums:
    """A product that is still a sum to be formed: `slabs` [S, M, N] float32, the products over S ranges of K
    (splitk_gemm).  add_rmsnorm and residual_add take it in place of a delta and add the slabs in order."""
    slabs: torch.Tensor

    @property
    def shape(self):
        return self.slabs.shape[1:]

    @property
    def device(self):
        return self.slabs.device


def can_split_sums(M: int, N: int, K: int, dtype) -> bool:
    """Whether a product of these sizes whose result goes to the residual stream is done as partial sums."""
    if not (SPLIT_SUMS and dtype == torch.bfloat16 and SPLIT_SUM_ROWS[0] <= M <= SPLIT_SUM_ROWS[1] and K % 8 == 0 and N >= 1):
        return False
    return K >= 2 * N or (K >= N and N <= SPLIT_SUM_SQUARE_WIDTH)


def linear_partial_sums(x: torch.Tensor, w: torch.Tensor, streamed: Optional[StreamedWeight] = None) -> PartialSums:
    """x [M, K] . w[N, K]^T as float32 partial sums over ranges of K (bf16 operands, 1 to 128 rows).  streamed: w's
    streamed copy, read instead of w."""
    require_gpu()
    _dev(x, "x", torch.bfloat16, 2)
    _dev(w, "w", torch.bfloat16, 2)
    ldx = _rows(x, "x")
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"linear_partial_sums: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit")
    wp, wl, tiled = _weight_arg(w, streamed, "linear_partial_sums")
    if not _fn("splitk_gemm", "bn_splitk_gemm_supports")(M, N, K, ldx, wl, tiled) or (x.data_ptr() | wp) % 16:
        raise KernelError(f"linear_partial_sums: the kernel takes 1 to 128 rows, K a multiple of 8 and 16-byte aligned "
                          f"operands, not x {tuple(x.shape)} (row stride {ldx}), w {tuple(w.shape)} (row stride {wl})")
    S = _fn("splitk_gemm", "bn_splitk_gemm_splits")(N, K, tiled)
    slabs = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
    _check(_fn("splitk_gemm", "bn_splitk_gemm")(x.data_ptr(), wp, slabs.data_ptr(), M, N, K, ldx, wl, S, tiled,
                                                _stream()), "splitk_gemm")
    return PartialSums(slabs)


FUSE_NORMS = os.environ.get("BITNET_NO_FUSED_NORM", "") in ("", "0")
FUSED_ROWS = 16           # rows the fused products take (one MFMA tile of activations)
FUSED_SLOTS = 512         # column tiles of 16 whose sums of squares a consumer adds up: streams up to 8,192 wide


@dataclass
class DeferredNorm:
    """An RMSNorm that has not been applied yet.  `scaled` is the bf16 copy of the stream already
    multiplied by the norm's weights, `slots` [M, n] the sums of squares of the stream's rows in
    parts; a product that consumes it (linear_prenorm, linear_swiglu_prenorm) multiplies its
    result's rows by 1/sqrt(mean + eps).  `stream`, `weight`, `eps` are what the plain kernel needs
    when the consumer cannot take it (materialize)."""
    scaled: torch.Tensor
    slots: torch.Tensor
    stream: torch.Tensor
    weight: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.scaled.shape

    @property
    def dtype(self):
        return self.scaled.dtype

    @property
    def device(self):
        return self.scaled.device

    def materialize(self, out_dtype=None, rows=None) -> torch.Tensor:
        return add_rmsnorm(self.stream, None, self.weight, self.eps, out_dtype or self.scaled.dtype, rows)


DEFER_ROWS = (17, 128)    # row counts at which a norm is left to its consumer through sum_deferred (below: the fused products)


def can_sum_deferred(M: int, D: int, dtype) -> bool:
    """Whether the residual stream of M rows of D columns leaves the norm of a consumer that asks for it undone
    (sum_deferred) instead of norming the rows itself."""
    return FUSE_NORMS and dtype == torch.bfloat16 and DEFER_ROWS[0] <= M <= DEFER_ROWS[1] and D % 8 == 0 and D >= 8


def sum_deferred(x: torch.Tensor, delta, weight: torch.Tensor, eps: float) -> DeferredNorm:
    """x (float32 [M, D], in place) += delta (a bf16 or float32 tensor, PartialSums, or None), and what the next norm
    (weights `weight`, `eps`) needs of the new x for a consumer that applies it itself: the bf16 copy times the weights
    and the rows' sums of squares in pieces of 1,024 columns.  One kernel over the whole chip."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(weight, "weight", torch.float32, 1)
    M, D = x.shape
    if not x.is_contiguous() or weight.numel() != D or not weight.is_contiguous() or D % 4 or M < 1 or M > 65535:
        raise KernelError(f"sum_deferred: x {tuple(x.shape)} must be contiguous with a width that is a multiple of 4, "
                          f"weight have {D} elements")
    n_parts, dptr, ddt = 0, None, 0
    if isinstance(delta, PartialSums):
        if tuple(delta.shape) != (M, D) or not delta.slabs.is_contiguous():
            raise KernelError(f"sum_deferred: partial sums {tuple(delta.shape)} do not match x {tuple(x.shape)}")
        n_parts, dptr, ddt = delta.slabs.shape[0], delta.slabs.data_ptr(), _DT[torch.float32]
    elif delta is not None:
        _dev(delta, "delta", dims=2)
        if tuple(delta.shape) != (M, D) or not delta.is_contiguous() or delta.dtype not in _DT:
            raise KernelError(f"sum_deferred: delta {tuple(delta.shape)} ({delta.dtype}) does not match x {tuple(x.shape)}")
        n_parts, dptr, ddt = 1, delta.data_ptr(), _DT[delta.dtype]
    scaled = torch.empty((M, D), dtype=torch.bfloat16, device=x.device)
    slots = torch.empty((M, _fn("elementwise", "bn_add_rmsnorm_parts_pieces")(D)), dtype=torch.float32, device=x.device)
    _check(_fn("elementwise", "bn_sum_deferred")(ddt, x.data_ptr(), dptr, n_parts, M, weight.data_ptr(), scaled.data_ptr(),
                                                 slots.data_ptr(), D, _stream()), "sum_deferred")
    return DeferredNorm(scaled, slots, x, weight, float(eps))


def swiglu_scaled(gu: torch.Tensor, pre: DeferredNorm, activation: str = "silu") -> torch.Tensor:
    """act(s * gate) * (s * up) for gu = [T, 2F] (bf16, gate and up interleaved in blocks of 8) that is the product of a
    deferred norm's copy with the gate and up weights; s the rows' 1/sqrt(mean + eps)."""
    require_gpu()
    _dev(gu, "gu", torch.bfloat16, 2)
    T, F = gu.shape[0], gu.shape[1] // 2
    if not gu.is_contiguous() or gu.shape[1] % 16 or pre.slots.shape[0] != T or not pre.slots.is_contiguous():
        raise KernelError(f"swiglu_scaled: gu {tuple(gu.shape)} / slots {tuple(pre.slots.shape)} do not fit")
    out = torch.empty((T, F), dtype=gu.dtype, device=gu.device)
    if T:
        _check(_fn("elementwise", "bn_swiglu_scaled")(out.data_ptr(), gu.data_ptr(), T, F, _act(activation), pre.slots.data_ptr(),
                                                      pre.slots.shape[1], pre.stream.shape[1], float(pre.eps), _stream()),
               "swiglu_scaled")
    return out


def can_fuse_norm(M: int, N: int, K: int, dtype) -> bool:
    """Whether a product of these sizes can take a norm into its kernel (either side of it)."""
    return (dtype == torch.bfloat16 and 1 <= M <= FUSED_ROWS and K % 8 == 0 and N >= 1
            and torch.cuda.is_available() and skinny_supported(M, N, K, K, K))


def _fused_call(x, w, y, M, N, K, glu8, pre: Optional[DeferredNorm], resid, resid_bf16, next_weight, slots_out,
                activation: str = "silu", streamed: Optional[StreamedWeight] = None):
    wp, wl, tiled = _weight_arg(w, streamed, "fused product", need_rows=STREAM_TILE_ROWS if glu8 else 0)
    _check(_fn("skinny_gemm", "bn_skinny_gemm_fused")(
        x.data_ptr(), wp, y.data_ptr() if y is not None else None, M, N, K, _rows(x, "x"), wl,
        N if y is not None else 0, int(glu8), _act(activation),
        pre.slots.data_ptr() if pre is not None else None, pre.slots.shape[1] if pre is not None else 0,
        pre.stream.shape[1] if pre is not None else 0, float(pre.eps) if pre is not None else 0.0,
        resid.data_ptr() if resid is not None else None, _rows(resid, "resid") if resid is not None else 0,
        resid_bf16.data_ptr() if resid_bf16 is not None else None, N if resid_bf16 is not None else 0,
        next_weight.data_ptr() if next_weight is not None else None,
        slots_out.data_ptr() if slots_out is not None else None, tiled, _stream()), "skinny_gemm(fused)")


def _check_deferred(pre: DeferredNorm, K: int) -> int:
    _dev(pre.scaled, "deferred norm: scaled", torch.bfloat16, 2)
    _dev(pre.slots, "deferred norm: slots", torch.float32, 2)
    M = pre.scaled.shape[0]
    if (pre.scaled.shape[1] != K or pre.stream.shape[1] != K or pre.slots.shape[0] != M
            or not pre.slots.is_contiguous() or pre.slots.shape[1] > FUSED_SLOTS or pre.scaled.data_ptr() % 16):
        raise KernelError(f"deferred norm: copy {tuple(pre.scaled.shape)}, slots {tuple(pre.slots.shape)} do not fit "
                          f"an input width of {K}")
    return M


def linear_prenorm(pre: DeferredNorm, w: torch.Tensor, streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """linear(rmsnorm(stream), w) for a deferred norm, in one kernel (bf16, up to 16 rows).  streamed: w's streamed
    copy, read instead of w."""
    require_gpu()
    _dev(w, "w", torch.bfloat16, 2)
    N, K = w.shape
    M = _check_deferred(pre, K)
    if not can_fuse_norm(M, N, K, torch.bfloat16) or w.data_ptr() % 16:
        raise KernelError(f"linear_prenorm: {M} rows, w {tuple(w.shape)} cannot be fused")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _fused_call(pre.scaled, w, y, M, N, K, False, pre, None, None, None, None, streamed=streamed)
    return y


def linear_swiglu_prenorm(pre: DeferredNorm, w_gate_up: torch.Tensor, activation: str = "silu",
                          streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """linear_swiglu(rmsnorm(stream), w) for gate and up interleaved in blocks of 8, in one kernel.  streamed: w's
    streamed copy, read instead of w."""
    require_gpu()
    _dev(w_gate_up, "w_gate_up", torch.bfloat16, 2)
    F, K = w_gate_up.shape[0] // 2, w_gate_up.shape[1]
    M = _check_deferred(pre, K)
    if (w_gate_up.shape[0] % 16 == 0 and w_gate_up.data_ptr() % 16 == 0
            and _staged_swiglu_rows(M, LIBRARY_PRODUCTS, w_gate_up.shape[0], streamed)):
        y = _staged_swiglu(pre.scaled, w_gate_up, pre, activation, streamed)
        if y is not None:
            return y
    if M > FUSED_ROWS and w_gate_up.shape[0] % 16 == 0 and LIBRARY_PRODUCTS:
        # more rows than the fused kernel takes: the library's product of the copy, and the norm's factor in the
        # kernel of the gated unit, which runs anyway
        return swiglu_scaled(torch.matmul(pre.scaled, w_gate_up.t()), pre, activation)
    if w_gate_up.shape[0] % 16 or not can_fuse_norm(M, F, K, torch.bfloat16) or w_gate_up.data_ptr() % 16:
        raise KernelError(f"linear_swiglu_prenorm: {M} rows, w {tuple(w_gate_up.shape)} cannot be fused")
    y = torch.empty((M, F), dtype=torch.bfloat16, device=w_gate_up.device)
    _fused_call(pre.scaled, w_gate_up, y, M, F, K, True, pre, None, None, None, None, activation, streamed)
    return y


def _fused_tiles(N: int, tile_rows: int = 0) -> int:
    """Column tiles of the fused product kernel for N columns (over a streamed copy with tile_rows rows a tile if that
    is not 0): one partial sum of squares per row and tile."""
    return int(_fn("skinny_gemm", "bn_skinny_gemm_fused_tiles")(int(N), int(tile_rows)))


def can_defer_norm(M: int, N: int, K: int, dtype) -> bool:
    """Whether linear_into_stream takes a product of these sizes (N is the stream's width)."""
    return FUSE_NORMS and can_fuse_norm(M, N, K, dtype) and _fused_tiles(N) <= FUSED_SLOTS


def linear_into_stream(x: torch.Tensor, w: torch.Tensor, stream: torch.Tensor, weight: torch.Tensor,
                       eps: float, streamed: Optional[StreamedWeight] = None) -> DeferredNorm:
    """stream += linear(x, w) (float32 stream [M, N], in place), and what the next norm (weights
    `weight`, `eps`) needs: the bf16 copy of the new stream times the weights and the rows' sums of
    squares in parts.  Returns that norm, deferred."""
    require_gpu()
    _dev(x, "x", torch.bfloat16, 2)
    _dev(w, "w", torch.bfloat16, 2)
    _dev(stream, "stream", torch.float32, 2)
    _dev(weight, "weight", torch.float32, 1)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(stream.shape) != (M, N) or weight.numel() != N or not weight.is_contiguous():
        raise KernelError(f"linear_into_stream: x {tuple(x.shape)}, w {tuple(w.shape)}, stream {tuple(stream.shape)}, "
                          f"weight {tuple(weight.shape)} do not agree")
    if not can_defer_norm(M, N, K, torch.bfloat16) or x.data_ptr() % 16 or w.data_ptr() % 16:
        raise KernelError(f"linear_into_stream: {M} rows, w {tuple(w.shape)} cannot be fused")
    if streamed is not None and _fused_tiles(N, streamed.tile_rows) > FUSED_SLOTS:
        streamed = None                       # more rows of tiles than a consumer adds up slots
    scaled = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    slots = torch.empty((M, _fused_tiles(N, streamed.tile_rows if streamed is not None else 0)), dtype=torch.float32,
                        device=x.device)
    _fused_call(x, w, None, M, N, K, False, None, stream, scaled, weight, slots, streamed=streamed)
    return DeferredNorm(scaled, slots, stream, weight, float(eps))


# --------------------------------------------------------------------------------------
# position encoding + cache write, attention
# --------------------------------------------------------------------------------------

KV_BLOCK = _build.header_constant("BN_KV_BLOCK")       # positions in a block of a blocked page


def kernel_v_layout(dtype, head_dim: int = 0) -> str:
    """The page layout (KVNeed.v_layout) that the attention kernels of this library read fastest at a cache type and
    head size: "blocked" for bf16 at the head sizes of the matrix-core kernels (keys and values of a page in those
    kernels' own order, blocked_page_index), else bf16 values transposed inside a page ([pages, Hkv, hs, PAGE]) and
    float32 values like the keys ([pages, Hkv, PAGE, hs]).  Without a head size: "transposed" or "rows".  The vector
    kernel and the cache write take rows and transposed values at either type; the matrix-core kernels take blocked
    pages alone."""
    if dtype != torch.bfloat16:
        return "rows"
    return "blocked" if head_dim and mfma_attention(dtype, head_dim) else "transposed"


def _page_layout(dtype, hs: int, v_transposed, blocked) -> str:
    """The layout that a caller names with v_transposed (None, False, True) and blocked (None, False, True); neither:
    kernel_v_layout."""
    if blocked:
        if v_transposed is False or dtype != torch.bfloat16 or hs % 32:
            raise KernelError(f"blocked pages are bf16 pages of head sizes that are multiples of 32 (got {dtype}, {hs})")
        return "blocked"
    if v_transposed is None:
        return kernel_v_layout(dtype, hs if blocked is None else 0)
    return "transposed" if v_transposed else "rows"


_LAYOUT_CODES = {"rows": 0, "transposed": 1, "blocked": 2}       # BN_KV_* of csrc/rope_kv.hip; + 4: values by page tiles


def _check_pages(k_pages, v_pages, Hkv, hs, dtype, v_transposed=None, blocked=None) -> str:
    """Checks both page tensors against the layout that the caller names (_page_layout) and returns it.  The kernels here
    want values as wide as keys.  Blocked pages have the shapes of pages with transposed values."""
    layout = _page_layout(dtype, hs, v_transposed, blocked)
    v_shape = (Hkv, PAGE, hs) if layout == "rows" else (Hkv, hs, PAGE)
    for t, nm, shape in ((k_pages, "k_pages", (Hkv, PAGE, hs)), (v_pages, "v_pages", v_shape)):
        _dev(t, nm, dtype, 4)
        if tuple(t.shape[1:]) != shape or not t.is_contiguous():
            raise KernelError(f"{nm}: expected contiguous [pages, {', '.join(map(str, shape))}], got {tuple(t.shape)}")
    if k_pages.shape[0] != v_pages.shape[0]:
        raise KernelError("k_pages and v_pages differ in their number of pages")
    return layout


def blocked_page_index(hs: int):
    """Where the elements of a (page, kv head) lie in a blocked page (csrc/common.h), as two int64 tensors: k_index[p, d]
    = the place of dimension d of the key at position p, v_index[d, p] = the place of dimension d of the value at
    position p, both counted in elements from the beginning of the (page, kv head).  Position p = 32 b + r: the keys'
    operand tiles hold the block's positions 8 (i / 4) + i % 4 (tile 0) and 4 further (tile 1) in tile row i, a lane
    group g the dimensions 32 c + 8 g .. + 7; the values' tiles hold dimension 16 t + i in row i, a lane group the
    positions 8 g .. 8 g + 7 of the block."""
    if hs % 32:
        raise KernelError(f"blocked pages need a head size that is a multiple of 32, got {hs}")
    p = torch.arange(PAGE).view(PAGE, 1)
    d = torch.arange(hs).view(1, hs)
    b, r = p // 32, p % 32
    tile, i = (r // 4) % 2, (r // 8) * 4 + r % 4
    k_index = 32 * hs * b + 8 * (64 * (2 * (d // 32) + tile) + 16 * ((d // 8) % 4) + i) + d % 8
    v_index = 32 * hs * b + 8 * (64 * (d // 16) + 16 * ((p // 8) % 4) + d % 16) + p % 8
    return k_index.contiguous(), v_index.t().contiguous()


def to_blocked_pages(k_rows: torch.Tensor, v_transposed: torch.Tensor):
    """Pages [n, Hkv, PAGE, hs] of keys and [n, Hkv, hs, PAGE] of transposed values as blocked pages (the same shapes)."""
    hs = k_rows.shape[-1]
    ki, vi = (t.to(k_rows.device).reshape(-1) for t in blocked_page_index(hs))
    k = torch.empty_like(k_rows).view(*k_rows.shape[:2], -1)
    v = torch.empty_like(v_transposed).view(*v_transposed.shape[:2], -1)
    k[..., ki] = k_rows.reshape(*k_rows.shape[:2], -1)
    v[..., vi] = v_transposed.reshape(*v_transposed.shape[:2], -1)
    return k.view(k_rows.shape), v.view(v_transposed.shape)


def from_blocked_pages(k_blocked: torch.Tensor, v_blocked: torch.Tensor):
    """The inverse of to_blocked_pages: keys as rows, values transposed."""
    hs = k_blocked.shape[-1]
    ki, vi = (t.to(k_blocked.device).reshape(-1) for t in blocked_page_index(hs))
    k = k_blocked.reshape(*k_blocked.shape[:2], -1)[..., ki].view(k_blocked.shape)
    v = v_blocked.reshape(*v_blocked.shape[:2], -1)[..., vi].view(v_blocked.shape)
    return k.contiguous(), v.contiguous()


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, H: int, Hkv: int, hs: int, *,
                  inv_freq=None, rope_dims: int = 0, seq_index=None, block_table=None,
                  k_pages=None, v_pages=None, page_tiles=None, v_transposed=None, blocked=None) -> None:
    """Rotate the Q heads of qkv ([T, (H+2Hkv)*hs]) in place, rotate the K heads and store
    them and the V heads at each token's position of its sequence's pages.
    k_pages None: rotate Q only.  rope_dims 0: no rotation.  positions < 0: padding rows.
    page_tiles (optional, [n, 4] int32 = sequence, first row, rows, position of the first; each
    tile inside one page, all rows covered): transposed or blocked V pages are then filled by a kernel
    that stores runs of positions instead of single elements.
    v_transposed, blocked: the layout of the pages (neither: kernel_v_layout of qkv's type and hs)."""
    require_gpu()
    _dev(qkv, "qkv", dims=2)
    _dev(positions, "positions", torch.int32, 1)
    T = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    if qkv.shape[1] < (H + 2 * Hkv) * hs or positions.numel() != T or not positions.is_contiguous():
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} / positions {tuple(positions.shape)} do not "
                          f"fit H={H} Hkv={Hkv} hs={hs}")
    if rope_dims:
        _dev(inv_freq, "inv_freq", torch.float32, 1)
        if rope_dims % 2 or rope_dims > hs or inv_freq.numel() != rope_dims // 2 or not inv_freq.is_contiguous():
            raise KernelError(f"rope_kv_write: rope_dims {rope_dims} does not fit hs={hs} / inv_freq "
                              f"{tuple(inv_freq.shape)}")
    bt_stride = 0
    layout = "rows"
    if k_pages is not None:
        layout = _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, v_transposed, blocked)
        _dev(seq_index, "seq_index", torch.int32, 1)
        _dev(block_table, "block_table", torch.int32, 2)
        if seq_index.numel() != T or not seq_index.is_contiguous() or not block_table.is_contiguous():
            raise KernelError("rope_kv_write: seq_index must have one entry per token; tables contiguous")
        bt_stride = block_table.shape[1]
    if T == 0:
        return
    tiled_v = (page_tiles is not None and k_pages is not None and layout != "rows" and qkv.dtype == torch.bfloat16     # a bf16 kernel
               and hs % 8 == 0 and stride % 8 == 0
               and qkv.data_ptr() % 16 == 0 and hs * (PAGE + 2) * 2 <= 65536 and Hkv <= 65535)
    if tiled_v:
        _dev(page_tiles, "page_tiles", torch.int32, 2)
        if page_tiles.shape[1] != 4 or not page_tiles.is_contiguous() or page_tiles.shape[0] == 0:
            raise KernelError("rope_kv_write: page_tiles must be a contiguous [n, 4] tensor")
    if (tiled_v and rope_dims > 0 and rope_dims % 16 == 0
            and (k_pages.data_ptr() | v_pages.data_ptr()) % 16 == 0):
        # the rows that the 16-byte kernel takes: rotation, keys and the values' tiles in one launch
        _check(_fn("rope_kv", "bn_rope_kv_write_tiles")(
            qkv.data_ptr(), stride, positions.data_ptr(), seq_index.data_ptr(), block_table.data_ptr(), bt_stride,
            k_pages.data_ptr(), v_pages.data_ptr(), inv_freq.data_ptr(), rope_dims, T, H, Hkv, hs, _LAYOUT_CODES[layout],
            page_tiles.data_ptr(), page_tiles.shape[0], _stream()), "rope_kv_write(tiles)")
        return
    _check(_fn("rope_kv", "bn_rope_kv_write")(
        _code(qkv.dtype), qkv.data_ptr(), stride, positions.data_ptr(),
        seq_index.data_ptr() if k_pages is not None else None,
        block_table.data_ptr() if k_pages is not None else None, bt_stride,
        k_pages.data_ptr() if k_pages is not None else None,
        v_pages.data_ptr() if k_pages is not None else None,
        inv_freq.data_ptr() if rope_dims else None, rope_dims, T, H, Hkv, hs,
        _LAYOUT_CODES[layout] + (4 if tiled_v else 0), _stream()), "rope_kv_write")
    if tiled_v:
        _check(_fn("rope_kv", "bn_v_transposed_write")(
            qkv.data_ptr(), stride, page_tiles.data_ptr(), page_tiles.shape[0], block_table.data_ptr(), bt_stride,
            v_pages.data_ptr(), H, Hkv, hs, int(layout == "blocked"), _stream()), "v_transposed_write")


MAX_HEAD_DIM = _build.header_constant("BN_MAX_HEAD_DIM")    # the attention kernels take every even head size up to this


def _pow2_at_least(n: int) -> int:
    p = 1
    while p < n:
        p *= 2
    return p


MFMA_HEAD_DIMS = (_build.header_constant("BN_MFMA_HEAD_DIM_SMALL"), _build.header_constant("BN_MFMA_HEAD_DIM_LARGE"))


def mfma_attention(dtype, hs: int) -> bool:
    """Whether the matrix-core attention kernels take this cache type and head size (bn_attn_mfma_supports, answered
    from the header so that asking loads no kernel)."""
    return dtype == torch.bfloat16 and int(hs) in MFMA_HEAD_DIMS


def attention_row_shape(H: int, Hkv: int, decode: bool, dtype=None, hs: int = 0):
    """(RT, GT, QT): what one workgroup covers: QT query tokens x GT heads of one kv group
    (RT = QT * GT rows for the vector kernel)."""
    G = H // Hkv
    GT = min(_pow2_at_least(G), 16)
    if decode:
        return GT, GT, 1
    if dtype is not None and mfma_attention(dtype, hs):
        qt = _fn("attn_mfma", "bn_attn_mfma_prompt_tokens")(int(hs), GT)
        return qt * GT, GT, qt
    return 16, GT, 16 // GT


def pair_tiles(rows: list) -> list:
    """The order in which the prompt form of the matrix-core attention wants its tiles (sequence, first row, rows,
    position of the first): it gives a workgroup two consecutive tiles of the list when there are more tiles than
    CUs, and a causal tile's work grows with its position.  So a sequence's tile with the most keys is followed by
    its tile with the fewest, the second by the last but one, and so on (equal work per workgroup); sequences follow
    each other, longest first, so that workgroups that run together walk the same keys; the middle tiles of
    sequences with an odd number of them are paired with each other at the end.  The result of the attention does
    not depend on the order."""
    by_seq = {}
    for r in rows:
        by_seq.setdefault(r[0], []).append(r)
    keys = lambda r: r[3] + r[2]
    out, single = [], []
    for seq in sorted(by_seq, key=lambda q: -max(keys(r) for r in by_seq[q])):
        ts = sorted(by_seq[seq], key=lambda r: -keys(r))
        n = len(ts)
        for p in range(n // 2):
            out += [ts[p], ts[n - 1 - p]]
        if n % 2:
            single.append(ts[n // 2])
    single.sort(key=lambda r: -keys(r))
    n = len(single)
    for p in range(n // 2):
        out += [single[p], single[n - 1 - p]]
    if n % 2:
        out.append(single[n // 2])
    return out


# Workgroups that a decode attention launch aims for when it cuts the keys: one for every CU of this chip.  (Measured at
# 8,000 and 32,000 cached tokens a sequence and 1 to 8 sequences of the 8B shape: about 256 workgroups are fastest
# whatever the batch, 29 us against 35 for 504 at one sequence of 32,000 tokens, 183 against 188 at eight.)
DECODE_TARGET_WGS = int(os.environ.get("BITNET_DECODE_WGS", "256"))


def decode_splits(n_seqs: int, H: int, Hkv: int, max_len: int, dtype=None):
    """(n_splits, chunk): how the keys of a decode step are cut so that the launch fills the
    chip.  A function of the batch's shape and of max_len alone.  A float32 cache is cut in runs of F32_FOLD_KEYS
    positions whatever the batch: both forms of the float32 kernel sum a query's keys run by run and fold the runs in
    order, so a decode step may give every run a workgroup and float32 logits stay equal bit for bit under every cut."""
    if dtype == torch.float32:
        return max(1, (max_len + F32_FOLD_KEYS - 1) // F32_FOLD_KEYS), F32_FOLD_KEYS
    RT, GT, _ = attention_row_shape(H, Hkv, True)
    G = H // Hkv
    wgs = max(1, n_seqs * Hkv * ((G + GT - 1) // GT))
    pages = max(1, (max_len + PAGE - 1) // PAGE)
    # about DECODE_TARGET_WGS workgroups, but no split shorter than SPLIT_MIN_PAGES pages: below that the merging costs
    # more than the parallelism gains (measured at batch 1, 8 and 64 of the 8B shape)
    want = max(1, min(pages // SPLIT_MIN_PAGES, 64, (DECODE_TARGET_WGS + wgs - 1) // wgs))
    chunk = ((pages + want - 1) // want) * PAGE
    n_splits = (pages * PAGE + chunk - 1) // chunk
    return n_splits, chunk


def split_chunk(max_len: int, n_splits: int) -> int:
    """Keys per split when a launch of n_splits splits meets sequences of up to max_len keys (bn_split_chunk of
    csrc/common.h): what the kernels compute themselves when the length comes in device memory."""
    pages = max(1, (max_len + PAGE - 1) // PAGE)
    return max(SPLIT_MIN_PAGES, (pages + n_splits - 1) // n_splits) * PAGE


def can_fuse_decode(dtype, H: int, Hkv: int, hs: int) -> bool:
    """Whether decode attention can rotate Q and K and store the new K, V itself."""
    return mfma_attention(dtype, hs) and H // Hkv <= 16


def attention(qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
              block_table: torch.Tensor, H: int, Hkv: int, hs: int, scale: float, *, window: int = 0,
              tiles=None, qt: int = 0, seq_lens=None, n_splits: int = 1, chunk: int = 0,
              force_vector: bool = False, fused_rotate=None, fused_write: bool = False, by_length=None,
              max_len_dev=None, v_transposed=None, row_scale: Optional["DeferredNorm"] = None, blocked=None) -> None:
    """Causal attention of the (rotated) Q heads in qkv over the paged cache.

    Prompt form: `tiles` [n, 4] int32 = (sequence, first token row, tokens (<= qt), position of
    the first), qt = the QT of attention_row_shape(H, Hkv, False, dtype, hs).
    Decode form: tiles None, seq_lens [B] int32 (keys in the cache, the new one included; 0 for a
    padding row); row b of qkv is sequence b's token; n_splits/chunk from decode_splits.  Every entry of
    block_table names a page of the pool, also those behind a sequence's last page (0 will do): the
    matrix-core kernel asks for a workgroup's first block of keys before it knows the sequence's length.
    bf16 with head size 64 or 128 over blocked pages runs on the matrix cores, everything else on the vector ALUs,
    which read rows and transposed values (force_vector: say so where the pages are not blocked and the head size
    would be the other kernel's; its qt then is that of attention_row_shape without dtype).
    Decode on the matrix cores can do the work of rope_kv_write itself (can_fuse_decode):
    fused_rotate = inv_freq [hs/2]: qkv arrives unrotated, Q and the new K are rotated inside;
    fused_write: the new K, V of every row (from qkv) are stored at position seq_lens - 1 first.
    by_length (decode form, optional): [B] int32, a permutation of the rows, longest sequence
    first; the matrix-core kernel hands out its workgroups in that order when a launch puts several
    on every CU, so that long and short sequences share CUs.  It changes no result.
    max_len_dev (decode form, optional): a device int32 holding the longest sequence's key count; with
    n_splits > 1 the kernels then cut the keys into n_splits runs of split_chunk(max_len, n_splits) and
    `chunk` is not used, so that one captured launch serves every length up to the block table's width.
    v_transposed, blocked: the layout of the pages (neither: kernel_v_layout of qkv's type and hs).
    row_scale (decode form on the matrix cores with fused_rotate): a DeferredNorm whose factor the rows of qkv still
    lack (qkv is the product of its bf16 copy with the stacked weights); the kernel multiplies q and the new key and
    value of every row by it."""
    require_gpu()
    _dev(qkv, "qkv", dims=2)
    _dev(out, "out", qkv.dtype, 2)
    layout = _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, v_transposed, blocked)
    vt = layout != "rows"
    _dev(block_table, "block_table", torch.int32, 2)
    T = qkv.shape[0]
    if H % Hkv or qkv.shape[1] < H * hs or out.shape != (T, H * hs) or not out.is_contiguous():
        raise KernelError(f"attention: qkv {tuple(qkv.shape)} / out {tuple(out.shape)} do not fit H={H} hs={hs}")
    if hs % 2 or hs < 2 or hs > MAX_HEAD_DIM:
        raise KernelError(f"attention: head size {hs} is not supported (even, at most {MAX_HEAD_DIM})")
    if not block_table.is_contiguous():
        raise KernelError("attention: block_table must be contiguous")
    decode = tiles is None
    use_mfma = layout == "blocked"
    if use_mfma and (force_vector or not mfma_attention(qkv.dtype, hs)):
        raise KernelError(f"attention: blocked pages are read by the matrix-core kernels alone (head size {hs}, "
                          f"force_vector={force_vector})")
    if not use_mfma and mfma_attention(qkv.dtype, hs) and not force_vector:
        force_vector = True          # pages in another order than the matrix-core kernels': the vector kernel reads them
    RT, GT, QT = attention_row_shape(H, Hkv, decode, qkv.dtype if use_mfma else None, hs)
    if decode:
        _dev(seq_lens, "seq_lens", torch.int32, 1)
        if seq_lens.numel() != T or block_table.shape[0] < T or not seq_lens.is_contiguous():
            raise KernelError("attention(decode): one seq_lens entry and one block_table row per token")
        n_tiles = T
    else:
        _dev(tiles, "tiles", torch.int32, 2)
        if tiles.shape[1] != 4 or not tiles.is_contiguous() or qt != QT:
            raise KernelError(f"attention(prompt): tiles must be [n, 4] built for qt={QT}, got qt={qt}")
        n_tiles = tiles.shape[0]
        n_splits, chunk = 1, 0
    if T == 0 or n_tiles == 0:
        return
    part_o = part_ml = None
    fold = F32_FOLD_KEYS if qkv.dtype == torch.float32 else 0       # float32: runs of keys folded in order, in both forms
    if fold:
        if decode and n_splits > 1 and chunk != fold:
            raise KernelError(f"attention: a float32 cache's keys are split in runs of {fold}, not {chunk}")
        max_len_dev = None                                          # and the runs do not follow the longest sequence
    if max_len_dev is not None:
        _dev(max_len_dev, "max_len_dev", torch.int32)
        if not decode or max_len_dev.numel() != 1:
            raise KernelError("attention: max_len_dev is one int32 and belongs to the decode form")
        chunk = split_chunk(block_table.shape[1] * PAGE, n_splits)         # of the longest sequence the table can hold
    if n_splits > 1:
        if chunk <= 0 or chunk % PAGE:
            raise KernelError(f"attention: chunk {chunk} must be a positive multiple of {PAGE}")
        if n_splits * chunk < block_table.shape[1] * PAGE:
            raise KernelError(f"attention: {n_splits} splits of {chunk} keys do not cover the "
                              f"{block_table.shape[1]} pages of the block table")
        if n_splits > (1024 if fold else 64):
            raise KernelError("attention: at most 64 splits (1,024 runs of a float32 cache)")
        part_o = torch.empty((T * H * n_splits, hs), dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty((T * H * n_splits, 2), dtype=torch.float32, device=qkv.device)
    po = part_o.data_ptr() if part_o is not None else None
    pm = part_ml.data_ptr() if part_ml is not None else None
    sl = seq_lens.data_ptr() if decode else None
    tl = tiles.data_ptr() if not decode else None
    if by_length is not None:
        _dev(by_length, "by_length", torch.int32, 1)
        if not decode or by_length.numel() != T or not by_length.is_contiguous():
            raise KernelError("attention: by_length is one entry per row of the decode form")
    fused = fused_rotate is not None or fused_write
    if fused and not (use_mfma and decode and can_fuse_decode(qkv.dtype, H, Hkv, hs)):
        raise KernelError("attention: rotation / cache write inside the kernel needs the decode form on the "
                          "matrix cores with at most 16 heads per kv head")
    if fused_rotate is not None:
        _dev(fused_rotate, "fused_rotate", torch.float32, 1)
        if fused_rotate.numel() != hs // 2 or not fused_rotate.is_contiguous():
            raise KernelError(f"attention: fused rotation needs {hs // 2} frequencies (full rotary)")
    if fused_write and qkv.shape[1] < (H + 2 * Hkv) * hs:
        raise KernelError("attention: fused cache write needs the K and V heads in qkv")
    if row_scale is not None:
        if not (use_mfma and decode and fused_rotate is not None):
            raise KernelError("attention: a deferred norm's factor is applied by the decode form on the matrix cores "
                              "with the rotation inside the kernel, and by nothing else")
        _dev(row_scale.slots, "row_scale.slots", torch.float32, 2)
        if row_scale.slots.shape[0] != T or not row_scale.slots.is_contiguous() or not 1 <= row_scale.slots.shape[1] <= 64:
            raise KernelError(f"attention: row_scale slots {tuple(row_scale.slots.shape)} do not fit {T} rows (1 to 64 pieces)")
        _check(_fn("attn_mfma", "bn_attn_mfma_scaled")(
            qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * hs, k_pages.data_ptr(), v_pages.data_ptr(),
            block_table.data_ptr(), block_table.shape[1], sl, T, H, Hkv, hs, GT, int(window), float(scale), int(n_splits),
            int(chunk), po, pm, fused_rotate.data_ptr(), int(bool(fused_write)),
            by_length.data_ptr() if by_length is not None else None,
            max_len_dev.data_ptr() if max_len_dev is not None else None, row_scale.slots.data_ptr(),
            row_scale.slots.shape[1], row_scale.stream.shape[1], float(row_scale.eps), _stream()), "attention(mfma, scaled)")
        return
    if use_mfma:
        _check(_fn("attn_mfma", "bn_attn_mfma")(
            qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * hs, k_pages.data_ptr(), v_pages.data_ptr(),
            block_table.data_ptr(), block_table.shape[1], sl, tl, n_tiles, T, H, Hkv, hs, GT, int(window),
            float(scale), int(n_splits), int(chunk), po, pm,
            fused_rotate.data_ptr() if fused_rotate is not None else None, int(fused_rotate is not None),
            int(bool(fused_write)), by_length.data_ptr() if by_length is not None else None,
            max_len_dev.data_ptr() if max_len_dev is not None else None, _stream()),
            "attention(mfma)")
        return
    _check(_fn("attn_rows", "bn_attn_rows")(
        _code(qkv.dtype), qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * hs,
        k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1],
        sl, tl, n_tiles, T, H, Hkv, hs, RT, GT, int(window), float(scale), int(n_splits), int(chunk),
        po, pm, int(vt), max_len_dev.data_ptr() if max_len_dev is not None else None, int(fold), _stream()), "attention")


# --------------------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------------------

def _logits_ok(logits):
    _dev(logits, "logits", torch.float32, 2)
    return _rows(logits, "logits")


def argmax(logits: torch.Tensor) -> torch.Tensor:
    require_gpu()
    ld = _logits_ok(logits)
    B, V = logits.shape
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if B:
        wv = wi = None
        if B <= 256 and V >= 16384:          # few rows of a large vocabulary: two stages
            wv = torch.empty((B, 64), dtype=torch.float32, device=logits.device)
            wi = torch.empty((B, 64), dtype=torch.int32, device=logits.device)
        _check(_fn("sampling", "bn_argmax")(logits.data_ptr(), ld, B, V, out.data_ptr(),
                                            wv.data_ptr() if wv is not None else None,
                                            wi.data_ptr() if wi is not None else None, _stream()), "argmax")
    return out


def repeat_penalty_(logits: torch.Tensor, recent: torch.Tensor, penalty: float) -> None:
    """In place: every distinct token id of a row of `recent` (int32, -1 = none) is penalised once."""
    require_gpu()
    ld = _logits_ok(logits)
    _dev(recent, "recent", torch.int32, 2)
    if recent.shape[0] != logits.shape[0] or not recent.is_contiguous():
        raise KernelError("repeat_penalty: one contiguous row of recent tokens per row of logits")
    if logits.shape[0] and recent.shape[1]:
        _check(_fn("sampling", "bn_repeat_penalty")(logits.data_ptr(), ld, logits.shape[0], logits.shape[1],
                                                    recent.data_ptr(), recent.shape[1], float(penalty),
                                                    _stream()), "repeat_penalty")


WIDE_SAMPLE_VOCAB = 16384                 # from this many logits a row on, sampling spreads a row over 32 workgroups
_WIDE_ROW_WORDS = 2 * 4 * 256 + 3 * 32    # WIDE_ROW_WORDS of csrc/sampling.hip


def sample(logits: torch.Tensor, temperature: float, top_p: float, uniforms=None, *,
           force_one_workgroup: bool = False) -> torch.Tensor:
    """One token id per row.  temperature 0: argmax.  uniforms: float32 [B] in [0, 1)."""
    require_gpu()
    if temperature == 0.0:
        return argmax(logits)                 # the same first maximum, in two stages for a large vocabulary
    ld = _logits_ok(logits)
    B, V = logits.shape
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if B == 0:
        return out
    _dev(uniforms, "uniforms", torch.float32, 1)
    if uniforms.numel() != B or not uniforms.is_contiguous():
        raise KernelError("sample: one uniform number per row")
    if V >= WIDE_SAMPLE_VOCAB and B <= 65535 and not force_one_workgroup:
        # a large vocabulary: every pass over a row is spread over 32 workgroups
        ws = torch.zeros((B, _WIDE_ROW_WORDS), dtype=torch.int64, device=logits.device)
        _check(_fn("sampling", "bn_sample_wide")(logits.data_ptr(), ld, B, V, ws.data_ptr(), uniforms.data_ptr(),
                                                 float(temperature), float(top_p), out.data_ptr(), _stream()),
               "sample(wide)")
        return out
    probs = torch.empty((B, V), dtype=torch.float32, device=logits.device)
    _check(_fn("sampling", "bn_sample")(logits.data_ptr(), ld, B, V, probs.data_ptr(), uniforms.data_ptr(),
                                        float(temperature), float(top_p), out.data_ptr(), _stream()), "sample")
    return out
