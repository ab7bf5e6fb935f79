"""Python faces of the HIP kernels.  Each wrapper checks on the host that operand shapes,
dtypes and strides are what its kernel and grid assume, then launches on torch's current
stream.  There is no fallback: without the compiled library every call raises.
"""

from __future__ import annotations

import ctypes
import functools
from ctypes import c_double, c_float, c_int, c_longlong, c_void_p
from typing import Optional, Tuple

import torch

from . import build as _build

EPI_F32, EPI_BF16, EPI_ADD_F32, EPI_SWIGLU_BF16 = 0, 1, 2, 3
ATT_PART = 64          # keys per partition of the bfloat16 attention fold


def fold_group_tiles(head_dim: int) -> int:
    """Tiles (of 16 query columns) one wave of the fold kernel owns; a wave's tiles must belong
    to one sequence, so the host pads every sequence's tile list to a multiple of this."""
    return int(_fn("bw_attention_fold_group_tiles")(int(head_dim)))
HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256)
PAGE_SIZES = (8, 16, 32, 64)       # tokens in a page that the attention kernels and the cache writes take

_ERRORS = {
    -2: "sizes or strides out of the kernel's range",
    -3: "misaligned pointer or stride",
    -4: f"head size not compiled in (supported: {HEAD_DIMS})",
    -5: "page size not supported (a power of two from 4 to 64 is needed)",
    -6: "scratch smaller than attention_decode_scratch asks for",
    -8: "the workgroup's partials do not fit the compute unit's LDS",
    -7: "sizes beyond what the library's static scratch holds",
}

_SIGS = {
    "bw_embed": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_rmsnorm": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "bw_add": [c_void_p, c_void_p, c_longlong, c_void_p],
    "bw_add_bias": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_convert": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_swiglu_f32": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "bw_gather_rows_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_rope_kvwrite": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                        c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_f32": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_add_scratch": [c_int, c_int, c_int, c_void_p, c_void_p],
    "bw_gemm_add_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_longlong, c_void_p,
                         c_int, c_void_p],
    "bw_gemm_add_bf16_static": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_add_bf16_static_max": [c_void_p, c_void_p],
    "bw_gemm_qkv_rope_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_attention_f32_tiles": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p,
                               c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "bw_attention_f32": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                         c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "bw_attention_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_longlong,
                          c_void_p, c_int, c_void_p],
    "bw_attention_decode_scratch": [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    "bw_attention_fold_group_tiles": [c_int],
    "bw_norm_gemm_supported": [c_int, c_int],
    "bw_norm_gemm_wide_supported": [c_int, c_int, c_int, c_int],
    "bw_norm_gemm_bf16": [c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_int, c_void_p],
    "bw_norm_qkv_rope_bf16": [c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                              c_int, c_int, c_int, c_void_p],
    "bw_chain_sync_words": [],
    "bw_chain_begin": [c_void_p, c_int, c_void_p, c_int],
    "bw_chain_flush": [c_void_p],
    "bw_chain_end": [c_void_p],
    "bw_sample": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    "bw_fingerprint": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p],
}

_fns = {}

# While a chain is open (``chain`` below) the library keeps the decode products that can run as phases of one
# launch back; these entry points may be called meanwhile (they join the chain, launch through the library's own
# path that sends the waiting phases first, or launch nothing).  Every other one is a launch that must come after
# what waits.
_CHAIN_KEEPS = frozenset({
    "bw_gemm_bf16", "bw_gemm_add_bf16", "bw_norm_gemm_bf16", "bw_norm_qkv_rope_bf16",
    "bw_gemm_add_scratch", "bw_norm_gemm_supported", "bw_norm_gemm_wide_supported", "bw_attention_decode_scratch",
    "bw_attention_fold_group_tiles", "bw_gemm_add_bf16_static_max", "bw_chain_sync_words", "bw_chain_begin",
    "bw_chain_flush", "bw_chain_end",
})
_chain_open = False


def _fn(name: str):
    if _chain_open and name not in _CHAIN_KEEPS:
        _check(_fn("bw_chain_flush")(_stream()), "chain flush")
    f = _fns.get(name)
    if f is None:
        lib = _build.load()
        f = getattr(lib, name)
        f.argtypes = _SIGS[name]
        f.restype = c_int
        _fns[name] = f
    return f


def available() -> bool:
    """True if the library is built or can be built here (no GPU needed to answer)."""
    try:
        _build.load()
        return True
    except _build.KernelLibraryError:
        return False


def _check(code: int, what: str) -> None:
    if code != 0:
        why = _ERRORS.get(code, f"HIP error {code}")
        raise RuntimeError(f"{what}: {why}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """The current stream's handle (the stream a graph capture has made current, too).  torch's own
    ``current_stream()`` builds a Python object for it at some 8 us a call, which an eager step of a short
    prompt pays 170 times; the raw handle costs a fraction of a microsecond."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, dtype, what: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{what} must live on the GPU (there is no CPU path)")
    if t.dtype != dtype:
        raise ValueError(f"{what} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{what} must be contiguous")


def _is_bf16(t: torch.Tensor, what: str) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise ValueError(f"{what} must be bfloat16 or float32, got {t.dtype}")


# ------------------------------------------------------------------------------ several products, one launch

CHAIN_SPIN_LIMIT = 200000      # looks at a phase's flag before a wait gives up (some tenths of a second)


def chain_sync_words() -> int:
    return int(_fn("bw_chain_sync_words")())


class chain:
    """``with ops.chain(sync, err):`` the decode products of up to 16 rows asked for inside (RMSNorm + product with SwiGLU,
    with a 32-bit store, or with rotation and cache write; residual adds) do not leave one by one: they wait and
    run as phases of one launch, in the order they were asked for, when anything else is launched through this
    module or the block ends.  A phase asks for its weights while the phase before it still runs, and waits inside
    the kernel only for what that phase writes: the same bits, fewer kernel boundaries.  ``sync``: int32 zeros,
    ``chain_sync_words()`` of them (left zero by every launch); ``err``: an int32 word that gets a bit if a wait
    inside a launch gave up (then the step's results are void and ``sync`` has to be zeroed).  Everything put on the
    stream inside the block must come through this module: a launch from elsewhere would overtake what waits."""

    def __init__(self, sync: torch.Tensor, err: torch.Tensor, spin_limit: int = CHAIN_SPIN_LIMIT):
        _need(sync, torch.int32, "sync")
        _need(err, torch.int32, "err")
        if sync.numel() < chain_sync_words() or err.numel() < 1:
            raise ValueError(f"chain: sync needs {chain_sync_words()} words and err one")
        self.sync, self.err, self.spin_limit = sync, err, int(spin_limit)

    def __enter__(self):
        global _chain_open
        if _chain_open:
            raise RuntimeError("a chain is already open")
        _check(_fn("bw_chain_begin")(self.sync.data_ptr(), self.sync.numel(), self.err.data_ptr(), self.spin_limit), "chain")
        _chain_open = True
        return self

    def __exit__(self, *exc):
        global _chain_open
        _chain_open = False
        _check(_fn("bw_chain_end")(_stream()), "chain")
        return False


# ------------------------------------------------------------------------------ row ops

TOKEN_FROM_FEEDBACK = -2     # a token id that means: take this row's token from ``feedback``


def embed(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor, feedback: Optional[torch.Tensor] = None) -> None:
    """out[r, :] = float(table[tokens[r], :]); a negative token gives a zero row, except TOKEN_FROM_FEEDBACK,
    which reads the row's token from ``feedback`` (int32, a row each) if that is given."""
    _need(tokens, torch.int32, "tokens")
    _need(out, torch.float32, "out")
    rows = tokens.numel()
    vocab, width = table.shape
    if not table.is_cuda or not table.is_contiguous():
        raise ValueError("embedding table must be a contiguous GPU tensor")
    if out.shape[0] < rows or out.shape[1] != width:
        raise ValueError(f"embed: out {tuple(out.shape)} does not fit {rows} rows of width {width}")
    if feedback is not None:
        _need(feedback, torch.int32, "feedback")
        if feedback.numel() < rows:
            raise ValueError("embed: feedback is shorter than the rows")
    _check(_fn("bw_embed")(tokens.data_ptr(), None if feedback is None else feedback.data_ptr(), table.data_ptr(),
                           _is_bf16(table, "table"), out.data_ptr(), rows, width, vocab, _stream()), "embed")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, rows: int, eps: float) -> None:
    """out[r] = (x[r] * 1/sqrt(mean(x[r]^2) + eps)) * weight; out float32 (reference order of
    operations) or bfloat16 (32-bit arithmetic, one rounding)."""
    _need(x, torch.float32, "x")
    dim = x.shape[-1]
    if weight.numel() != dim or not weight.is_cuda:
        raise ValueError(f"rmsnorm: weight has {weight.numel()} elements, rows are {dim} wide")
    if x.shape[0] < rows or out.shape[0] < rows or out.shape[-1] != dim or not out.is_contiguous() or not out.is_cuda:
        raise ValueError("rmsnorm: out does not fit x")
    _check(_fn("bw_rmsnorm")(x.data_ptr(), weight.data_ptr(), _is_bf16(weight, "weight"), out.data_ptr(),
                             _is_bf16(out, "out"), rows, dim, out.stride(0), float(eps), _stream()), "rmsnorm")


def add_(x: torch.Tensor, y: torch.Tensor, rows: int) -> None:
    _need(x, torch.float32, "x")
    _need(y, torch.float32, "y")
    if x.shape[1:] != y.shape[1:] or x.shape[0] < rows or y.shape[0] < rows:
        raise ValueError("add_: shapes differ")
    _check(_fn("bw_add")(x.data_ptr(), y.data_ptr(), rows * x.stride(0), _stream()), "add")


def add_bias(x: torch.Tensor, bias: torch.Tensor, rows: int) -> None:
    """x[:rows] += bias (32-bit, one addition an element): a projection's bias behind its product."""
    _need(x, torch.float32, "x")
    _need(bias, torch.float32, "bias")
    if bias.dim() != 1 or bias.shape[0] != x.shape[1] or x.shape[0] < rows:
        raise ValueError(f"add_bias: x {tuple(x.shape)} and bias {tuple(bias.shape)} do not match")
    _check(_fn("bw_add_bias")(x.data_ptr(), bias.data_ptr(), rows, x.shape[1], x.stride(0), _stream()), "add_bias")


def convert(src: torch.Tensor, dst: torch.Tensor, rows: int) -> None:
    """dst[:rows] = src[:rows] between float32 and bfloat16 (narrowing rounds to nearest even)."""
    if not (src.is_cuda and dst.is_cuda) or src.dim() != 2 or dst.dim() != 2:
        raise ValueError("convert: two GPU matrices are needed")
    if src.shape[1] != dst.shape[1] or src.shape[0] < rows or dst.shape[0] < rows:
        raise ValueError(f"convert: {tuple(src.shape)} does not fit {tuple(dst.shape)} for {rows} rows")
    if src.stride(1) != 1 or dst.stride(1) != 1:
        raise ValueError("convert: rows must be contiguous")
    _check(_fn("bw_convert")(src.data_ptr(), _is_bf16(src, "src"), dst.data_ptr(), _is_bf16(dst, "dst"), rows, src.shape[1],
                             src.stride(0), dst.stride(0), _stream()), "convert")


def swiglu_f32(gate_up: torch.Tensor, out: torch.Tensor, rows: int) -> None:
    _need(gate_up, torch.float32, "gate_up")
    _need(out, torch.float32, "out")
    inter = out.shape[1]
    if gate_up.shape[1] != 2 * inter or gate_up.shape[0] < rows or out.shape[0] < rows:
        raise ValueError("swiglu: gate_up must be [rows, 2*inter] for out [rows, inter]")
    _check(_fn("bw_swiglu_f32")(gate_up.data_ptr(), out.data_ptr(), rows, inter, _stream()), "swiglu")


def gather_rows(x: torch.Tensor, index: torch.Tensor, out: torch.Tensor, count: int) -> None:
    _need(x, torch.float32, "x")
    _need(index, torch.int32, "index")
    _need(out, torch.float32, "out")
    if out.shape[1] != x.shape[1] or out.shape[0] < count or index.numel() < count:
        raise ValueError("gather_rows: out does not fit")
    _check(_fn("bw_gather_rows_f32")(x.data_ptr(), index.data_ptr(), out.data_ptr(), count, x.shape[1], x.stride(0),
                                     _stream()), "gather_rows")


def rope_kvwrite(qkv: torch.Tensor, q_out: Optional[torch.Tensor], positions: torch.Tensor, row_seq: torch.Tensor,
                 block_table: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, k_cache: torch.Tensor,
                 v_cache: torch.Tensor, rows: int, heads: int, kv_heads: int, head_dim: int, page_size: int,
                 write_cache: bool = True) -> None:
    """Rotate q and k of every row at its position and store k, v in the row's page slot.
    32-bit caches: q, k rotated in place in ``qkv``.  bfloat16 caches: q goes to ``q_out``."""
    _need(qkv, torch.float32, "qkv")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    bf = _is_bf16(k_cache, "k_cache")
    if v_cache.dtype != k_cache.dtype:
        raise ValueError("k and v caches must have one dtype")
    width = (heads + 2 * kv_heads) * head_dim
    if qkv.shape[1] != width or qkv.shape[0] < rows or positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError(f"rope_kvwrite: qkv must be [>= {rows}, {width}]")
    if cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise ValueError("rope_kvwrite: tables must be [positions, head_dim/2]")
    page_elems = kv_heads * page_size * head_dim
    if k_cache.numel() % page_elems or v_cache.numel() != k_cache.numel():
        raise ValueError("rope_kvwrite: cache size is no multiple of a page")
    if bf:
        if q_out is None:
            raise ValueError("rope_kvwrite: bfloat16 needs q_out")
        _need(q_out, torch.bfloat16, "q_out")
        if q_out.shape[1] != heads * head_dim or q_out.shape[0] < rows:
            raise ValueError("rope_kvwrite: q_out must be [rows, heads*head_dim]")
    _check(_fn("bw_rope_kvwrite")(qkv.data_ptr(), q_out.data_ptr() if q_out is not None else 0, positions.data_ptr(),
                                  row_seq.data_ptr(), block_table.data_ptr(), block_table.stride(0), cos.data_ptr(),
                                  sin.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), bf, rows, heads, kv_heads,
                                  head_dim, page_size, int(write_cache), _stream()), "rope_kvwrite")


# ------------------------------------------------------------------------------ matrix products

def gemm_f32(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows: int, accumulate: bool = False) -> None:
    """out[:rows] (+)= x[:rows] @ w.T with one k-ascending fused multiply-add chain per output."""
    _need(x, torch.float32, "x")
    _need(out, torch.float32, "out")
    if not w.is_cuda or not w.is_contiguous() or w.dim() != 2:
        raise ValueError("gemm_f32: weight must be a contiguous [N, K] GPU tensor")
    N, K = w.shape
    if x.shape[1] != K or out.shape[1] != N or x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError(f"gemm_f32: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not match")
    _check(_fn("bw_gemm_f32")(x.data_ptr(), w.data_ptr(), _is_bf16(w, "weight"), out.data_ptr(), rows, N, K,
                              x.stride(0), out.stride(0), int(accumulate), _stream()), "gemm_f32")


@functools.lru_cache(maxsize=None)
def gemm_add_scratch(rows: int, N: int, K: int) -> Tuple[int, int]:
    """(float32 elements, int32 counters) that a residual add of this shape wants as ``scratch``
    to give every 2048-segment of K workgroups of its own; (0, 0): it would not.  (A function of the
    three sizes alone: asked once for each.)"""
    floats, counters = ctypes.c_longlong(0), ctypes.c_int(0)
    _check(_fn("bw_gemm_add_scratch")(rows, N, K, ctypes.addressof(floats), ctypes.addressof(counters)), "gemm_add_scratch")
    return int(floats.value), int(counters.value)


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows: int, epilogue: int,
              scratch: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> None:
    """out[:rows] = epilogue(x[:rows] @ w.T) on the matrix cores; see gemm_bf16.hip for the
    arithmetic.  EPI_SWIGLU_BF16 takes the stacked weight [2N, K] (gate rows, then up rows).
    ``scratch`` (EPI_ADD_F32 only): the tensors ``gemm_add_scratch`` asks for (float32, int32
    zeros); the bits do not depend on it."""
    _need(x, torch.bfloat16, "x")
    _need(w, torch.bfloat16, "weight")
    if w.dim() != 2:
        raise ValueError("gemm_bf16: weight must be [N, K]")
    N, K = w.shape
    if epilogue == EPI_SWIGLU_BF16:
        if N % 2:
            raise ValueError("gemm_bf16: SwiGLU needs a stacked weight with an even number of rows")
        N //= 2
    want = torch.bfloat16 if epilogue in (EPI_BF16, EPI_SWIGLU_BF16) else torch.float32
    _need(out, want, "out")
    if x.shape[1] != K or out.shape[1] != N or x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError(f"gemm_bf16: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not match")
    if K % 8:
        raise ValueError(f"gemm_bf16: inner size {K} must be a multiple of 8 (16-byte operand loads)")
    if scratch is not None and epilogue == EPI_ADD_F32:
        sc_f, sc_c = scratch
        _need(sc_f, torch.float32, "scratch")
        _need(sc_c, torch.int32, "scratch counters")
        _check(_fn("bw_gemm_add_bf16")(x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, N, K, x.stride(0), out.stride(0),
                                       sc_f.data_ptr(), sc_f.numel(), sc_c.data_ptr(), sc_c.numel(), _stream()), "gemm_bf16")
        return
    _check(_fn("bw_gemm_bf16")(x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, N, K, x.stride(0), out.stride(0),
                               epilogue, _stream()), "gemm_bf16")


# ------------------------------------------------------------------------------ decode fusions

_decode_ok = {}


def norm_gemm_supported(rows: int, inner: int) -> bool:
    """Whether the fused RMSNorm + product kernel (rows kept in LDS) takes this many rows of this width."""
    key = (rows, inner)
    if key not in _decode_ok:
        _decode_ok[key] = bool(_fn("bw_norm_gemm_supported")(rows, inner))
    return _decode_ok[key]


def qkv_rope_head_dim_ok(head_dim: int, inner: int) -> bool:
    """Head sizes the fused norm + q|k|v + rotation kernel takes: multiples of 32 (a workgroup
    is a pair of 16-column strips half a head apart) and 16 or 48 (a workgroup is a head); its epilogue
    reuses the LDS that held the rows, so a workgroup's 32-bit products must fit a row of ``inner`` elements."""
    if head_dim % 16 or head_dim < 16 or not (head_dim % 32 == 0 or head_dim <= 64):
        return False
    return (32 if head_dim % 32 == 0 else head_dim) * 4 <= (inner + 8) * 2


def norm_gemm_wide_supported(rows: int, tiles_of: int, columns: int, inner: int) -> bool:
    """Rows wider than a segment of K (2048): up to 8 of them, up to two segments, for products with at least 64
    workgroups of ``columns`` output columns (``tiles_of`` columns in all)."""
    key = (rows, tiles_of, columns, inner)
    if key not in _decode_ok:
        _decode_ok[key] = bool(_fn("bw_norm_gemm_wide_supported")(rows, tiles_of, inner, columns))
    return _decode_ok[key]


def can_fuse_norm(rows: int, weight: torch.Tensor, x: torch.Tensor, columns: int = 64, stacked: int = 1) -> bool:
    """Whether RMSNorm + product can run as one kernel for this step.  ``columns``: output columns a workgroup of the
    kernel for many columns (32 for SwiGLU and for heads in halves, else 64); ``stacked``: weights stacked in ``weight``
    (2 for gate|up)."""
    K = weight.shape[1]
    if not (weight.dtype == torch.bfloat16 and x.dtype == torch.float32 and x.shape[1] == K and x.stride(0) % 4 == 0):
        return False
    return norm_gemm_supported(rows, K) or norm_gemm_wide_supported(rows, weight.shape[0] // stacked, columns, K)


def norm_gemm_bf16(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor,
                   rows: int, epilogue: int) -> None:
    """out[:rows] = epilogue(rmsnorm(x[:rows]) @ w.T) in one kernel; the bits of rmsnorm followed
    by gemm_bf16.  epilogue as for gemm_bf16 (EPI_SWIGLU_BF16 takes the stacked weight [2N, K])."""
    _need(x, torch.float32, "x")
    _need(w, torch.bfloat16, "weight")
    N, K = w.shape
    if epilogue == EPI_SWIGLU_BF16:
        N //= 2
    _need(out, torch.bfloat16 if epilogue in (EPI_BF16, EPI_SWIGLU_BF16) else torch.float32, "out")
    glu = epilogue == EPI_SWIGLU_BF16
    if not can_fuse_norm(rows, w, x, 32 if glu else 64, 2 if glu else 1) or norm_weight.numel() != K or not norm_weight.is_cuda:
        raise ValueError(f"norm_gemm_bf16: {rows} rows of width {x.shape[1]} against weight {tuple(w.shape)} cannot be fused")
    if out.shape[1] != N or out.shape[0] < rows or x.shape[0] < rows:
        raise ValueError("norm_gemm_bf16: out does not fit")
    _check(_fn("bw_norm_gemm_bf16")(x.data_ptr(), x.stride(0), norm_weight.data_ptr(), _is_bf16(norm_weight, "norm weight"),
                                    float(eps), w.data_ptr(), out.data_ptr(), out.stride(0), rows, N, K, epilogue,
                                    _stream()), "norm_gemm_bf16")


def norm_qkv_rope_bf16(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w_qkv: torch.Tensor, q_out: torch.Tensor,
                       positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor, cos: torch.Tensor,
                       sin: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, rows: int, heads: int,
                       kv_heads: int, head_dim: int, page_size: int, write_cache: bool = True) -> None:
    """RMSNorm, the stacked q|k|v product, rotation and the cache write in one kernel (one
    workgroup per head); the bits of rmsnorm, gemm_bf16 and rope_kvwrite run one after the other."""
    _need(x, torch.float32, "x")
    _need(w_qkv, torch.bfloat16, "qkv weight")
    _need(q_out, torch.bfloat16, "q_out")
    _need(k_cache, torch.bfloat16, "k_cache")
    _need(v_cache, torch.bfloat16, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    N, K = w_qkv.shape
    if N != (heads + 2 * kv_heads) * head_dim or not qkv_rope_head_dim_ok(head_dim, K):
        raise ValueError("norm_qkv_rope_bf16: weight is not [q|k|v] heads of a supported size")
    if not can_fuse_norm(rows, w_qkv, x) or norm_weight.numel() != K:
        raise ValueError("norm_qkv_rope_bf16: this step cannot be fused")
    if q_out.shape[1] != heads * head_dim or q_out.shape[0] < rows or positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("norm_qkv_rope_bf16: buffers too small")
    if cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise ValueError("norm_qkv_rope_bf16: tables must be [positions, head_dim/2]")
    _check(_fn("bw_norm_qkv_rope_bf16")(x.data_ptr(), x.stride(0), norm_weight.data_ptr(),
                                        _is_bf16(norm_weight, "norm weight"), float(eps), w_qkv.data_ptr(),
                                        q_out.data_ptr(), positions.data_ptr(), row_seq.data_ptr(),
                                        block_table.data_ptr(), block_table.stride(0), cos.data_ptr(), sin.data_ptr(),
                                        k_cache.data_ptr(), v_cache.data_ptr(), rows, heads, kv_heads, head_dim, K,
                                        page_size, int(write_cache), _stream()), "norm_qkv_rope_bf16")


# ------------------------------------------------------------------------------ attention

def attention_f32(q: torch.Tensor, positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, rows: int, heads: int,
                  kv_heads: int, head_dim: int, page_size: int, window: int, scale: float) -> None:
    """q: [rows, stride] float32 with head h at columns h*head_dim.. (the stacked q|k|v rows
    serve as they are); caches [pages, kv_heads, page_size, head_dim] float32."""
    _need(q, torch.float32, "q")
    _need(out, torch.float32, "out")
    _need(k_cache, torch.float32, "k_cache")
    _need(v_cache, torch.float32, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    if head_dim not in HEAD_DIMS:
        raise ValueError(f"attention: head size {head_dim} is not supported; supported: {HEAD_DIMS}")
    if q.shape[0] < rows or q.shape[1] < heads * head_dim or out.shape[0] < rows or out.shape[1] != heads * head_dim:
        raise ValueError("attention_f32: q or out too small")
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    _check(_fn("bw_attention_f32")(q.data_ptr(), q.stride(0), positions.data_ptr(), row_seq.data_ptr(),
                                   block_table.data_ptr(), block_table.stride(0), k_cache.data_ptr(),
                                   v_cache.data_ptr(), out.data_ptr(), out.stride(0), rows, heads, kv_heads, head_dim,
                                   page_size, int(window), float(scale), _stream()), "attention_f32")


def attention_f32_tiles(q: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor, tiles: torch.Tensor,
                        num_tiles: int, tiled, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                        heads: int, kv_heads: int, head_dim: int, page_size: int, window: int, scale: float) -> None:
    """``attention_f32`` over tiles ([tiles, 4] int32 = first row, rows, request, 0; a tile's rows are consecutive
    rows of one request).  ``tiled`` True (1): a workgroup per tile of up to 16 rows, keys and values shared
    through LDS; 2: a wave per tile of up to 32 rows, both products as chains of single-step matrix instructions
    (head sizes up to 128 either way); False: a workgroup per tile's first row.  The bits are those of
    ``attention_f32``."""
    _need(q, torch.float32, "q")
    _need(out, torch.float32, "out")
    _need(k_cache, torch.float32, "k_cache")
    _need(v_cache, torch.float32, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(block_table, torch.int32, "block_table")
    _need(tiles, torch.int32, "tiles")
    if head_dim not in HEAD_DIMS or (tiled and head_dim > 128):
        raise ValueError(f"attention: head size {head_dim} is not supported here")
    if tiles.numel() < 4 * num_tiles or q.shape[1] < heads * head_dim or out.shape[1] != heads * head_dim:
        raise ValueError("attention_f32_tiles: tiles, q or out too small")
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    _check(_fn("bw_attention_f32_tiles")(q.data_ptr(), q.stride(0), positions.data_ptr(), block_table.data_ptr(),
                                         block_table.stride(0), tiles.data_ptr(), int(num_tiles), int(tiled),
                                         k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), out.stride(0), heads,
                                         kv_heads, head_dim, page_size, int(window), float(scale), _stream()),
           "attention_f32_tiles")


def attention_bf16(q: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                   tiles: Optional[torch.Tensor], num_tiles: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   out: torch.Tensor, heads: int, kv_heads: int, head_dim: int, page_size: int, window: int,
                   scale: float, decode: bool = False,
                   scratch: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> None:
    """q, out: [rows, heads*head_dim] bfloat16; k pages [kv_heads, page, hd], v pages
    [kv_heads, hd, page]; tiles int32 [n, 4] = (first row, tokens, sequence, 0).

    k_cache and v_cache are [pages, kv_heads*page_size*head_dim]: page numbers from the table
    are clamped into the pool, so a stale table entry can cost nothing worse than a wasted load.

    ``decode`` False: a workgroup folds all partitions for ``fold_group_tiles(head_dim)`` tiles;
    the tiles of a sequence must come in runs padded to that number (empty tiles allowed).
    ``decode`` True (tiles of one token each; ``tiles`` None means "tile t is row t of sequence
    t"): a workgroup per tile whose waves take one 64-key partition each and fold through LDS
    in partition order.  The bits are the same either way.

    ``scratch`` (decode only): the tensors ``attention_decode_scratch`` asks for, (float32, int32
    zeros).  With them a launch of few tiles is split over several workgroups per tile; without
    them it is not.  The bits are the same again."""
    _need(q, torch.bfloat16, "q")
    _need(out, torch.bfloat16, "out")
    _need(k_cache, torch.bfloat16, "k_cache")
    _need(v_cache, torch.bfloat16, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(block_table, torch.int32, "block_table")
    if tiles is not None:
        _need(tiles, torch.int32, "tiles")
    elif not decode:
        raise ValueError("attention_bf16: implicit tiles are for decoded tokens only")
    if head_dim not in HEAD_DIMS:
        raise ValueError(f"attention: head size {head_dim} is not supported; supported: {HEAD_DIMS}")
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    if q.shape[1] != heads * head_dim or out.shape[1] != heads * head_dim or (
            tiles is not None and tiles.numel() < 4 * num_tiles):
        raise ValueError("attention_bf16: q, out or tiles do not fit")
    if tiles is None and (positions.numel() < num_tiles or block_table.shape[0] < num_tiles):
        raise ValueError("attention_bf16: fewer rows or block tables than implicit tiles")
    page_elems = kv_heads * page_size * head_dim
    if k_cache.dim() != 2 or k_cache.shape[1] != page_elems or v_cache.shape != k_cache.shape:
        raise ValueError(f"attention_bf16: caches must be [pages, {page_elems}]")
    sc_f = sc_c = None
    if scratch is not None and decode:
        sc_f, sc_c = scratch
        _need(sc_f, torch.float32, "scratch")
        _need(sc_c, torch.int32, "scratch counters")
    _check(_fn("bw_attention_bf16")(q.data_ptr(), q.stride(0), positions.data_ptr(), block_table.data_ptr(),
                                    block_table.stride(0), tiles.data_ptr() if tiles is not None else 0, num_tiles,
                                    k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[0], out.data_ptr(),
                                    out.stride(0), heads, kv_heads, head_dim, page_size, int(window), float(scale), int(decode),
                                    sc_f.data_ptr() if sc_f is not None else 0, sc_f.numel() if sc_f is not None else 0,
                                    sc_c.data_ptr() if sc_c is not None else 0, sc_c.numel() if sc_c is not None else 0,
                                    _stream()),
           "attention_bf16")


def attention_decode_scratch(num_tiles: int, heads: int, kv_heads: int, head_dim: int, table_stride: int,
                             page_size: int) -> Tuple[int, int]:
    """(float32 elements, int32 counters) that a decode launch of ``num_tiles`` tiles wants as
    ``scratch`` to split its tiles over workgroups; (0, 0): it would not split."""
    floats, counters = ctypes.c_longlong(0), ctypes.c_int(0)
    _check(_fn("bw_attention_decode_scratch")(num_tiles, heads, kv_heads, head_dim, table_stride, page_size,
                                              ctypes.addressof(floats), ctypes.addressof(counters)),
           "attention_decode_scratch")
    return int(floats.value), int(counters.value)


def qkv_rope_gemm_ok(rows: int, head_dim: int, inner: int, all_heads: int = 0) -> bool:
    """Whether the q|k|v product of normalised rows can take rotation and cache write into its
    epilogue.  Up to 64 rows (a workgroup per 32 or 16 rotary pairs of a head), or a few blocks of 64 rows whose
    workgroups are 512 at most: head sizes in multiples of 64, K in steps of 64, and enough heads (q, k and v
    heads together) for 64 workgroups.  More rows: heads of 64 and one segment of K."""
    tiles = all_heads * (head_dim // 64)
    small = head_dim % 64 == 0 and inner % 64 == 0 and tiles >= 64
    if rows > 64:
        # (a few blocks of 64 rows at once, while their workgroups fit the chip together: any head size the small kernel takes)
        at_once = small and tiles * ((rows + 63) // 64) <= 512
        return at_once or (head_dim == 64 and inner <= 2048 and inner % 8 == 0)
    return small


def gemm_qkv_rope_bf16(x: torch.Tensor, w_qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                       row_seq: torch.Tensor, block_table: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor, rows: int, heads: int, kv_heads: int,
                       head_dim: int, page_size: int, write_cache: bool = True) -> None:
    """The stacked q|k|v product with rotation and cache write in its epilogue (the shapes of
    ``qkv_rope_gemm_ok``); the bits of gemm_bf16 into a 32-bit buffer followed by rope_kvwrite."""
    _need(x, torch.bfloat16, "x")
    _need(w_qkv, torch.bfloat16, "qkv weight")
    _need(q_out, torch.bfloat16, "q_out")
    _need(k_cache, torch.bfloat16, "k_cache")
    _need(v_cache, torch.bfloat16, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    N, K = w_qkv.shape
    if N != (heads + 2 * kv_heads) * head_dim or not qkv_rope_gemm_ok(rows, head_dim, K, heads + 2 * kv_heads):
        raise ValueError("gemm_qkv_rope_bf16: not a [q|k|v] weight, or a shape the rotary epilogue does not take")
    if x.shape[1] != K or x.shape[0] < rows or q_out.shape[1] != heads * head_dim or q_out.shape[0] < rows:
        raise ValueError("gemm_qkv_rope_bf16: buffers do not fit")
    if positions.numel() < rows or row_seq.numel() < rows or cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise ValueError("gemm_qkv_rope_bf16: positions or rotary tables do not fit")
    _check(_fn("bw_gemm_qkv_rope_bf16")(x.data_ptr(), x.stride(0), w_qkv.data_ptr(), q_out.data_ptr(),
                                        positions.data_ptr(), row_seq.data_ptr(), block_table.data_ptr(),
                                        block_table.stride(0), cos.data_ptr(), sin.data_ptr(), k_cache.data_ptr(),
                                        v_cache.data_ptr(), rows, heads, kv_heads, head_dim, K, page_size,
                                        int(write_cache), _stream()), "gemm_qkv_rope_bf16")


# ------------------------------------------------------------------------------ sampling

def sample(logits: torch.Tensor, rows: int, temperature: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor) -> None:
    """out[r] = first maximum of row r if temperature[r] <= 0, else the inverse-CDF draw at
    uniform[r] from softmax(logits[r] / temperature[r])."""
    _need(logits, torch.float32, "logits")
    _need(temperature, torch.float32, "temperature")
    _need(uniform, torch.float64, "uniform")
    _need(out, torch.int32, "out")
    if logits.shape[0] < rows or temperature.numel() < rows or uniform.numel() < rows or out.numel() < rows:
        raise ValueError("sample: buffers shorter than the number of rows")
    _check(_fn("bw_sample")(logits.data_ptr(), logits.shape[1], logits.stride(0), rows, temperature.data_ptr(),
                            uniform.data_ptr(), out.data_ptr(), _stream()), "sample")


def fingerprint(logits: torch.Tensor, rows: int, h_in: torch.Tensor, h_out: torch.Tensor) -> None:
    """h_out[r] = the reference's logits hash chained from h_in[r] (int64 bit patterns)."""
    _need(logits, torch.float32, "logits")
    _need(h_in, torch.int64, "h_in")
    _need(h_out, torch.int64, "h_out")
    _check(_fn("bw_fingerprint")(logits.data_ptr(), logits.shape[1], logits.stride(0), rows, h_in.data_ptr(),
                                 h_out.data_ptr(), _stream()), "fingerprint")
