"""Python faces of the HIP kernels: argument checks on the host, then one call into the library.

Every function checks what its kernel and grid assume (device, dtype, contiguity, shapes) before the
launch and raises ``KernelError`` with the library's message when the kernel refuses a size. There is no
other implementation behind these functions: without the built library, or with tensors that are not on
the GPU, they raise.
"""
from __future__ import annotations

import ctypes
import functools
import threading
from typing import Optional, Tuple

import torch

from . import build as _build

F32, BF16 = 0, 1
EPI_STORE, EPI_ADD, EPI_GATED = 0, 1, 2
# gate functions of the gated epilogue by name; the code rides in bits 8 and up of the kernels' epilogue argument
# (csrc/common.h), and a kernel refuses a code it was not built with
GATE_FUNCTIONS = {"silu": 0}


class KernelError(RuntimeError):
    pass


_lib = None
_lock = threading.Lock()
_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_L = ctypes.c_longlong


def library():
    """Loads (building first when nothing current is built) the kernel library."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.ensure_built()
                try:
                    lib = ctypes.CDLL(path)
                except OSError as e:
                    raise KernelError(f"cannot load the kernel library {path}: {e}") from None
                lib.jllm_last_error.restype = ctypes.c_char_p
                _declare(lib)
                _lib = lib
    return _lib


def library_path() -> Optional[str]:
    return _build.find_library()


def _declare(lib) -> None:
    sig = {
        "jllm_embed": [_P, _I, _P, _P, _I, _I, _F, _P],
        "jllm_rmsnorm": [_P, _P, _I, _I, _P, _I, _F, _P, _I, _I, _P],
        "jllm_gemm_generic": [_P, _I, _I, _P, _P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
        "jllm_qk_norm_rope_store": [_P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P],
        "jllm_paged_attention_generic": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _P],
        "jllm_argmax": [_P, _I, _I, _I, _P, _P, _P],
        "jllm_sample": [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P],
        "jllm_adjust_logits": [_P, _I, _P, _P, _I, _F, _F, _F, _P, _P, _I, _P],
        "jllm_token_logprobs": [_P, _I, _I, _I, _P, _I, _P, _P, _P, _P],
        "jllm_copy_words": [_P, _P, _L, _P],
        "jllm_copy_page_rows": [_P, _I, _I, _I, _I, _L, _I, _I, _I, _P],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _I
    lib.jllm_compute_units.argtypes = []
    lib.jllm_compute_units.restype = _I
    lib.jllm_probe_read.argtypes = [_P, _L, _P, _P]
    lib.jllm_probe_read.restype = _I
    lib.jllm_probe_mfma.argtypes = [_I, _P, ctypes.POINTER(ctypes.c_double), _P]
    lib.jllm_probe_mfma.restype = _I
    for name, args in _OPTIONAL_SIGS.items():
        if hasattr(lib, name):
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = _I


_OPTIONAL_SIGS = {
    "jllm_gemm_skinny_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "jllm_gemm_skinny_norm_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _F, _P],
    "jllm_gemm_mfma_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P],
    "jllm_gemm_pingpong_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P],
    "jllm_gemm_stream_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P],
    "jllm_gemm_stream_norm_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _I, _P, _P, _I, _F, _P],
    "jllm_decode_attention_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P, _I, _I, _P],
    "jllm_decode_attention_fused_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _I,
                                         _I, _I, _I, _F, _I, _P, _P, _I, _I, _P],
    "jllm_prefill_attention_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P],
}


def _call(name: str, *args) -> None:
    lib = library()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.jllm_last_error().decode("utf-8", "replace"))


_counts: dict = {}


def stats() -> dict:
    """How often each kernel that may decline a shape ran and declined since the last ``reset_stats``, and how often
    the general kernels ran in their place: {"ran": {name: n}, "declined": {name: n}, "general": {name: n}}. A
    product or attention call that is meant to take a matrix-core kernel shows here when it did not."""
    out = {"ran": {}, "declined": {}, "general": {}}
    for (kind, name), n in _counts.items():
        out[kind][name] = n
    return out


def reset_stats() -> None:
    _counts.clear()


def _count(kind: str, name: str) -> None:
    _counts[(kind, name)] = _counts.get((kind, name), 0) + 1


def _try(name: str, *args) -> bool:
    """Calls a kernel that may decline a shape: True when it ran, False when it declined (another kernel runs)."""
    lib = library()
    fn = getattr(lib, name, None)
    if fn is None:
        _count("declined", name)
        return False
    rc = fn(*args)
    if rc < 0:
        raise KernelError(lib.jllm_last_error().decode("utf-8", "replace"))
    _count("ran" if rc == 0 else "declined", name)
    return rc == 0


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}")


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("the engine's kernels run on the GPU only; got a tensor on " + str(t.device))


def _ptr(t: Optional[torch.Tensor]):
    """The tensor's address as the entry points take it (their pointer arguments are declared, so a plain int does)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current HIP stream's handle. A step of a small model is hundreds of launches whose kernels take a few
    microseconds each, so the host's time per launch is what such a step costs: the handle is asked of torch's own
    binding (a fraction of a microsecond) where it has one, not through a new Stream object (several)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _rows2d(t: torch.Tensor, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what} must be a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")


def _i32(t: Optional[torch.Tensor], n: int, what: str) -> None:
    if t is None:
        return
    if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < n:
        raise KernelError(f"{what} must be a contiguous int32 tensor of at least {n} entries")


# ------------------------------------------------------------------------------------------------ ops


def embed(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """x[t, :] = scale * table[ids[t], :] as fp32 (the residual stream)."""
    _dev(table, ids)
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [vocab, width] tensor")
    n = ids.numel()
    _i32(ids, n, "token ids")
    out = torch.empty((n, table.shape[1]), dtype=torch.float32, device=table.device)
    _call("jllm_embed", _ptr(table), _code(table.dtype), _ptr(ids), _ptr(out), n, table.shape[1], float(scale), _stream())
    return out


def rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of fp32 rows of ``x`` (all, or those listed in ``rows``) into a new tensor of ``out_dtype``."""
    _dev(x, gain, rows)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous():
        raise KernelError("rmsnorm input must be a contiguous fp32 [rows, width] tensor")
    d = x.shape[1]
    if gain.numel() != d or not gain.is_contiguous():
        raise KernelError(f"rmsnorm gain has {gain.numel()} entries, the rows have {d}")
    n = x.shape[0] if rows is None else rows.numel()
    _i32(rows, n, "row list")
    out = activation_rows(n, d, out_dtype, x.device)
    _call("jllm_rmsnorm", _ptr(x), _ptr(rows), n, d, _ptr(gain), _code(gain.dtype), float(eps), _ptr(out),
          _code(out_dtype), out.stride(0), _stream())
    return out


PAD_ROWS_FROM = 128   # from this many rows on, activation rows get a stride that is no multiple of 4 KB
PAD_ELEMENTS = 64


def activation_rows(n: int, width: int, dtype: torch.dtype, device) -> torch.Tensor:
    """An uninitialised [n, width] activation tensor for a product to read. With many rows whose length in bytes is a
    multiple of 4 KB, every row of a tile would start in the same memory channel and the tiles of all compute units
    would queue for it; such rows are laid 64 elements further apart (the tensor is a view with that row stride).
    Measured on the gate/up product of the 8B shape at 2,048 rows: 0.93 -> 1.12 PFLOP/s."""
    if n >= PAD_ROWS_FROM and (width * dtype.itemsize) % 4096 == 0:
        return torch.empty((n, width + PAD_ELEMENTS), dtype=dtype, device=device)[:, :width]
    return torch.empty((n, width), dtype=dtype, device=device)


class NormedRows:
    """RMS-normalised rows that may not have been computed: the fp32 rows ``x``, the gain and eps of the norm and
    the type its output would have. ``gemm`` takes it in place of its input. When the product that last added into
    ``x`` has left ``scaled`` (bf16 ``x * gain``) and ``partials`` (sums of squares of ``x`` per row, in pieces), a
    product of few rows uses those and scales its sums by the rows' rsqrt(mean square + eps) at the end: the norm
    costs no launch and no pass over memory. ``tensor()`` computes the rows for everyone else."""

    def __init__(self, x: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype: torch.dtype,
                 scaled: Optional[torch.Tensor] = None, partials: Optional[torch.Tensor] = None):
        self.x, self.gain, self.eps, self.out_dtype = x, gain, float(eps), out_dtype
        self.scaled, self.partials = scaled, partials
        self._rows = None

    @property
    def shape(self):
        return self.x.shape

    def tensor(self) -> torch.Tensor:
        if self._rows is None:
            self._rows = rmsnorm(self.x, self.gain, self.eps, self.out_dtype)
        return self._rows


def _skinny_norm(a, w, w2, bias, out, epilogue, emit=None, normed: Optional[NormedRows] = None) -> bool:
    """The weight-streaming products (up to 16 rows, up to 64 rows) with a norm on either side; False when the kernel
    does not take the case."""
    M, K = a.shape
    N = w.shape[0]
    if M > STREAM_MAX_ROWS or a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    e_rows, e_gain, e_part = emit if emit is not None else (None, None, None)
    n_part = normed.partials if normed is not None else None
    head = (_ptr(a), a.stride(0), _ptr(w), _ptr(w2), _ptr(bias), _code(bias.dtype) if bias is not None else F32,
            _ptr(out), _code(out.dtype), out.stride(0), M, N, K, int(epilogue))
    tail = (_ptr(e_rows), _ptr(e_gain), _code(e_gain.dtype) if e_gain is not None else F32, _ptr(e_part), _ptr(n_part),
            n_part.shape[1] if n_part is not None else 0, normed.eps if normed is not None else 0.0, _stream())
    few = M <= SKINNY_MAX_ROWS
    rows2 = _skinny_second_rows(N, w2 is not None) if few else 0
    if few and not _few_rows_prefer_stream(N, K, w2 is not None):
        return _try("jllm_gemm_skinny_norm_bf16", *head, rows2, *tail)
    parts = _stream_parts(N, K, w2 is not None) if K % 128 == 0 else 0
    if parts >= 2:
        partial = torch.empty((parts * (2 if w2 is not None else 1) * M * N,), dtype=torch.float32, device=a.device)
        if _try("jllm_gemm_stream_norm_bf16", *head, parts, _ptr(partial), *tail):
            return True
    return few and _try("jllm_gemm_skinny_norm_bf16", *head, rows2, *tail)  # the second kernel declined (N % 256, one part)


def gemm_add_then_norm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gain: torch.Tensor, eps: float,
                       norm_dtype: torch.dtype, *, bias: Optional[torch.Tensor] = None, exact: bool = False) -> NormedRows:
    """``out += a @ w.T (+ bias)`` (the fp32 residual), returning the RMSNorm of the new ``out`` rows, with ``gain``
    and ``eps``, as a ``NormedRows``: for few bf16 rows the product prepares that norm on its way out."""
    if isinstance(a, NormedRows):
        a = a.tensor()
    if not exact and norm_dtype == torch.bfloat16 and a.dim() == 2 and a.shape[0] <= STREAM_MAX_ROWS \
            and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous() \
            and w.shape[1] == a.shape[1] and w.shape[0] % 16 == 0 and a.shape[0] > 0 and a.stride(1) == 1 \
            and out.dtype == torch.float32 and out.dim() == 2 and out.shape == (a.shape[0], w.shape[0]) and out.is_contiguous() \
            and gain.numel() == w.shape[0] and gain.is_contiguous() \
            and (bias is None or (bias.numel() == w.shape[0] and bias.is_contiguous())):
        _dev(a, w, bias, out, gain)
        M, N = out.shape
        scaled = torch.empty((M, N), dtype=torch.bfloat16, device=out.device)
        partials = torch.empty((M, N // 16), dtype=torch.float32, device=out.device)
        if _skinny_norm(a, w, None, bias, out, EPI_ADD, emit=(scaled, gain, partials)):
            return NormedRows(out, gain, eps, norm_dtype, scaled, partials)
    gemm(a, w, bias=bias, out=out, epilogue=EPI_ADD, exact=exact)
    return NormedRows(out, gain, eps, norm_dtype)


def gemm(a: torch.Tensor, w: torch.Tensor, *, w2: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
         out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None, epilogue: int = EPI_STORE,
         exact: bool = False, gate: int = 0) -> torch.Tensor:
    """out = a @ w.T (+ bias) with ``w`` [N, K] row-major.

    EPI_STORE writes ``out_dtype``; EPI_ADD adds into the fp32 ``out`` (the residual stream); EPI_GATED
    writes gate(a @ w.T) * (a @ w2.T) with the gate function of code ``gate`` (``GATE_FUNCTIONS``; 0 = SiLU).
    ``exact`` forces the plain-FMA fp32-accumulation kernel. ``a`` may be a ``NormedRows``.
    """
    normed = None
    if isinstance(a, NormedRows):
        if a.scaled is not None and a._rows is None and not exact:
            normed, a = a, a.scaled
        else:
            a = a.tensor()
    _dev(a, w, w2, bias, out)
    _rows2d(a, "gemm input")
    if w.dim() != 2 or not w.is_contiguous():
        raise KernelError("gemm weight must be a contiguous [N, K] tensor")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"gemm: input rows have {K} entries, weight rows {w.shape[1]}")
    if (epilogue == EPI_GATED) != (w2 is not None):
        raise KernelError("gemm: the gated epilogue takes exactly two weights")
    if gate:
        if epilogue != EPI_GATED or not 0 < gate < (1 << 20):
            raise KernelError(f"gemm: gate function {gate} without the gated epilogue")
        epilogue = int(epilogue) | (int(gate) << 8)  # the kernels take it apart again and refuse what they do not have
    if w2 is not None and (w2.shape != w.shape or w2.dtype != w.dtype or not w2.is_contiguous()):
        raise KernelError("gemm: the two weights of the gated epilogue must agree in shape and type")
    if bias is not None and (bias.numel() != N or not bias.is_contiguous()):
        raise KernelError(f"gemm: bias has {bias.numel()} entries for {N} outputs")
    if epilogue == EPI_ADD:
        if out is None or out.dtype != torch.float32:
            raise KernelError("gemm: the accumulate epilogue needs an fp32 output to add into")
    if out is None:
        out = activation_rows(M, N, out_dtype or a.dtype, a.device)
    _rows2d(out, "gemm output")
    if out.shape[0] != M or out.shape[1] != N:
        raise KernelError(f"gemm: output is {tuple(out.shape)}, expected {(M, N)}")
    if M == 0:
        return out
    if normed is not None:
        if _skinny_norm(a, w, w2, bias, out, epilogue, normed=normed):
            return out
        a = normed.tensor()  # the long way: the norm as a launch of its own
    if not exact and _fast_gemm is not None and _fast_gemm(a, w, w2, bias, out, epilogue):
        return out
    if not exact:
        _count("general", "jllm_gemm_generic")
    _call("jllm_gemm_generic", _ptr(a), _code(a.dtype), a.stride(0), _ptr(w), _ptr(w2), _code(w.dtype), _ptr(bias),
          _code(bias.dtype) if bias is not None else F32, _ptr(out), _code(out.dtype), out.stride(0), M, N, K,
          int(epilogue), _stream())
    return out


MAX_HEAD_DIM = 512     # what the general attention kernel takes (csrc/attention_generic.hip); the fast ones take less
MAX_HEADS = 65535      # query heads + 2 x kv heads: a grid dimension of the kernel that prepares q and k


def check_attention_shape(heads: int, kv_heads: int, head_dim: int, rotary_dim: int) -> None:
    """Raises when no attention kernel of the library takes these sizes, with the limit in the message: asked when a
    model is built, so that a folder whose sizes cannot run is refused at load and not at its first step."""
    if heads <= 0 or kv_heads <= 0 or heads % kv_heads != 0:
        raise KernelError(f"attention: {heads} query heads over {kv_heads} kv heads")
    if not 0 < head_dim <= MAX_HEAD_DIM:
        raise KernelError(f"attention: head_dim {head_dim} is beyond what the attention kernels take (1..{MAX_HEAD_DIM})")
    if heads + 2 * kv_heads > MAX_HEADS:
        raise KernelError(f"attention: {heads} + 2 x {kv_heads} heads are more than the kernels' grids take ({MAX_HEADS})")
    if rotary_dim and (rotary_dim < 2 or rotary_dim > head_dim or rotary_dim % 2):
        raise KernelError(f"attention: a rotary width of {rotary_dim} for head_dim {head_dim} (even, 2..head_dim, is taken)")


SKINNY_MAX_ROWS = 16   # up to here the weight-streaming kernel; its activation traffic grows with the rows
TILE_COLS = 128
# first a workgroup for every compute unit; then two of the small tile's workgroups share a compute unit ...
SPLIT_LONG_STEPS = 16     # ... where each still has this many 64-wide K steps


@functools.lru_cache(maxsize=8192)
def _k_splits(M: int, N: int, K: int, gated: bool) -> int:
    """How many ways the tiled kernel cuts K so that a product with few output tiles still fills the GPU. Splits are
    doubled until every compute unit has a workgroup, and further, up to two per compute unit, only while the K range
    of a workgroup stays long (short ranges are mostly prologue, and every split writes and reads a partial
    result). Measured on the products of the 8B shape at 96 to 1,024 rows against every power of two: this choice
    is the fastest or within 3 % of it; the four products together at 384 rows 324 -> 283 us, at 512 rows
    332 -> 304, at 1,024 rows 559 -> 534 against filling the compute units once."""
    if gated:
        return 1
    tiles = -(-N // TILE_COLS) * -(-M // 128)
    steps = K // 64

    def possible(s):
        return s <= 16 and steps % s == 0 and steps // s >= 4

    splits = 1
    cus = compute_units()
    while tiles * splits < cus and possible(splits * 2):
        splits *= 2
    while tiles * splits * 2 <= 2 * cus and possible(splits * 2) and steps // (splits * 2) >= SPLIT_LONG_STEPS:
        splits *= 2
    return splits


PINGPONG_SPLIT_MIN_K = 1024    # a K range this long per workgroup pays for the partial sums of a cut in two or four
PINGPONG_MIN_ROWS = 257        # below, the 256-row tile is mostly empty rows
# Estimated times, in microseconds, fitted to the sweep that `_pingpong_plan` describes:
PINGPONG_STEP_US = 0.69        # 32 of K on a 256 x 256 tile, one workgroup a compute unit
TILED_STEP_US = 0.54           # 32 of K on the other kernel's 128 x 128 tiles, two workgroups a compute unit
TILED_ROUND_US = 4.4           # what a round of the other kernel's workgroups costs beside its K steps
PINGPONG_SUM_US = 2.3e-6       # per element of a partial result: written in 32-bit, read back and summed
TILED_SUM_US = 1.9e-6


@functools.lru_cache(maxsize=8192)
def _pingpong_plan(M: int, N: int, K: int, gated: bool) -> Tuple[int, int]:
    """(rows of the output tile, ways K is cut) with which the two-group kernel takes a product, or (0, 1) when the
    other tiled kernel is the better choice. The 256 x 256 tile moves the fewest bytes per multiply (a compute unit
    fills its LDS at 32 bytes a clock at most, which is what this tile needs at the matrix cores' full rate) but
    needs enough tiles to fill the compute units; since the kernel's loads cost no vector instructions, K ranges
    down to 1,024 pay as well (ranges of 512 and cuts in eight were slower). A 128-row form of the same kernel was
    measured (86 / 88 us and 222 / 235 alone, 90 / 88 and 254 / 234 inside the model) and not kept.

    Plain products: the choice with the smallest estimated time. Workgroups run in rounds (one per compute unit here,
    two of the other kernel's); a round takes its K steps, and a cut of K adds the partial sums' traffic. The five
    constants were fitted to a sweep of the plain products of the 8B, 14B and 32B shapes at 25 row counts from 320 to
    4,096 (225 cases) with every choice measured (the other kernel, K whole, in two, in four), the other kernel's step
    a little above its least-squares value because near a tie this kernel wins more often: the estimate's choice is
    0.2 % behind the best on average, within 5 % in 222 cases and 8 % behind at worst (8B qkv at 1,152 rows). The
    conditions that stood here before (a fill of 0.6 of the compute units for K whole, cuts only within one round)
    were 3.7 % behind on average and 30 to 54 % where 0.5 to 0.6 of the compute units had a tile and no cut fitted
    (8B qkv at 1,536 rows 126 us against 93; 32B down at 1,792 rows 832 against 539) and 15 to 22 % where a second
    round was a quarter full (14B and 32B down at 4,096 rows)."""
    if K % 32 or K < 128:
        return 0, 1
    cus = compute_units()
    if gated:
        # The gated product cannot cut K, so what decides is how the two kernels' workgroups fall into rounds: this
        # kernel's one per compute unit, the other's (tiles of 128 rows by 64 outputs) two. A round of this kernel takes
        # about 1.25 of the other's. Swept on the 8B, 14B and 32B shapes at 160 to 1,024 rows: within 3 % of the better
        # kernel everywhere (before: 19 % behind at 640 rows of the 8B shape, where 288 tiles are a full round and an
        # eighth of one, and 26 to 32 % at 160 to 256 rows of the 14B shape, where 136 tiles in one round beat 544 small
        # ones in two).
        big = -(-N // 128) * -(-M // 256)
        rounds = -(-big // cus)
        rounds_other = -(-(-(-N // 64) * -(-M // 128)) // (2 * cus))
        if rounds_other > 1:
            return (256, 1) if 1.25 * rounds <= rounds_other else (0, 1)
        # both in one round (65 to 128 rows): the large tile where it gives most compute units a workgroup (gate/up of
        # the 32B shape at 96 and 128 rows, 200 tiles: 143 and 145 us against 160 and 161; the 14B shape's 136 tiles
        # are a tie, the 8B shape's 96 lose, 87 us against 57)
        return (256, 1) if big >= 0.7 * cus else (0, 1)
    if M < PINGPONG_MIN_ROWS:
        return 0, 1
    splits = _k_splits(M, N, K, False)
    rounds = -(-(-(-N // TILE_COLS) * -(-M // 128) * splits) // (2 * cus))
    best = rounds * (TILED_STEP_US * K / (32 * splits) + TILED_ROUND_US) + (TILED_SUM_US * M * N * splits if splits > 1 else 0)
    plan = (0, 1)
    tiles = -(-N // 256) * -(-M // 256)
    for cut in (1, 2, 4):
        if cut > 1 and (K % 64 or (K // 32) % cut or K // cut < PINGPONG_SPLIT_MIN_K):
            continue
        t = -(-tiles * cut // cus) * PINGPONG_STEP_US * K / (32 * cut) + (PINGPONG_SUM_US * M * N * cut if cut > 1 else 0)
        if t < best:
            best, plan = t, (256, cut)
    return plan


STREAM_MAX_ROWS = 64   # up to here the second weight-streaming kernel (activations through LDS)


MI355X_COMPUTE_UNITS = 256      # what the rules below were measured on; stands in where no GPU is visible


@functools.lru_cache(maxsize=None)
def compute_units() -> int:
    """Compute units of the GPU, asked of the device once; on a machine without one, the MI355X's (so that the
    host-side rules can be looked at anywhere)."""
    global _compute_units
    if _compute_units:
        return _compute_units
    if torch.cuda.is_available():
        n = int(library().jllm_compute_units())
        if n > 0:
            _compute_units = n
            return n
    return MI355X_COMPUTE_UNITS


_compute_units = 0


STREAM_PART_COST = 0.02         # what one more part costs (partial sums, a shorter K range), as a fraction, per weight
STREAM_MIN_BLOCKS = 4           # 128-wide K blocks a part has at least


@functools.lru_cache(maxsize=None)
def _stream_parts(N: int, K: int, gated: bool) -> int:
    """How many ways the second weight-streaming kernel cuts K, from N and K alone (never from the number of rows:
    a row's sum must not depend on its batch). A compute unit streams about as fast with one workgroup as with
    two, so what counts is the largest number of workgroups any compute unit gets: the count that minimises
    ceil(workgroups / compute units) / workgroups, times a small price per part. Any count goes, not only powers
    of two. Against a sweep of every count on the four products of the 8B, 14B and 32B shapes at 32 and 64 rows this
    choice is 1 % from the best on average (6 % at worst); doubling up to a target was 10 % (down product of the 14B
    shape: 8 parts, 320 workgroups, 54.9 us; 6 parts 47.2; gate/up: 4 parts, 544 workgroups, 99.1 us; 5 parts
    88.1)."""
    tiles = -(-N // 128)
    nblk = K // 128
    step = 1 if gated else 2
    best, best_cost = 1, None
    COMPUTE_UNITS = compute_units()
    most = 1 if tiles >= 2 * COMPUTE_UNITS else min(nblk, 32)  # many column tiles: rounds are full enough as they are
    for parts in range(1, most + 1):
        per = -(-nblk // parts)
        per = -(-per // step) * step  # whole steps, as the kernel rounds
        if -(-nblk // per) != parts or (parts > 1 and per < STREAM_MIN_BLOCKS):
            continue
        groups = tiles * parts
        cost = -(-groups // COMPUTE_UNITS) / groups * (1.0 + STREAM_PART_COST * parts * (2 if gated else 1))
        if best_cost is None or cost < best_cost - 1e-12:
            best, best_cost = parts, cost
    return best


STREAM_BASE = 1.23     # the second kernel's time against the first's at one row, same bytes, both with full rounds
STREAM_MERGE_MB = 17   # its second launch (the merge of the K parts), in megabytes of streaming time
SKINNY_ROW_COST = 0.45  # what 16 rows of activations add to the first kernel's time, as a fraction


def _round_fill(groups: int) -> float:
    """The share of the compute units' rounds that `groups` workgroups fill."""
    cus = compute_units()
    return groups / (cus * -(-groups // cus))


@functools.lru_cache(maxsize=None)
def _skinny_second_rows(N: int, gated: bool) -> int:
    """Weight rows that a workgroup of the first weight-streaming kernel owns beyond its 16 (0, 4, 8, 12 or 16) for a
    product of up to 16 rows: more than none where N / 16 workgroups leave some compute units with one workgroup more
    than the others and N / (16 + rows) fill their rounds by a fifth more. On 256 compute units N = 6144 gives 24
    rows (256 workgroups against 384) and N = 5120 gives 20 (256 against 320). Measured at 8 rows on N = 5120: K =
    5120 19.2 -> 15.1 us, K = 8192 27.9 -> 21.9, K = 17408 56.4 -> 42.1 (the K-cutting kernel: 45.2), K = 25600
    81.9 -> 60.1 (60.6). Where the rounds fill by less there is nothing to gain: N = 7168 with 28 rows (256 against
    448) 21.6 -> 20.8 us at 8 rows and 17.2 -> 18.2 at one, N = 10240 with 20 rows 29.2 -> 29.0. The gated product
    has its second tile taken (the up weight)."""
    if gated or N % 16:
        return 0
    best, best_fill = 0, _round_fill(N // 16) + 0.2
    for rows in (4, 8, 12, 16):
        if N % (16 + rows) == 0 and _round_fill(N // (16 + rows)) > best_fill + 1e-9:
            best, best_fill = rows, _round_fill(N // (16 + rows))
    return best


@functools.lru_cache(maxsize=None)
def _few_rows_prefer_stream(N: int, K: int, gated: bool) -> bool:
    """Which weight-streaming kernel takes products of up to 16 rows of this shape. The first kernel gives 16 weight
    rows to a workgroup and cannot cut K over workgroups: with N / 16 just above a multiple of the compute units a few
    of them get one workgroup more and everybody waits for those, unless a workgroup can own a few rows more
    (`_skinny_second_rows`). The second kernel cuts K as well and fills its rounds, at the price of a second launch
    and of being a little slower byte for byte. From N and K alone (priced at 8 rows), so that all products of up to
    16 rows of one shape come from one kernel. Measured at 8 rows, first against second kernel, 16 weight rows per
    workgroup: down product of the 14B shape 56.6 / 46.7 us, of the 32B shape 82.4 / 62.3; every product of the 8B
    shape is faster in the first, and so are those two with 20 rows per workgroup (42.1 and 60.1 us)."""
    if K % 128 or N % 16:
        return False
    COMPUTE_UNITS = compute_units()
    fill16 = _round_fill(N // (16 + _skinny_second_rows(N, gated)))
    parts = _stream_parts(N, K, gated)
    groups = -(-N // 128) * parts
    fill = groups / (COMPUTE_UNITS * -(-groups // COMPUTE_UNITS))
    mb = N * K * 2 * (2 if gated else 1) / 1e6
    first = mb / fill16 * (1.0 + SKINNY_ROW_COST * 0.5 * (0.5 if gated else 1.0))
    second = mb / fill * STREAM_BASE + STREAM_MERGE_MB
    return second < 0.95 * first


def _fast_gemm(a, w, w2, bias, out, epilogue) -> bool:
    """The bf16 matrix-core kernels: a weight-streaming one for up to 16 rows, another for up to 64; for many rows
    the two-group kernel with 256 x 256 tiles where enough of them fill the GPU (`_pingpong_plan`), else the other
    tiled kernel (with K cut over several workgroups when the output has few tiles). Each declines shapes it does
    not take; then the plain-FMA kernel runs."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    M, K = a.shape
    N = w.shape[0]
    head = (_ptr(a), a.stride(0), _ptr(w), _ptr(w2), _ptr(bias), _code(bias.dtype) if bias is not None else F32,
            _ptr(out), _code(out.dtype), out.stride(0), M, N, K, int(epilogue))
    if M <= SKINNY_MAX_ROWS and not _few_rows_prefer_stream(N, K, w2 is not None) \
            and _try("jllm_gemm_skinny_bf16", *head, _skinny_second_rows(N, w2 is not None), _stream()):
        return True
    if M <= STREAM_MAX_ROWS and K % 128 == 0:
        parts = _stream_parts(N, K, w2 is not None)
        partial = torch.empty((parts * (2 if w2 is not None else 1) * M * N,), dtype=torch.float32, device=a.device) \
            if parts > 1 else None
        if _try("jllm_gemm_stream_bf16", *head, parts, _ptr(partial), _stream()):
            return True
    tile_rows, cut = _pingpong_plan(M, N, K, w2 is not None)
    if tile_rows:
        partial = torch.empty((cut * M * N,), dtype=torch.float32, device=a.device) if cut > 1 else None
        if _try("jllm_gemm_pingpong_bf16", *head, tile_rows, cut, _ptr(partial), _stream()):
            return True
    splits = _k_splits(M, N, K, w2 is not None) if K % 64 == 0 else 1
    partial = torch.empty((splits * M * N,), dtype=torch.float32, device=a.device) if splits > 1 else None
    if _try("jllm_gemm_mfma_bf16", *head, splits, _ptr(partial), _stream()):
        return True
    return M <= 64 and _try("jllm_gemm_skinny_bf16", *head, 0, _stream())


def qk_norm_rope_store(qkv: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
                       cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], gq: Optional[torch.Tensor],
                       gk: Optional[torch.Tensor], eps: float, heads: int, kv_heads: int, head_dim: int,
                       rotary_dim: int, page_size: int, k_cache: Optional[torch.Tensor],
                       v_cache: Optional[torch.Tensor], write_kv: bool = True) -> None:
    """In place on qkv [T, (H + 2 Hkv) * hd]: per-head RMSNorm of q and k (when gains are given), rotation by
    the table rows of ``positions``, and the store of k and v into the layer's pages at ``slots``."""
    _dev(qkv, positions, slots, cos, sin, gq, gk, k_cache, v_cache)
    _rows2d(qkv, "qkv")
    T = qkv.shape[0]
    if qkv.shape[1] != (heads + 2 * kv_heads) * head_dim:
        raise KernelError(f"qkv rows have {qkv.shape[1]} entries, expected {(heads + 2 * kv_heads) * head_dim}")
    _i32(positions, T, "positions")
    _i32(slots, T, "slots")
    if (cos is None) != (sin is None):
        raise KernelError("cos and sin tables come together")
    if cos is not None:
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or not cos.is_contiguous() or not sin.is_contiguous() \
                or cos.dim() != 2 or cos.shape != sin.shape or cos.shape[1] != rotary_dim // 2:
            raise KernelError("rotary tables must be contiguous fp32 [positions, rotary_dim/2]")
    for g in (gq, gk):
        if g is not None and (g.numel() != head_dim or not g.is_contiguous()):
            raise KernelError(f"q/k norm gain must have head_dim={head_dim} entries")
    if gq is not None and gk is not None and gq.dtype != gk.dtype:
        raise KernelError("q and k norm gains must share a type")
    if write_kv:
        for c in (k_cache, v_cache):
            if c is None or c.dtype != qkv.dtype or not c.is_contiguous() or c.dim() != 4 \
                    or c.shape[1] != kv_heads or c.shape[2] != page_size or c.shape[3] != head_dim:
                raise KernelError("the layer cache must be a contiguous [pages, kv_heads, page_size, head_dim] tensor "
                                  "of the activations' type")
    gd = _code(gq.dtype) if gq is not None else F32
    _call("jllm_qk_norm_rope_store", _ptr(qkv), _code(qkv.dtype), qkv.stride(0), _ptr(positions), _ptr(slots), _ptr(cos),
          _ptr(sin), _ptr(gq), _ptr(gk), gd, float(eps), T, heads, kv_heads, head_dim, rotary_dim, page_size,
          _ptr(k_cache), _ptr(v_cache), 1 if write_kv else 0, _stream())


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    row_req: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int, head_dim: int,
                    window: int, scale: float, meta=None, exact: bool = False,
                    slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of every row of ``q`` [T, H*hd] (a view with any row stride) over its request's pages.
    ``meta`` may carry host-side batch facts (row counts, longest context) that let a faster kernel be chosen.
    ``slopes`` (fp32, one per query head): the score of key j for the row at p gets slopes[h] * (j - p) added (a
    position encoding that biases scores by distance); only the general kernel takes it."""
    _dev(q, k_cache, v_cache, block_table, row_req, positions, slopes)
    if slopes is not None and (slopes.dtype != torch.float32 or slopes.numel() != heads or not slopes.is_contiguous()):
        raise KernelError(f"score slopes must be a contiguous fp32 tensor with one entry per query head ({heads})")
    _rows2d(q, "q")
    T = q.shape[0]
    if q.shape[1] != heads * head_dim:
        raise KernelError(f"q rows have {q.shape[1]} entries, expected {heads * head_dim}")
    for c in (k_cache, v_cache):
        if c.dtype != q.dtype or not c.is_contiguous() or c.dim() != 4 or c.shape[1] != kv_heads or c.shape[3] != head_dim:
            raise KernelError("the layer cache must be a contiguous [pages, kv_heads, page_size, head_dim] tensor")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block table must be a contiguous int32 [requests, max_blocks] tensor")
    _i32(row_req, T, "row -> request map")
    _i32(positions, T, "positions")
    out = activation_rows(T, heads * head_dim, q.dtype, q.device)
    if T == 0:
        return out
    if not exact and slopes is None and _fast_attention is not None and _fast_attention(q, out, k_cache, v_cache, block_table, row_req,
                                                                      positions, heads, kv_heads, head_dim, window,
                                                                      scale, meta):
        return out
    if not exact and slopes is None:
        _count("general", "jllm_paged_attention_generic")
    _call("jllm_paged_attention_generic", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _code(q.dtype), _ptr(k_cache),
          _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(row_req), _ptr(positions), T, heads, kv_heads,
          head_dim, k_cache.shape[2], int(window), float(scale), _ptr(slopes), _stream())
    return out


DECODE_WORKGROUPS_PER_CU = 3   # workgroups of the decode attention that a compute unit holds at once
DECODE_MAX_SPLIT = 1024        # keys per workgroup at most (the kernels take up to 2048)


def _decode_split(rows: int, kv_heads: int, max_ctx: int) -> int:
    """Keys per workgroup of the decode attention: the smallest power of two from 128 to 1,024 with which one round of
    workgroups covers the step (small batches: short ranges, many workgroups; large ones the other way round). A
    workgroup's start (table entries, q, the first keys' latency) and end (the merge of its waves) are paid once per
    range: on 12 layers of the 8B shape ranges of up to 1,024 keys against 512 took a decode step from 3.31 to 3.25 ms
    at batch 64, from 5.23 to 5.08 at batch 128 and from 2.04 to 1.95 at batch 8 with 7,900 keys; 2,048 changes nothing
    more."""
    split = 128 if max_ctx <= 1024 else 256  # beyond that, fewer ranges to merge beat more workgroups even for one row
    resident = DECODE_WORKGROUPS_PER_CU * compute_units()
    while split < DECODE_MAX_SPLIT and rows * kv_heads * (-(-max_ctx // split)) > resident:
        split *= 2
    return split


def _fast_attention(q, out, k_cache, v_cache, block_table, row_req, positions, heads, kv_heads, head_dim, window, scale,
                    meta) -> bool:
    """The bf16 kernels: single rows per request (decode steps) go to the split-key kernel, anything else to the
    matrix-core kernel for portions. Both decline what they do not take; then the general kernel runs. ``meta``
    carries what the host knows about the batch: ``max_context`` (keys of the longest request after this step)
    and ``decode_only``."""
    if q.dtype != torch.bfloat16 or meta is None:
        return False
    T = q.shape[0]
    max_ctx = int(meta["max_context"])
    if meta.get("decode_only"):
        split = _decode_split(T, kv_heads, max_ctx)
        splits = (max_ctx - 1) // split + 1
        part_acc = torch.empty((T * heads * splits * head_dim,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * heads * splits * 2,), dtype=torch.float32, device=q.device)
        return _try("jllm_decode_attention_bf16", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_cache),
                    _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(row_req), _ptr(positions), T, heads,
                    kv_heads, head_dim, k_cache.shape[2], int(window), float(scale), max_ctx - 1, _ptr(part_acc),
                    _ptr(part_ml), splits, split, _stream())
    seg = meta.get("segments_dev")
    if seg is None:
        return False
    n_tiles = meta["n_tiles"]
    single = meta.get("single_rows")
    if single is not None and meta.get("n_tiles_multi", n_tiles) < n_tiles:
        # a mixed step: the requests with one row each (decoding beside prompt portions) lie together and go through
        # the kernel for single rows; the portions' tiles come first in the list, so the list simply ends earlier
        r0, n = single
        rows = slice(r0, r0 + n)
        split = _decode_split(n, kv_heads, max_ctx)
        splits = (max_ctx - 1) // split + 1
        part_acc = torch.empty((n * heads * splits * head_dim,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n * heads * splits * 2,), dtype=torch.float32, device=q.device)
        if _try("jllm_decode_attention_bf16", _ptr(q[rows]), q.stride(0), _ptr(out[rows]), out.stride(0), _ptr(k_cache),
                _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(row_req[rows]), _ptr(positions[rows]), n,
                heads, kv_heads, head_dim, k_cache.shape[2], int(window), float(scale), max_ctx - 1, _ptr(part_acc),
                _ptr(part_ml), splits, split, _stream()):
            n_tiles = meta["n_tiles_multi"]
            if n_tiles == 0:
                return True
    return _try("jllm_prefill_attention_bf16", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_cache),
                _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(seg), _ptr(positions), n_tiles,
                meta["requests"], heads, kv_heads, head_dim, k_cache.shape[2], int(window), max_ctx, float(scale),
                int(meta.get("key_groups", 0)), _stream())


def decode_attention_fused(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                           row_req: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
                           cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], gq: Optional[torch.Tensor],
                           gk: Optional[torch.Tensor], eps: float, heads: int, kv_heads: int, head_dim: int,
                           rotary_dim: int, window: int, scale: float, meta: Optional[dict],
                           write_kv: bool = True) -> Optional[torch.Tensor]:
    """A decode step's whole attention in one launch, from the projection output ``qkv`` [rows, (H + 2 Hkv) * hd]
    (left as it is): q/k norm, rotation, store of the new key and value at ``slots`` and attention over the pages
    in one launch, the merge of the key splits in a second. Returns the output [rows, H * hd], or None when the kernel does not take the case
    (then ``qk_norm_rope_store`` and ``paged_attention`` do the same in three launches."""
    if qkv.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or meta is None or not meta.get("decode_only"):
        return None
    _dev(qkv, k_cache, v_cache, block_table, row_req, positions, slots, cos, sin, gq, gk)
    device = qkv.device
    _rows2d(qkv, "qkv")
    T = qkv.shape[0]
    if qkv.shape[1] != (heads + 2 * kv_heads) * head_dim:
        raise KernelError(f"qkv rows have {qkv.shape[1]} entries, expected {(heads + 2 * kv_heads) * head_dim}")
    _i32(positions, T, "positions")
    _i32(row_req, T, "row_req")
    _i32(slots, T, "slots")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block table must be a contiguous int32 [requests, blocks] tensor")
    if k_cache.shape != v_cache.shape or k_cache.dim() != 4 or k_cache.shape[1] != kv_heads or k_cache.shape[3] != head_dim \
            or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("k/v cache must be contiguous [pages, kv_heads, page_size, head_dim]")
    if (cos is None) != (sin is None) or (gq is None) != (gk is None):
        raise KernelError("cos/sin and the q/k gains come in pairs")
    if cos is not None and (cos.dtype != torch.float32 or sin.dtype != torch.float32 or not cos.is_contiguous()
                            or not sin.is_contiguous() or cos.dim() != 2 or cos.shape != sin.shape
                            or cos.shape[1] != rotary_dim // 2):
        raise KernelError("rotary tables must be contiguous fp32 [positions, rotary_dim/2]")
    for g in (gq, gk):
        if g is not None and (g.numel() != head_dim or not g.is_contiguous()):
            raise KernelError(f"q/k norm gain must have head_dim={head_dim} entries")
    if gq is not None and gq.dtype != gk.dtype:
        return None
    if write_kv and slots is None:
        raise KernelError("a cache write needs slots")
    max_ctx = int(meta["max_context"])
    split = _decode_split(T, kv_heads, max_ctx)
    splits = (max_ctx - 1) // split + 1
    out = torch.empty((T, heads * head_dim), dtype=qkv.dtype, device=device)
    if T == 0:
        return out
    part_acc = torch.empty((T * heads * splits * head_dim,), dtype=torch.float32, device=device)
    part_ml = torch.empty((T * heads * splits * 2,), dtype=torch.float32, device=device)
    ok = _try("jllm_decode_attention_fused_bf16", _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _ptr(k_cache),
              _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(row_req), _ptr(positions), _ptr(slots),
              _ptr(cos), _ptr(sin), _ptr(gq), _ptr(gk), _code(gq.dtype) if gq is not None else F32, float(eps),
              int(rotary_dim), 1 if write_kv else 0, T, heads, kv_heads, head_dim, k_cache.shape[2], int(window),
              float(scale), max_ctx - 1, _ptr(part_acc), _ptr(part_ml), splits, split, _stream())
    return out if ok else None


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Index of the largest entry of each fp32 row, the lowest index among equals."""
    _dev(logits)
    if logits.dtype != torch.float32:
        raise KernelError("argmax takes fp32 logits")
    _rows2d(logits, "logits")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    scratch = torch.empty((logits.shape[0] * 64,), dtype=torch.int32, device=logits.device)  # candidates of long rows
    _call("jllm_argmax", _ptr(logits), logits.stride(0), logits.shape[0], logits.shape[1], _ptr(out), _ptr(scratch),
          _stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    """One token per fp32 row: greedy where temperature is 0 (or top_k is 1), else top-k / top-p / min-p
    filtering and one draw with the row's uniform number in [0, 1)."""
    _dev(logits, temperature, top_k, top_p, min_p, uniform)
    if logits.dtype != torch.float32:
        raise KernelError("sample takes fp32 logits")
    _rows2d(logits, "logits")
    n = logits.shape[0]
    for t, dt, what in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p"), (min_p, torch.float32, "min_p"), (uniform, torch.float64, "uniform")):
        if t.dtype != dt or t.numel() != n or not t.is_contiguous():
            raise KernelError(f"sample: {what} must be a contiguous {dt} tensor with one entry per row")
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _call("jllm_sample", _ptr(logits), logits.stride(0), n, logits.shape[1], _ptr(temperature), _ptr(top_k), _ptr(top_p),
          _ptr(min_p), _ptr(uniform), _ptr(out), _stream())
    return out


def token_logprobs(logits: torch.Tensor, tokens: torch.Tensor, top: int = 0):
    """Natural-log probabilities of ``tokens`` (one per fp32 row) under the softmax of the raw logits, and the
    ``top`` most likely tokens of each row with theirs (most likely first, the lower index first among equals):
    (logprob [n] fp32, ids [n, top] int32, logprobs [n, top] fp32)."""
    _dev(logits, tokens)
    if logits.dtype != torch.float32:
        raise KernelError("token_logprobs takes fp32 logits")
    _rows2d(logits, "logits")
    n, vocab = logits.shape
    _i32(tokens, n, "tokens")
    if not 0 <= top <= vocab:
        raise KernelError(f"{top} alternatives of a vocabulary of {vocab}")
    lp = torch.empty((n,), dtype=torch.float32, device=logits.device)
    ids = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    tlp = torch.empty((n, top), dtype=torch.float32, device=logits.device)
    _call("jllm_token_logprobs", _ptr(logits), logits.stride(0), n, vocab, _ptr(tokens), int(top), _ptr(lp),
          _ptr(ids) if top else None, _ptr(tlp) if top else None, _stream())
    return lp, ids, tlp


def adjust_logits(row: torch.Tensor, seen_ids: Optional[torch.Tensor], counts: Optional[torch.Tensor],
                  repetition: float, presence: float, frequency: float, bias_ids: Optional[torch.Tensor] = None,
                  bias_vals: Optional[torch.Tensor] = None) -> None:
    """In place on one fp32 logits row: repetition / presence / frequency penalties over the seen tokens, then
    the bias entries."""
    _dev(row, seen_ids, counts, bias_ids, bias_vals)
    if row.dtype != torch.float32 or row.dim() != 1 or not row.is_contiguous():
        raise KernelError("adjust_logits takes one contiguous fp32 row")
    n_seen = 0 if seen_ids is None else seen_ids.numel()
    n_bias = 0 if bias_ids is None else bias_ids.numel()
    _i32(seen_ids, n_seen, "seen ids")
    _i32(counts, n_seen, "counts")
    _i32(bias_ids, n_bias, "bias ids")
    if bias_vals is not None and (bias_vals.dtype != torch.float32 or bias_vals.numel() != n_bias):
        raise KernelError("bias values must be fp32, one per bias id")
    _call("jllm_adjust_logits", _ptr(row), row.numel(), _ptr(seen_ids), _ptr(counts), n_seen, float(repetition),
          float(presence), float(frequency), _ptr(bias_ids), _ptr(bias_vals), n_bias, _stream())


def copy_words(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst[:] = src for int32 tensors as a kernel in the current stream; either side may be pinned host memory, which
    the GPU reads or writes itself. The step's description goes up this way and the sampled tokens come down this way:
    a copy through the copy engine is started and waited for outside the stream of kernels (about 0.4 ms of idle GPU
    between two decode steps of 64 requests), and a copy on a second stream slows every launch of the first while
    both are active (0.1 ms of a 3.7 ms step at batch 1)."""
    for t in (src, dst):
        if t.dtype != torch.int32 or not t.is_contiguous() or not (t.is_cuda or t.is_pinned()):
            raise KernelError("copy_words takes contiguous int32 tensors on the GPU or in pinned host memory")
    if src.numel() != dst.numel() or not (src.is_cuda or dst.is_cuda):
        raise KernelError("copy_words copies between tensors of one size, at least one of them on the GPU")
    _call("jllm_copy_words", _ptr(src), _ptr(dst), src.numel(), _stream())


def copy_page_rows(storage: torch.Tensor, src: int, dst: int, rows: int) -> None:
    """Copies the first ``rows`` positions of page ``src`` to page ``dst`` in every run of one per-position tensor of
    a group, laid out [runs, pages, outer, page_size, inner] (any element type; attention's keys: outer = kv heads,
    inner = head size)."""
    _dev(storage)
    if storage.dim() != 5 or not storage.is_contiguous():
        raise KernelError("a group's row storage must be a contiguous [runs, pages, outer, page_size, inner] tensor")
    runs, pages, outer, page_size, inner = storage.shape
    _call("jllm_copy_page_rows", _ptr(storage), runs, pages, outer, page_size, inner * storage.element_size(), int(src),
          int(dst), int(rows), _stream())


def measured_peaks(read_bytes: int = 4 << 30, mfma_iters: int = 20000) -> dict:
    """What this GPU delivers, measured now: read bandwidth of HBM (a kernel that only streams ``read_bytes`` in) in
    bytes a second, and the bf16 matrix-core rate (a kernel that only issues MFMAs from registers) in flop a second.
    The best of three runs each."""
    lib = library()
    dev = torch.device("cuda", torch.cuda.current_device())
    buf = torch.empty(read_bytes, dtype=torch.uint8, device=dev)
    buf.zero_()
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    flops = ctypes.c_double(0.0)

    def timed(launch):
        best = None
        for _ in range(4):  # the first run warms up
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            launch()
            b.record()
            torch.cuda.synchronize()
            t = a.elapsed_time(b) * 1e-3
            best = t if best is None else min(best, t)
        return best

    def read():
        if lib.jllm_probe_read(_ptr(buf), read_bytes, _ptr(sink), _stream()) != 0:
            raise KernelError(lib.jllm_last_error().decode("utf-8", "replace"))

    def mfma():
        if lib.jllm_probe_mfma(mfma_iters, _ptr(sink), ctypes.byref(flops), _stream()) != 0:
            raise KernelError(lib.jllm_last_error().decode("utf-8", "replace"))

    t_read = timed(read)
    t_mfma = timed(mfma)
    del buf
    return {"hbm_read_bytes_per_s": read_bytes / t_read, "mfma_bf16_flop_per_s": flops.value / t_mfma}
