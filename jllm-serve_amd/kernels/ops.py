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
GATE_FUNCTIONS = {"silu": 0, "gelu_tanh": 1, "swish_clamped": 2}  # "swish_clamped" takes a limit (``gate_limit``)


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
        "jllm_gemm_generic": [_P, _I, _I, _P, _P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _P],
        "jllm_qk_norm_rope_store": [_P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P],
        "jllm_paged_attention_generic": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _P],
        "jllm_argmax": [_P, _I, _I, _I, _P, _P, _P],
        "jllm_sample": [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P],
        "jllm_adjust_logits": [_P, _I, _P, _P, _I, _F, _F, _F, _P, _P, _I, _P],
        "jllm_token_logprobs": [_P, _I, _I, _I, _P, _I, _P, _P, _P, _P],
        "jllm_copy_words": [_P, _P, _L, _P],
        "jllm_latent_prepare": [_P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _F, _P, _P, _P, _P, _P, _I, _P, _P],
        "jllm_latent_heads_generic": [_P, _I, _I, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P],
        "jllm_latent_attention_generic": [_P, _I, _P, _I, _I, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _P],
        "jllm_moe_route": [_P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P],
        "jllm_moe_gemm_generic": [_P, _I, _I, _P, _P, _I, _P, _I, _I, _I, _I, _P, _P, _I, _I, _I, _I, _I, _F, _I, _F, _P],
        "jllm_moe_combine": [_P, _P, _I, _I, _I, _F, _P, _P, _P, _P, _I, _I, _I, _P],
        "jllm_moe_router": [_P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _P, _P, _I, _I, _I, _P],
        "jllm_gather_add": [_P, _I, _P, _I, _I, _P, _I, _I, _P],
        "jllm_dyntanh_read": [_P, _P, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _P],
        "jllm_streams_write": [_P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
        "jllm_concat_rows": [_P, _P, _I, _I, _P, _I, _I, _P],
        "jllm_ssm_scan": [_P, _I, _P, _I, _I, _I, _P, _P, _P, _I, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _P],
        "jllm_gated_group_norm": [_P, _I, _P, _I, _I, _P, _I, _F, _I, _I, _I, _P, _I, _I, _P],
        "jllm_copy_page_rows": [_P, _I, _I, _I, _I, _L, _I, _I, _I, _P],
        "jllm_layernorm_seam": [_P, _P, _I, _I, _P, _I, _P, _I, _I, _F, _F, _P, _P, _P, _P, _P, _I, _F, _P, _I, _I, _P],
        "jllm_qkv_prepare": [_P, _I, _I, _I, _P, _P, _I, _I, _I, _I, _I, _P, _P, _I, _F, _P, _P, _I, _F, _I, _P, _P, _I, _I, _I, _P],
        "jllm_attention_dv_generic": [_P, _I, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _F, _I, _P, _P],
        "jllm_heads_finish": [_P, _I, _I, _I, _I, _I, _I, _F, _I, _F, _F, _P, _I, _P, _I, _I, _I, _F, _P, _I, _I, _I, _P],
        "jllm_heads_finish_split": [_P, _I, _I, _I, _I, _I, _F, _I, _F, _F, _P, _I, _P, _I, _I, _I, _F, _P, _I, _I, _I, _P, _P],
        "jllm_short_conv": [_P, _I, _P, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _P, _P],
        "jllm_gated_delta": [_P, _I, _P, _I, _I, _I, _I, _P, _P, _I, _P, _I, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I, _P],
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
    "jllm_gemm_skinny_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "jllm_gemm_skinny_norm_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P, _I, _P, _P, _I, _F, _P],
    "jllm_gemm_mfma_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P],
    "jllm_gemm_pingpong_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P],
    "jllm_gemm_stream_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P],
    "jllm_gemm_stream_norm_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P, _P, _I, _P, _P, _I, _F, _P],
    "jllm_decode_attention_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P, _I, _I, _P],
    "jllm_decode_attention_fused_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _I,
                                         _I, _I, _I, _F, _I, _P, _P, _I, _I, _P],
    "jllm_prefill_attention_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "jllm_latent_attention_bf16": [_P, _I, _P, _I, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P, _I, _I, _P, _P],
    "jllm_latent_heads_bf16": [_P, _I, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P],
    "jllm_gemm_mfma_grouped_bf16": [_P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _I, _I, _P, _I, _P],
    "jllm_attention_dv_bf16": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _F, _F, _I, _I, _P, _I, _I, _I, _P, _P],
    "jllm_moe_gemm_bf16": [_P, _I, _I, _P, _P, _I, _P, _I, _I, _I, _I, _P, _P, _I, _I, _I, _I, _I, _F, _I, _F, _P],
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


def concat_rows(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[a | b] row by row in ``out_dtype``: two fp32 row sets of one shape side by side, as the input of one product."""
    _dev(a, b)
    for t in (a, b):
        if t.dtype != torch.float32 or t.dim() != 2 or not t.is_contiguous():
            raise KernelError("concat_rows takes contiguous fp32 [rows, width] tensors")
    if a.shape != b.shape:
        raise KernelError(f"concat_rows: {tuple(a.shape)} beside {tuple(b.shape)}")
    n, d = a.shape
    out = activation_rows(n, 2 * d, out_dtype, a.device)
    _call("jllm_concat_rows", _ptr(a), _ptr(b), n, d, _ptr(out), _code(out_dtype), out.stride(0), _stream())
    return out


def gather_add(x: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> None:
    """x[t, :] += table[ids[t], :] on fp32 rows (a learned table indexed by position, added at the input)."""
    _dev(x, table, ids)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous() or table.dim() != 2 or not table.is_contiguous() \
            or table.shape[1] != x.shape[1]:
        raise KernelError("gather_add takes contiguous fp32 rows [n, width] and a table [rows, width]")
    n = x.shape[0]
    _i32(ids, n, "row indices")
    _call("jllm_gather_add", _ptr(x), x.stride(0), _ptr(table), _code(table.dtype), table.shape[0], _ptr(ids), n, x.shape[1], _stream())


MAX_STREAMS = 16  # residual streams per row that the stream kernels take (csrc/streams.hip)


def _dyt(weight, bias, alpha, width):
    for t in (weight, bias):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != width:
            raise KernelError(f"the Dynamic-Tanh norm's weight and bias are contiguous fp32 tensors of {width} entries")
    if alpha.dtype != torch.float32 or alpha.numel() != 1:
        raise KernelError("the Dynamic-Tanh norm's slope is one fp32 number on the device")


def dyntanh(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, alpha: torch.Tensor, out_dtype: torch.dtype, *,
            streams: int = 1, read: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            copies: int = 1) -> torch.Tensor:
    """tanh(alpha * u) * weight + bias, element by element, in ``out_dtype``: u is the fp32 row of ``x`` [n, width], or,
    with ``read`` (fp32 [streams]), the weighted sum sum_s read[s] * x[t, s, :] of the row's streams (``x`` [n, streams x
    width]). ``rows``: the input row of every output row; ``copies``: the result is written that many times side by side
    (the start of several streams). No statistics of the row enter: the norm has no mean, variance or eps."""
    _dev(x, weight, bias, alpha, read, rows)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous() or x.shape[1] % max(streams, 1):
        raise KernelError("dyntanh takes contiguous fp32 rows [n, streams x width]")
    width = x.shape[1] // streams
    _dyt(weight, bias, alpha, width)
    if not 1 <= streams <= MAX_STREAMS or (streams > 1 and read is None):
        raise KernelError(f"dyntanh: {streams} streams (1..{MAX_STREAMS}, with their weights)")
    if read is not None and (read.dtype != torch.float32 or not read.is_contiguous() or read.numel() != streams):
        raise KernelError(f"dyntanh: the streams' weights are a contiguous fp32 tensor of {streams} entries")
    n = x.shape[0] if rows is None else rows.numel()
    _i32(rows, n, "row list")
    out = activation_rows(n, copies * width, out_dtype, x.device) if copies == 1 else \
        torch.empty((n, copies * width), dtype=out_dtype, device=x.device)
    _call("jllm_dyntanh_read", _ptr(x), _ptr(rows), n, width, streams, _ptr(read), _ptr(weight), _ptr(bias), _ptr(alpha),
          _ptr(out), _code(out_dtype), out.stride(0), int(copies), _stream())
    return out


def streams_write(x: torch.Tensor, y: torch.Tensor, mix: torch.Tensor, out_w: torch.Tensor, *, nxt=None,
                  out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """Every stream of every row rewritten from the row's previous streams together, in place on ``x`` fp32 [n, streams x width]:
    new[r] = sum_s mix[s, r] * old[s] + out_w[r] * y (``y`` fp32 [n, width], a sublayer's output; ``mix`` fp32 [streams,
    streams]: row = the stream read, column = the stream written). With ``nxt`` = (read [streams], weight, bias, alpha) the next sublayer's input is made
    in the same pass from the new streams and returned in ``out_dtype``: tanh(alpha * sum_r read[r] * new[r]) * weight +
    bias."""
    _dev(x, y, mix, out_w)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous() or y.dtype != torch.float32 or y.dim() != 2 \
            or y.stride(1) != 1 or y.shape[0] != x.shape[0] or x.shape[1] % y.shape[1]:
        raise KernelError("streams_write takes contiguous fp32 streams [n, streams x width] and fp32 rows [n, width]")
    n, width = y.shape
    S = x.shape[1] // width
    if not 1 <= S <= MAX_STREAMS:
        raise KernelError(f"streams_write: {S} streams (1..{MAX_STREAMS} are taken)")
    for t, k in ((mix, S * S), (out_w, S)):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != k:
            raise KernelError(f"streams_write: the mixing matrix and the output weights are contiguous fp32 tensors of {S * S} and {S} entries")
    out = None
    read = w = b = alpha = None
    if nxt is not None:
        read, w, b, alpha = nxt
        _dev(read, w, b, alpha)
        _dyt(w, b, alpha, width)
        if read.dtype != torch.float32 or not read.is_contiguous() or read.numel() != S:
            raise KernelError(f"streams_write: the next read's weights are a contiguous fp32 tensor of {S} entries")
        out = activation_rows(n, width, out_dtype or torch.float32, x.device)
    _call("jllm_streams_write", _ptr(x), _ptr(y), y.stride(0), n, width, S, _ptr(mix), _ptr(out_w), _ptr(read), _ptr(w),
          _ptr(b), _ptr(alpha), _ptr(out), _code(out.dtype) if out is not None else F32, out.stride(0) if out is not None else 0,
          _stream())
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


def _skinny_norm(a, w, w2, bias, out, epilogue, emit=None, normed: Optional[NormedRows] = None,
                 gate_limit: float = 0.0) -> bool:
    """The weight-streaming products (up to 16 rows, up to 64 rows) with a norm on either side; False when the kernel
    does not take the case."""
    M, K = a.shape
    N = w.shape[0]
    if M > STREAM_MAX_ROWS or a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    e_rows, e_gain, e_part = emit if emit is not None else (None, None, None)
    n_part = normed.partials if normed is not None else None
    head = (_ptr(a), a.stride(0), _ptr(w), _ptr(w2), _ptr(bias), _code(bias.dtype) if bias is not None else F32,
            _ptr(out), _code(out.dtype), out.stride(0), M, N, K, int(epilogue), float(gate_limit))
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
         exact: bool = False, gate: int = 0, gate_limit: float = 0.0) -> torch.Tensor:
    """out = a @ w.T (+ bias) with ``w`` [N, K] row-major.

    EPI_STORE writes ``out_dtype``; EPI_ADD adds into the fp32 ``out`` (the residual stream); EPI_GATED
    writes gate(a @ w.T, a @ w2.T) with the gate function of code ``gate`` (``GATE_FUNCTIONS``; 0 = SiLU times the
    second product) and its parameter ``gate_limit`` where it has one.
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
        if _skinny_norm(a, w, w2, bias, out, epilogue, normed=normed, gate_limit=gate_limit):
            return out
        a = normed.tensor()  # the long way: the norm as a launch of its own
    if not exact and _fast_gemm is not None and _fast_gemm(a, w, w2, bias, out, epilogue, gate_limit):
        return out
    if not exact:
        _count("general", "jllm_gemm_generic")
    _call("jllm_gemm_generic", _ptr(a), _code(a.dtype), a.stride(0), _ptr(w), _ptr(w2), _code(w.dtype), _ptr(bias),
          _code(bias.dtype) if bias is not None else F32, _ptr(out), _code(out.dtype), out.stride(0), M, N, K,
          int(epilogue), float(gate_limit), _stream())
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


def _fast_gemm(a, w, w2, bias, out, epilogue, gate_limit: float = 0.0) -> bool:
    """The bf16 matrix-core kernels: a weight-streaming one for up to 16 rows, another for up to 64; for many rows
    the two-group kernel with 256 x 256 tiles where enough of them fill the GPU (`_pingpong_plan`), else the other
    tiled kernel (with K cut over several workgroups when the output has few tiles). Each declines shapes it does
    not take; then the plain-FMA kernel runs."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    M, K = a.shape
    N = w.shape[0]
    head = (_ptr(a), a.stride(0), _ptr(w), _ptr(w2), _ptr(bias), _code(bias.dtype) if bias is not None else F32,
            _ptr(out), _code(out.dtype), out.stride(0), M, N, K, int(epilogue), float(gate_limit))
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


# ------------------------------------------------------------------------------------------------ latent attention

MAX_LATENT = 1024      # the latent a cached row may hold (csrc/latent_generic.hip; the matrix-core kernel takes up to 512)


def check_latent_shape(heads: int, kv_rank: int, rot_dim: int, rot_dims: int) -> None:
    """Raises when no latent-attention kernel takes these sizes; asked when a model is built."""
    if not 0 < heads <= MAX_HEADS:
        raise KernelError(f"latent attention: {heads} heads")
    if not 0 < kv_rank <= MAX_LATENT:
        raise KernelError(f"latent attention: a latent of {kv_rank} is beyond what the kernels take (1..{MAX_LATENT})")
    if rot_dim < 0 or rot_dims < 0 or rot_dims > rot_dim or rot_dims % 2:
        raise KernelError(f"latent attention: {rot_dims} rotated dimensions of a key part of {rot_dim} (even, at most the part)")


def _tables(cos, sin, rot_dims):
    if rot_dims and (cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32
                     or not cos.is_contiguous() or not sin.is_contiguous() or cos.dim() != 2 or cos.shape != sin.shape
                     or cos.shape[1] != rot_dims // 2):
        raise KernelError("rotary tables must be contiguous fp32 [positions, rotary_dim/2]")


def latent_prepare(y: torch.Tensor, q_rank: int, gq: torch.Tensor, eps: float, *, kv_off: int = 0, kv_rank: int = 0,
                   rot_dim: int = 0, rot_dims: int = 0, gkv: Optional[torch.Tensor] = None,
                   positions: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
                   cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                   cache: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From the down-projections' output ``y`` [T, ...] (query latent first): the RMS-normed query latent [T, q_rank]
    (returned), and, with ``cache`` [pages, page_size, kv_rank + rot_dim], the RMS-normed latent y[:, kv_off : kv_off +
    kv_rank] and the key part behind it, rotated at the rows' positions, stored at the rows' ``slots``."""
    _dev(y, gq, gkv, positions, slots, cos, sin, cache)
    _rows2d(y, "latent projections")
    T = y.shape[0]
    if q_rank == 0:  # no query latent: only the cached row is prepared
        if cache is None:
            raise KernelError("latent_prepare: neither a query latent nor a cache to store into")
        cq = None
    else:
        if gq is None or gq.numel() != q_rank or not gq.is_contiguous():
            raise KernelError(f"the query latent's gain has {0 if gq is None else gq.numel()} entries for {q_rank}")
        cq = torch.empty((T, q_rank), dtype=y.dtype, device=y.device)
    if cache is not None:
        if cache.dtype != y.dtype or not cache.is_contiguous() or cache.dim() != 3 or cache.shape[2] != kv_rank + rot_dim:
            raise KernelError("the latent cache must be a contiguous [pages, page_size, kv_rank + rot_dim] tensor of the activations' type")
        if gkv is None or gkv.numel() != kv_rank or not gkv.is_contiguous() or (gq is not None and gkv.dtype != gq.dtype):
            raise KernelError(f"the latent's gain must have {kv_rank} entries of the query gain's type")
        _i32(positions, T, "positions")
        _i32(slots, T, "slots")
        _tables(cos, sin, rot_dims)
    _call("jllm_latent_prepare", _ptr(y), _code(y.dtype), y.stride(0), T, 0, q_rank, kv_off, kv_rank, rot_dim, rot_dims,
          _ptr(gq), _ptr(gkv), _code((gq if gq is not None else gkv).dtype), float(eps), _ptr(positions), _ptr(slots),
          _ptr(cos), _ptr(sin), _ptr(cq), cq.stride(0) if cq is not None else 0, _ptr(cache), _stream())
    return cq


def latent_heads(x: torch.Tensor, w: torch.Tensor, *, tail: int = 0, rot_dims: int = 0,
                 positions: Optional[torch.Tensor] = None, cos: Optional[torch.Tensor] = None,
                 sin: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, exact: bool = False) -> torch.Tensor:
    """One product per head in one launch: ``w`` is [H, N, K]; ``x`` [T, H * (K + tail)] holds each head's K inputs
    followed by ``tail`` more entries. Without ``gate``: out [T, H * (N + tail)], each head's N outputs followed by
    its tail, the first ``rot_dims`` of it rotated at the rows' positions (the query side of latent attention). With
    ``gate`` (a [T, H * N] view, ``tail`` 0): out [T, H * N] = product * sigmoid(gate) (the value side)."""
    _dev(x, w, positions, cos, sin, gate)
    _rows2d(x, "latent_heads input")
    if w.dim() != 3 or not w.is_contiguous():
        raise KernelError("latent_heads weights must be a contiguous [heads, N, K] tensor")
    H, N, K = w.shape
    T = x.shape[0]
    mode = 1 if gate is not None else 0
    if mode == 1 and tail:
        raise KernelError("latent_heads: the gated form has no tail")
    if x.shape[1] != H * (K + tail):
        raise KernelError(f"latent_heads: rows of {x.shape[1]} for {H} heads of {K} + {tail}")
    if mode == 0 and tail:
        _i32(positions, T, "positions")
        _tables(cos, sin, rot_dims)
    if gate is not None:
        _rows2d(gate, "gate rows")
        if gate.shape != (T, H * N) or gate.dtype != x.dtype:
            raise KernelError(f"latent_heads: gate rows are {tuple(gate.shape)}, expected {(T, H * N)} of the input's type")
    out = torch.empty((T, H * (N + tail)), dtype=x.dtype, device=x.device)
    if T == 0:
        return out
    if not exact and _fast_latent_heads(x, w, out, H, N, K, mode, tail, rot_dims, positions, cos, sin, gate):
        return out
    if not exact:
        _count("general", "jllm_latent_heads_generic")
    _call("jllm_latent_heads_generic", _ptr(x), _code(x.dtype), x.stride(0), K + tail, _ptr(w), _code(w.dtype), _ptr(out),
          out.stride(0), N + tail, T, H, N, K, mode, tail, rot_dims, _ptr(positions), _ptr(cos), _ptr(sin), _ptr(gate),
          gate.stride(0) if gate is not None else 0, _stream())
    return out


def _fast_latent_heads(x, w, out, H, N, K, mode, tail, rot_dims, positions, cos, sin, gate) -> bool:
    """The bf16 matrix-core kernel; it declines shapes whose rows do not start on 16-byte boundaries."""
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    return _try("jllm_latent_heads_bf16", _ptr(x), x.stride(0), K + tail, _ptr(w), _ptr(out), out.stride(0), N + tail,
                x.shape[0], H, N, K, mode, tail, rot_dims, _ptr(positions), _ptr(cos), _ptr(sin), _ptr(gate),
                gate.stride(0) if gate is not None else 0, _stream())


def latent_attention(qa: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, row_req: torch.Tensor,
                     positions: torch.Tensor, heads: int, kv_rank: int, window: int, scale: float,
                     sink: Optional[torch.Tensor], meta=None, exact: bool = False) -> torch.Tensor:
    """Causal attention of every row of ``qa`` [T, H * Dk] over its request's cached rows [pages, page_size, Dk]: a
    head's score of a row is its Dk query entries times the row, the values are the rows' first ``kv_rank`` entries;
    the query at p sees keys p + 1 - window .. p (window 0: all); exp(sink[h]) (fp32, one per head) joins the softmax's
    denominator. Returns [T, H * kv_rank]."""
    _dev(qa, cache, block_table, row_req, positions, sink)
    _rows2d(qa, "latent queries")
    T = qa.shape[0]
    if cache.dtype != qa.dtype or not cache.is_contiguous() or cache.dim() != 3:
        raise KernelError("the latent cache must be a contiguous [pages, page_size, Dk] tensor of the queries' type")
    Dk = cache.shape[2]
    if qa.shape[1] != heads * Dk or not 0 < kv_rank <= Dk:
        raise KernelError(f"latent queries have {qa.shape[1]} entries, expected {heads} x {Dk}")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block table must be a contiguous int32 [requests, max_blocks] tensor")
    if sink is not None and (sink.dtype != torch.float32 or sink.numel() != heads or not sink.is_contiguous()):
        raise KernelError(f"the sinks must be a contiguous fp32 tensor with one entry per head ({heads})")
    _i32(row_req, T, "row -> request map")
    _i32(positions, T, "positions")
    out = torch.empty((T, heads * kv_rank), dtype=qa.dtype, device=qa.device)
    if T == 0:
        return out
    if not exact and _fast_latent_attention(qa, out, cache, block_table, row_req, positions, heads, kv_rank, window, scale, sink, meta):
        return out
    if not exact:
        _count("general", "jllm_latent_attention_generic")
    _call("jllm_latent_attention_generic", _ptr(qa), qa.stride(0), _ptr(out), out.stride(0), _code(qa.dtype), _ptr(cache),
          _ptr(block_table), block_table.shape[1], _ptr(row_req), _ptr(positions), T, heads, kv_rank, Dk, cache.shape[1],
          int(window), float(scale), _ptr(sink), _stream())
    return out


LATENT_TILE_ROWS = 16  # rows of one request per run of the step's plan (parts/latent_attention.py)


def _fast_latent_attention(qa, out, cache, block_table, row_req, positions, heads, kv_rank, window, scale, sink, meta) -> bool:
    """The bf16 matrix-core kernel, for portions and single rows alike; it needs the step's runs of rows (``meta``:
    ``tiles_dev``, ``n_tiles``) and declines sizes it does not take."""
    if qa.dtype != torch.bfloat16 or meta is None or meta.get("tiles_dev") is None:
        return False
    n_tiles = int(meta["n_tiles"])
    split, n_z, part = 0, 1, None
    if meta.get("single_rows") and n_tiles == qa.shape[0]:
        split, n_z = _latent_split(n_tiles, heads, int(window), int(meta.get("max_context", 0)))
        if split:
            part = torch.empty((n_tiles * heads * n_z * (kv_rank + 4),), dtype=torch.float32, device=qa.device)
    return _try("jllm_latent_attention_bf16", _ptr(qa), qa.stride(0), _ptr(out), out.stride(0), _ptr(cache),
                _ptr(block_table), block_table.shape[1], _ptr(meta["tiles_dev"]), _ptr(positions), n_tiles,
                LATENT_TILE_ROWS, heads, kv_rank, cache.shape[2], cache.shape[1], int(window), float(scale), _ptr(sink),
                split, n_z, _ptr(part), _stream())


LATENT_SPLIT_MIN = 128  # keys a workgroup takes at least when a row's keys are cut over several


def _latent_split(rows: int, heads: int, window: int, max_ctx: int):
    """(keys per range, ranges per row) for a step of single rows, or (0, 1): a row's keys are cut over several
    workgroups where the step would otherwise leave most compute units idle (few rows, long spans). From the number of
    rows, the heads, the window and the longest context only (what a captured step's bucket fixes)."""
    span = min(window, max_ctx) if window > 0 else max_ctx
    groups = rows * -(-heads // 64)
    want = -(-2 * compute_units() // max(groups, 1))
    if span < 2 * LATENT_SPLIT_MIN or want < 2:
        return 0, 1
    split = max(LATENT_SPLIT_MIN, -(-(-(-span // want)) // 64) * 64)
    n_z = -(-span // split) + 1  # a span of that many keys touches at most this many absolute ranges
    while n_z > 64:  # the merge takes up to 64 ranges
        split *= 2
        n_z = -(-span // split) + 1
    return (split, n_z) if n_z > 2 else (0, 1)


# ------------------------------------------------------------------------------------------------ table-routed experts

# ------------------------------------------------------------------------------------------------ layer norm


def _same_type(what: str, *tensors):
    have = [t for t in tensors if t is not None]
    if any(t.dtype != have[0].dtype or not t.is_contiguous() for t in have):
        raise KernelError(f"{what} must be contiguous tensors of one type")
    return _code(have[0].dtype) if have else F32


def layernorm_seam(residual: torch.Tensor, eps: float, *, a: Optional[torch.Tensor] = None,
                   a2: Optional[torch.Tensor] = None, s1: float = 1.0, s2: float = 1.0, post=None,
                   add_vec: Optional[torch.Tensor] = None, nxt=None, out_dtype: Optional[torch.dtype] = None,
                   rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """What happens to the fp32 residual rows between two sublayers, in one launch, each part optional and in this
    order: ``residual += layer_norm(s1 * a (+ s2 * a2); post)``; ``residual += add_vec``; and the layer norm of the
    (new) rows with ``nxt`` as a new tensor of ``out_dtype``, which is returned. ``post`` and ``nxt`` are (weight,
    bias) pairs. With ``rows`` (int32) only the last part runs, over the listed rows."""
    _dev(residual, a, a2, add_vec, rows)
    if residual.dtype != torch.float32 or residual.dim() != 2 or not residual.is_contiguous():
        raise KernelError("the residual must be a contiguous fp32 [rows, width] tensor")
    n, d = residual.shape
    if rows is not None:
        if a is not None or add_vec is not None:
            raise KernelError("layernorm: a row list goes with the output norm alone")
        n = rows.numel()
        _i32(rows, n, "row list")
    for t in (a, a2):
        if t is not None:
            _rows2d(t, "a sublayer's output")
            if t.shape != (n, d):
                raise KernelError(f"layernorm: a sublayer's output is {tuple(t.shape)}, the residual {(n, d)}")
    if a is None and a2 is not None:
        raise KernelError("layernorm: a second branch without a first")
    if a is not None and a2 is not None and a2.dtype != a.dtype:
        raise KernelError("layernorm: both branches must share a type")
    if (a is not None) != (post is not None):
        raise KernelError("layernorm: a sublayer's output and its norm come together")
    vecs = [v for pair in (post, nxt) if pair is not None for v in pair] + ([add_vec] if add_vec is not None else [])
    for v in vecs:
        _dev(v)
        if v.numel() != d:
            raise KernelError(f"layernorm: a weight, bias or vector has {v.numel()} entries, the rows have {d}")
    wd = _same_type("layernorm weights, biases and vectors", *vecs)
    out = None
    if nxt is not None:
        out = activation_rows(n, d, out_dtype or torch.float32, residual.device)
    if n == 0:
        return out
    _call("jllm_layernorm_seam", _ptr(residual), _ptr(rows), n, d, _ptr(a), a.stride(0) if a is not None else 0, _ptr(a2),
          a2.stride(0) if a2 is not None else 0, _code(a.dtype) if a is not None else F32, float(s1), float(s2),
          _ptr(post[0]) if post else None, _ptr(post[1]) if post else None, _ptr(add_vec),
          _ptr(nxt[0]) if nxt else None, _ptr(nxt[1]) if nxt else None, wd, float(eps), _ptr(out),
          _code(out.dtype) if out is not None else F32, out.stride(0) if out is not None else 0, _stream())
    return out


# ------------------------------------------------------------------------------------------------ attention with sizes of its own


MAX_VALUE_DIM = 512    # what the attention kernels for separate key and value sizes take (csrc/attention_dv.hip)


def check_attention_dv_shape(heads: int, kv_heads: int, maps: int, dk: int, dv: int, rot_dims: int) -> None:
    """Raises when the attention kernels for separate key and value sizes do not take these sizes (asked when a model
    is built)."""
    if heads <= 0 or kv_heads <= 0 or heads % kv_heads != 0 or maps not in (1, 2):
        raise KernelError(f"attention: {heads} query heads over {kv_heads} kv heads with {maps} score maps")
    if not 0 < dv <= MAX_VALUE_DIM or dk <= 0:
        raise KernelError(f"attention: key size {dk}, value size {dv} (values of 1..{MAX_VALUE_DIM} are taken)")
    if (heads + kv_heads) * maps * dk * 4 > 64 * 1024:
        raise KernelError(f"attention: q and k of a row ({(heads + kv_heads) * maps * dk} entries) are more than the preparing kernel holds")
    if rot_dims and (rot_dims < 2 or rot_dims > dk or rot_dims % 2):
        raise KernelError(f"attention: a rotary width of {rot_dims} for heads of {dk} (even, 2..{dk}, is taken)")


def _check_kv_pages(k_cache, v_cache, k_slots, v_heads, dk, dv, dtype):
    if k_cache.dtype != dtype or not k_cache.is_contiguous() or k_cache.dim() != 4 or k_cache.shape[1] != k_slots or k_cache.shape[3] != dk:
        raise KernelError(f"the key pages must be a contiguous [pages, {k_slots}, page_size, {dk}] tensor of the activations' type")
    if v_cache.dtype != dtype or not v_cache.is_contiguous() or v_cache.dim() != 4 or v_cache.shape[1] != v_heads or v_cache.shape[3] != dv \
            or v_cache.shape[2] != k_cache.shape[2] or v_cache.shape[0] != k_cache.shape[0]:
        raise KernelError(f"the value pages must be a contiguous [pages, {v_heads}, page_size, {dv}] tensor beside the key pages")


def qkv_prepare(qkv: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor], heads: int, kv_heads: int,
                maps: int, dk: int, dv: int, k_cache: torch.Tensor, v_cache: torch.Tensor, *,
                gq: Optional[torch.Tensor] = None, gk: Optional[torch.Tensor] = None, eps: float = 0.0,
                cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rot_dims: int = 0,
                temp_coef: float = 0.0, temp_every: int = 0, norm_per_head: bool = False,
                pairing: str = "interleaved") -> None:
    """In place on the first columns of ``qkv`` rows [q: heads x maps x dk | k: kv_heads x maps x dk | v: kv_heads x
    dv]: with ``gq``/``gk`` an RMS norm with those gains over the whole of q and the whole of k (``norm_per_head``: over
    every head alone, with gains [dk] shared by the heads); with ``rot_dims`` the rotation of the pairs (2i, 2i + 1)
    (``pairing`` "half": (i, i + rot_dims / 2)) among the first ``rot_dims`` entries of every q and k head by the table
    rows of the positions; with ``temp_every`` q times 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1); then k and v go to
    the rows' ``slots`` in the pages (``slots`` None or negative entries: nothing is stored)."""
    _dev(qkv, positions, slots, gq, gk, cos, sin, k_cache, v_cache)
    _rows2d(qkv, "qkv")
    T = qkv.shape[0]
    q_slots, k_slots = heads * maps, kv_heads * maps
    if qkv.shape[1] < (q_slots + k_slots) * dk + kv_heads * dv:
        raise KernelError(f"qkv rows have {qkv.shape[1]} entries, fewer than q, k and v take")
    _i32(positions, T, "positions")
    _i32(slots, T, "slots")
    _tables(cos, sin, rot_dims)
    if (gq is None) != (gk is None):
        raise KernelError("the norm over the projections takes gains for both q and k")
    if pairing not in ("interleaved", "half"):
        raise KernelError(f"qkv_prepare: pairing '{pairing}' ('interleaved' and 'half' are built)")
    if gq is not None and norm_per_head and (gq.numel() != dk or gk.numel() != dk):
        raise KernelError(f"the gains of the heads' norm must have {dk} entries each")
    if gq is not None and not norm_per_head and (gq.numel() != q_slots * dk or gk.numel() != k_slots * dk):
        raise KernelError(f"the gains of the norm over the projections must have {q_slots * dk} and {k_slots * dk} entries")
    gd = _same_type("the gains of q and k", gq, gk)
    _check_kv_pages(k_cache, v_cache, k_slots, kv_heads, dk, dv, qkv.dtype)
    _call("jllm_qkv_prepare", _ptr(qkv), qkv.stride(0), _code(qkv.dtype), T, _ptr(positions), _ptr(slots), q_slots, k_slots,
          kv_heads, dk, dv, _ptr(gq), _ptr(gk), gd, float(eps), _ptr(cos), _ptr(sin), int(rot_dims), float(temp_coef),
          int(temp_every), _ptr(k_cache), _ptr(v_cache), k_cache.shape[2], 1 if norm_per_head else 0,
          1 if pairing == "half" else 0, _stream())


def attention_dv(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                 row_req: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int, maps: int, dk: int, dv: int,
                 scale: float, *, softcap: float = 0.0, window: int = 0, out_dtype: Optional[torch.dtype] = None,
                 meta=None, exact: bool = False, defer_merge: bool = False, keep_first: int = 0,
                 sinks: Optional[torch.Tensor] = None):
    """Causal attention of every row of ``q`` [T, heads x maps x dk] over its request's pages, keys [pages, kv_heads x
    maps, page_size, dk] and values [pages, kv_heads, page_size, dv]: map m of head h reads key slot (h / (heads /
    kv_heads)) * maps + m and value head h / (heads / kv_heads). Scores (q . k) * scale, capped as softcap * tanh(score
    / softcap) when ``softcap`` > 0. Returns [T, heads x maps x dv] in ``out_dtype`` (default: q's). With
    ``defer_merge`` a step whose rows were computed in key ranges comes back as a ``SplitHeads`` (the ranges' sums,
    unmerged), which ``heads_finish`` takes in place of the tensor and merges in its prologue. With ``window`` > 0 the
    query at p sees keys p + 1 - window .. p and, with ``keep_first``, the keys before ``keep_first`` as well.
    ``sinks`` (fp32 [heads], one map per head): exp(sink_h) joins head h's softmax denominator and has no value."""
    _dev(q, k_cache, v_cache, block_table, row_req, positions, sinks)
    if sinks is not None and (sinks.dtype != torch.float32 or not sinks.is_contiguous() or sinks.numel() != heads or maps != 1):
        raise KernelError(f"attention: the sinks must be a contiguous fp32 tensor of {heads} entries (and one map per head)")
    if keep_first < 0:
        raise KernelError(f"attention: {keep_first} first keys kept")
    _rows2d(q, "q")
    T = q.shape[0]
    if q.shape[1] != heads * maps * dk:
        raise KernelError(f"q rows have {q.shape[1]} entries, expected {heads * maps * dk}")
    _check_kv_pages(k_cache, v_cache, kv_heads * maps, kv_heads, dk, dv, q.dtype)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block table must be a contiguous int32 [requests, max_blocks] tensor")
    _i32(row_req, T, "row -> request map")
    _i32(positions, T, "positions")
    out = torch.empty((T, heads * maps * dv), dtype=out_dtype or q.dtype, device=q.device)
    if T == 0:
        return out
    if not exact and _fast_attention_dv is not None:
        got = _fast_attention_dv(q, out, k_cache, v_cache, block_table, row_req, positions, heads, kv_heads, maps, dk, dv, scale,
                                 softcap, window, meta, defer_merge, keep_first, sinks)
        if got is not False:
            return out if got is True else got
    if not exact:
        _count("general", "jllm_attention_dv_generic")
    _call("jllm_attention_dv_generic", _ptr(q), q.stride(0), _code(q.dtype), _ptr(out), out.stride(0), _code(out.dtype),
          _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(row_req), _ptr(positions), T, heads,
          kv_heads, maps, dk, dv, k_cache.shape[2], int(window), float(scale), float(softcap), int(keep_first), _ptr(sinks),
          _stream())
    return out


WIDE_TILE_ROWS = 128  # rows of one request per tile of the matrix-core kernel (csrc/attention_dv_mfma.hip)


class SplitHeads:
    """Attention rows that were computed in key ranges and are not merged yet: ``partial`` fp32 [rows x (heads x maps) x
    splits x (dv + 2)] (a range's unnormalised sums, its maximum as an exponent of two, its sum)."""

    def __init__(self, partial: torch.Tensor, splits: int, rows: int, slots: int, dv: int, sinks=None):
        self.partial, self.splits, self.rows, self.slots, self.dv = partial, splits, rows, slots, dv
        self.sinks = sinks  # fp32 [heads] or None: joins the denominator when the ranges are merged


def _fast_attention_dv(q, out, k_cache, v_cache, block_table, row_req, positions, heads, kv_heads, maps, dk, dv, scale,
                       softcap, window, meta, defer_merge=False, keep_first=0, sinks=None):
    """The matrix-core kernel: bf16 pages, fp32 out, and the step's rows cut into tiles by the caller (``meta``:
    "tiles_dev" int32 [n_tiles, 4] as (request, first row, rows, first position or -1), "n_tiles")."""
    tiles = meta.get("tiles_dev") if meta else None
    if tiles is None or q.dtype != torch.bfloat16 or out.dtype != torch.float32:
        return False
    n_tiles = int(meta["n_tiles"])
    _i32(tiles, 4 * n_tiles, "tiles")
    # steps of single rows: the key blocks of a row are shared by as many workgroups as fill the GPU about twice
    splits, per_split, partial = 1, 0, None
    T = q.shape[0]
    if meta.get("single_rows") and n_tiles == T:
        blocks = -(-max(int(meta.get("max_context", 1)), 1) // 64)
        # as many workgroups as are resident at once (two per compute unit; one for the instantiations with keys or
        # values beyond 128, whose LDS buffers fill a unit): a second round would start its chains of loads all over.
        # The heads of a key slot share a workgroup
        resident = (2 if dk <= 128 and dv <= 128 else 1) * compute_units()
        want = max(1, resident // max(1, n_tiles * kv_heads * maps))
        splits = max(1, min(want, blocks // WIDE_SPLIT_MIN_BLOCKS, 64))
        if splits > 1:
            per_split = -(-blocks // splits)
            splits = -(-blocks // per_split)
            partial = torch.empty((T * heads * maps * splits * (dv + 2),), dtype=torch.float32, device=q.device)
    defer = bool(defer_merge and partial is not None and dv <= 256)
    ran = _try("jllm_attention_dv_bf16", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_cache), _ptr(v_cache),
               _ptr(block_table), block_table.shape[1], _ptr(tiles), n_tiles, _ptr(positions), heads, kv_heads, maps, dk, dv,
               k_cache.shape[2], int(window), float(scale), float(softcap), splits, per_split, _ptr(partial),
               T if meta.get("single_rows") else -1, 1 if defer else 0, int(keep_first), _ptr(sinks), _stream())
    if ran and defer:
        return SplitHeads(partial, splits, T, heads * maps, dv, sinks)
    return ran


WIDE_SPLIT_MIN_BLOCKS = 2  # 64-key blocks a workgroup takes at least when a row's keys are shared out


HEAD_GATES = {"sigmoid": 0, "silu": 1}


def heads_finish(att: torch.Tensor, heads: int, maps: int, dv: int, out_dtype: torch.dtype, *, lam: float = 0.0,
                 normed: bool = False, eps: float = 0.0, norm_mul: float = 1.0, gain: Optional[torch.Tensor] = None,
                 gate: Optional[torch.Tensor] = None, gate_fn: str = "sigmoid", out: Optional[torch.Tensor] = None,
                 out_mul: float = 1.0, gate_per_head: bool = False) -> torch.Tensor:
    """From a mixer's heads [T, heads x maps x dv] to the output product's input [T, heads x dv]: with two maps
    o = a1 - lam * a2; ``normed``: o / sqrt(mean(o^2) + eps) * norm_mul per head (times ``gain`` [dv]); with ``gate``
    ([T, heads x dv], a view with any row stride; ``gate_per_head``: [T, heads], one number for a whole head) times
    sigmoid(gate) or, ``gate_fn`` "silu", silu(gate); times
    ``out_mul``. ``out``: where to write (a view with any row stride, [T, heads x dv]) instead of a new tensor."""
    if gate_fn not in HEAD_GATES:
        raise KernelError(f"heads_finish: gate function '{gate_fn}' ({sorted(HEAD_GATES)} are built)")
    split = att if isinstance(att, SplitHeads) else None
    if split is not None:
        if (split.slots, split.dv) != (heads * maps, dv):
            raise KernelError(f"the unmerged attention has {split.slots} slots of {split.dv}, expected {heads * maps} of {dv}")
        att, T = split.partial, split.rows
        _dev(att, gain, gate)
    else:
        _dev(att, gain, gate)
        _rows2d(att, "attention rows")
        T = att.shape[0]
        if att.shape[1] != heads * maps * dv:
            raise KernelError(f"attention rows have {att.shape[1]} entries, expected {heads * maps * dv}")
    if gate is not None:
        _rows2d(gate, "gate")
        if gate.shape != (T, heads if gate_per_head else heads * dv):
            raise KernelError(f"the gate is {tuple(gate.shape)}, expected {(T, heads if gate_per_head else heads * dv)}")
    if gain is not None and (gain.numel() != dv or not gain.is_contiguous()):
        raise KernelError(f"the heads' gain must have {dv} entries")
    if out is None:
        out = activation_rows(T, heads * dv, out_dtype, att.device)
    else:
        _dev(out)
        _rows2d(out, "heads' output")
        if out.shape != (T, heads * dv):
            raise KernelError(f"the heads' output is {tuple(out.shape)}, expected {(T, heads * dv)}")
    if T == 0:
        return out
    if split is not None:
        _call("jllm_heads_finish_split", _ptr(att), split.splits, T, heads, maps, dv, float(lam), 1 if normed else 0, float(eps),
              float(norm_mul), _ptr(gain), _code(gain.dtype) if gain is not None else F32, _ptr(gate),
              gate.stride(0) if gate is not None else 0, _code(gate.dtype) if gate is not None else F32, HEAD_GATES[gate_fn],
              float(out_mul), _ptr(out), out.stride(0), _code(out.dtype), 1 if gate_per_head else 0, _ptr(split.sinks), _stream())
        return out
    _call("jllm_heads_finish", _ptr(att), att.stride(0), _code(att.dtype), T, heads, maps, dv, float(lam), 1 if normed else 0,
          float(eps), float(norm_mul), _ptr(gain), _code(gain.dtype) if gain is not None else F32, _ptr(gate),
          gate.stride(0) if gate is not None else 0, _code(gate.dtype) if gate is not None else F32, HEAD_GATES[gate_fn],
          float(out_mul), _ptr(out), out.stride(0), _code(out.dtype), 1 if gate_per_head else 0, _stream())
    return out


# ------------------------------------------------------------------------------------------------ gated delta rule


MAX_CONV_TAPS = 16


def check_gated_delta_shape(heads: int, kv_heads: int, dk: int, dv: int, taps: int) -> None:
    """Raises when the delta-rule kernels do not take these sizes (asked when a model is built): a lane keeps a
    sixteenth of the key rows of one value column."""
    if heads <= 0 or kv_heads <= 0 or heads % kv_heads != 0:
        raise KernelError(f"gated delta rule: {heads} heads over {kv_heads} key heads")
    if not 1 <= taps <= MAX_CONV_TAPS:
        raise KernelError(f"gated delta rule: a convolution of {taps} taps (1..{MAX_CONV_TAPS} are taken)")
    if not 0 < dk <= 256 or dv <= 0:
        raise KernelError(f"gated delta rule: key size {dk} (1..256 are taken), value size {dv}")


def short_conv(x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, row_req: torch.Tensor, state_slots: torch.Tensor,
               n_requests: int, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu of a causal convolution over time per channel on the first C columns of ``x`` [T, >= C] (a view with any
    row stride), ``taps`` [C, K] with the last column for the current row, plus ``bias`` [C] (of the taps' type) where
    given. A request's rows are consecutive and in
    order; the inputs in front of its first row of this step come from ``state`` [slots, K - 1, C] (fp32, oldest
    first) at the request's slot, and the state then moves on by the step's rows. Returns [T, C]."""
    _dev(x, taps, state, row_req, state_slots, bias)
    _rows2d(x, "convolution input")
    T = x.shape[0]
    if taps.dim() != 2 or not taps.is_contiguous():
        raise KernelError("convolution taps must be a contiguous [channels, taps] tensor")
    C, K = taps.shape
    if bias is not None and (bias.numel() != C or bias.dtype != taps.dtype or not bias.is_contiguous()):
        raise KernelError(f"the convolution's bias must have {C} entries of the taps' type")
    if x.shape[1] < C:
        raise KernelError(f"convolution input rows have {x.shape[1]} entries for {C} channels")
    if state.dtype != torch.float32 or not state.is_contiguous() or (K > 1 and (state.dim() != 3 or state.shape[1:] != (K - 1, C))):
        raise KernelError(f"the convolution's state must be a contiguous fp32 [slots, {K - 1}, {C}] tensor")
    _i32(row_req, T, "row -> request map")
    _i32(state_slots, n_requests, "state slots")
    y = torch.empty((T, C), dtype=x.dtype, device=x.device)
    if T == 0:
        return y
    _call("jllm_short_conv", _ptr(x), x.stride(0), _ptr(y), y.stride(0), _code(x.dtype), T, int(n_requests), C, K, _ptr(taps),
          _ptr(bias), _code(taps.dtype), _ptr(state), _ptr(row_req), _ptr(state_slots), _stream())
    return y


def gated_delta(qkv: torch.Tensor, proj: torch.Tensor, a_off: int, b_off: int, a_log: torch.Tensor, dt_bias: torch.Tensor,
                state: torch.Tensor, row_req: torch.Tensor, state_slots: torch.Tensor, n_requests: int, heads: int,
                kv_heads: int, dk: int, dv: int, decay_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The gated delta rule over the step's rows, request by request and token by token, from and into ``state``
    [slots, heads, dv, dk] (fp32; a head's matrix S [dk, dv] column by column). ``qkv`` [T, kv_heads x dk | kv_heads x dk | heads x dv] are the convolved q, k, v;
    ``proj`` rows hold, at the given offsets, the inputs a and b of decay and write strength (heads each). Per head:
    q and k become unit vectors (q also / sqrt(dk)); beta = sigmoid(b); g = exp(-exp(a_log) softplus(a + dt_bias));
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q. Returns the raw o, fp32 [T, heads x dv]. With
    ``decay_rows`` (fp32 [T, heads x dk]) the decay is one number per head and key channel, g = exp(-exp(a_log[h])
    softplus(decay_rows + dt_bias)) with ``dt_bias`` of heads x dk entries, acting on the rows of S; ``a_off`` is unused."""
    _dev(qkv, proj, a_log, dt_bias, state, row_req, state_slots, decay_rows)
    channel = decay_rows is not None
    _rows2d(qkv, "convolved q, k, v")
    _rows2d(proj, "projection rows")
    T = qkv.shape[0]
    if proj.shape[0] != T or proj.dtype != qkv.dtype:
        raise KernelError("the projection rows and the convolved rows must agree in rows and type")
    if qkv.shape[1] != 2 * kv_heads * dk + heads * dv:
        raise KernelError(f"convolved rows have {qkv.shape[1]} entries, expected {2 * kv_heads * dk + heads * dv}")
    if channel:
        _rows2d(decay_rows, "decay rows")
        if decay_rows.dtype != torch.float32 or decay_rows.shape != (T, heads * dk):
            raise KernelError(f"the decay rows must be fp32 {(T, heads * dk)}, got {tuple(decay_rows.shape)} {decay_rows.dtype}")
        a_off = 0
    if max(a_off + (0 if channel else heads), b_off + heads) > proj.shape[1] or min(a_off, b_off) < 0:
        raise KernelError("a or b lie outside the projection rows")
    if a_log.numel() != heads or dt_bias.numel() != (heads * dk if channel else heads):
        raise KernelError(f"a_log must have {heads} entries, dt_bias {heads * dk if channel else heads}")
    wd = _same_type("a_log and dt_bias", a_log, dt_bias)
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 4 or state.shape[1:] != (heads, dv, dk):
        raise KernelError(f"the state must be a contiguous fp32 [slots, {heads}, {dv}, {dk}] tensor")
    _i32(row_req, T, "row -> request map")
    _i32(state_slots, n_requests, "state slots")
    out = torch.empty((T, heads * dv), dtype=torch.float32, device=qkv.device)
    if T == 0:
        return out
    # what the preparing kernel leaves for the recurrence: unit q and k, decay, write strength and q . k, in fp32
    prep = torch.empty((T, 2 * kv_heads * dk + 2 * heads + kv_heads + (heads * dk if channel else 0)), dtype=torch.float32,
                       device=qkv.device)
    _call("jllm_gated_delta", _ptr(qkv), qkv.stride(0), _ptr(proj), proj.stride(0), int(a_off), int(b_off), _code(qkv.dtype),
          _ptr(a_log), _ptr(dt_bias), wd, _ptr(prep), prep.stride(0), _ptr(state), _ptr(out), out.stride(0), _ptr(row_req),
          _ptr(state_slots), T, int(n_requests), heads, kv_heads, dk, dv, _ptr(decay_rows),
          decay_rows.stride(0) if channel else 0, _stream())
    return out


# ------------------------------------------------------------------------------------------------ state-space recurrence

MAX_SSM_STATE = 256    # state rows per head that the recurrence keeps in registers (csrc/ssm_scan.hip)


def check_ssm_shape(heads: int, groups: int, state: int, dv: int, taps: int) -> None:
    """Raises when the state-space kernels do not take these sizes (asked when a model is built)."""
    if heads <= 0 or groups <= 0 or heads % groups != 0:
        raise KernelError(f"state-space recurrence: {heads} heads over {groups} groups")
    if not 1 <= taps <= MAX_CONV_TAPS:
        raise KernelError(f"state-space recurrence: a convolution of {taps} taps (1..{MAX_CONV_TAPS} are taken)")
    if not 0 < state <= MAX_SSM_STATE or dv <= 0:
        raise KernelError(f"state-space recurrence: state size {state} (1..{MAX_SSM_STATE} are taken), value size {dv}")


def ssm_scan(xbc: torch.Tensor, proj: torch.Tensor, dt_off: int, a_log: torch.Tensor, dt_bias: torch.Tensor, skip: torch.Tensor,
             state: torch.Tensor, row_req: torch.Tensor, state_slots: torch.Tensor, n_requests: int, heads: int, groups: int,
             n: int, dv: int) -> torch.Tensor:
    """A selective state-space recurrence over the step's rows, request by request and token by token, from and into
    ``state`` [slots, heads, dv, n] (fp32; a head's matrix S [n, dv] column by column). ``xbc`` [T, heads x dv | groups x n | groups x n] are the convolved x, B, C;
    ``proj`` rows hold the step sizes' input (heads entries) from ``dt_off`` on. Per head (its group's B and C):
    dt = softplus(dt_in + dt_bias); S <- exp(-exp(a_log) dt) S + dt B x^T; y = S^T C + skip x. Returns y, fp32
    [T, heads x dv]."""
    _dev(xbc, proj, a_log, dt_bias, skip, state, row_req, state_slots)
    _rows2d(xbc, "convolved x, B, C")
    _rows2d(proj, "projection rows")
    T = xbc.shape[0]
    if proj.shape[0] != T or proj.dtype != xbc.dtype:
        raise KernelError("the projection rows and the convolved rows must agree in rows and type")
    if xbc.shape[1] != heads * dv + 2 * groups * n:
        raise KernelError(f"convolved rows have {xbc.shape[1]} entries, expected {heads * dv + 2 * groups * n}")
    if dt_off < 0 or dt_off + heads > proj.shape[1]:
        raise KernelError("the step sizes lie outside the projection rows")
    if a_log.numel() != heads or dt_bias.numel() != heads or skip.numel() != heads:
        raise KernelError(f"a_log, dt_bias and the skip weights must have {heads} entries")
    wd = _same_type("a_log, dt_bias and the skip weights", a_log, dt_bias, skip)
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 4 or state.shape[1:] != (heads, dv, n):
        raise KernelError(f"the state must be a contiguous fp32 [slots, {heads}, {dv}, {n}] tensor")
    _i32(row_req, T, "row -> request map")
    _i32(state_slots, n_requests, "state slots")
    out = torch.empty((T, heads * dv), dtype=torch.float32, device=xbc.device)
    if T == 0:
        return out
    _call("jllm_ssm_scan", _ptr(xbc), xbc.stride(0), _ptr(proj), proj.stride(0), int(dt_off), _code(xbc.dtype), _ptr(a_log),
          _ptr(dt_bias), _ptr(skip), wd, _ptr(state), _ptr(out), out.stride(0), _ptr(row_req), _ptr(state_slots), T,
          int(n_requests), heads, groups, n, dv, _stream())
    return out


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float, groups: int,
                     out_dtype: torch.dtype) -> torch.Tensor:
    """rmsnorm(y * silu(z)) * weight with the root mean square taken over each of ``groups`` equal parts of a row: ``y``
    fp32 [T, width], ``z`` [T, width] (a view with any row stride), ``weight`` [width]. The gate comes before the norm."""
    _dev(y, z, weight)
    _rows2d(y, "rows to norm")
    _rows2d(z, "gate rows")
    T, width = y.shape
    if y.dtype != torch.float32 or z.shape != (T, width):
        raise KernelError(f"gated_group_norm: fp32 rows {tuple(y.shape)} with a gate of {tuple(z.shape)}")
    if weight.numel() != width or not weight.is_contiguous() or groups <= 0 or width % groups:
        raise KernelError(f"gated_group_norm: a weight of {weight.numel()} for rows of {width} in {groups} groups")
    out = activation_rows(T, width, out_dtype, y.device)
    if T == 0:
        return out
    _call("jllm_gated_group_norm", _ptr(y), y.stride(0), _ptr(z), z.stride(0), _code(z.dtype), _ptr(weight), _code(weight.dtype),
          float(eps), T, width, int(groups), _ptr(out), _code(out_dtype), out.stride(0), _stream())
    return out


MOE_TILE_ROWS = 16      # rows of one expert that a workgroup of the grouped products takes in steps of few rows ...
MOE_TILE_ROWS_MANY = 128  # ... and where the experts get many rows each (portions of prompts): the tiled product's tile


class MoeRouting:
    """What ``moe_route`` made of a step: ``sorted`` [T * top] (the assignments t * top + k expert by expert), ``tiles``
    [max_tiles, 3] (expert, first place in sorted, rows; 0 rows = unused), ``place_of`` [T * top] (where each
    assignment lies in sorted) and the rows a tile holds at most."""

    def __init__(self, sorted_, tiles, place_of, max_tiles, tile_rows, top):
        self.sorted, self.tiles, self.place_of = sorted_, tiles, place_of
        self.max_tiles, self.tile_rows, self.top = max_tiles, tile_rows, top

    @property
    def many(self) -> bool:
        return self.tile_rows == MOE_TILE_ROWS_MANY


def moe_router(z: torch.Tensor, correction: Optional[torch.Tensor], groups: int, keep: int, top: int, scale: float,
               score: str = "sigmoid", group_score: str = "top2", normalize: bool = True):
    """From the router's fp32 logits ``z`` [T, experts]: s = sigmoid(z) (``score`` "softmax": softmax over all experts);
    the choice scores are s + ``correction``; the experts form ``groups`` equal groups of neighbours, a group's score is
    the sum of its two largest choice scores (``group_score`` "max": the largest) and only the ``keep`` best groups can be
    chosen from; the ``top`` largest choice scores among those win. Returns the chosen experts (int32 [T, top]) and their
    weights (fp32 [T, top]): s of the chosen / (their sum + 1e-20) * scale, or, not ``normalize``, s * scale."""
    if score not in ("sigmoid", "softmax") or group_score not in ("top2", "max"):
        raise KernelError(f"moe_router: score '{score}' (sigmoid, softmax) with group score '{group_score}' (top2, max)")
    _dev(z, correction)
    _rows2d(z, "router logits")
    if z.dtype != torch.float32:
        raise KernelError("the router's logits are fp32")
    T, E = z.shape
    if correction is not None and (correction.numel() != E or not correction.is_contiguous()):
        raise KernelError(f"the router's correction has {correction.numel()} entries for {E} experts")
    chosen = torch.empty((T, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=z.device)
    if T == 0:
        return chosen, weights
    _call("jllm_moe_router", _ptr(z), z.stride(0), _ptr(correction), _code(correction.dtype) if correction is not None else F32,
          T, E, int(groups), int(keep), int(top), float(scale), _ptr(chosen), _ptr(weights), 1 if score == "softmax" else 0,
          1 if group_score == "max" else 0, 1 if normalize else 0, _stream())
    return chosen, weights


def moe_route(token_ids: Optional[torch.Tensor], table: torch.Tensor, experts: int, many_ok: bool = False) -> MoeRouting:
    """Groups the assignments (row t, k-th expert of its token) by expert, on the device. ``token_ids`` None: row t's
    experts are ``table[t]`` (what a router chose for this step's rows). ``many_ok``: the caller's
    products can go through the tiled matrix-core kernel (bf16, K a multiple of 64): steps that give the experts 64 rows
    or more each on average are then cut into tiles of 128 rows, all others into tiles of 16."""
    _dev(token_ids, table)
    T = token_ids.numel() if token_ids is not None else table.shape[0]
    _i32(token_ids, T, "token ids")
    if table.dtype != torch.int32 or table.dim() != 2 or not table.is_contiguous():
        raise KernelError("the routing table must be a contiguous int32 [vocab, top] tensor")
    top = table.shape[1]
    A = T * top
    tile_rows = MOE_TILE_ROWS_MANY if many_ok and A >= 64 * experts else MOE_TILE_ROWS
    max_tiles = max(1, min(A, A // tile_rows + experts))
    sorted_ = torch.empty((max(A, 1),), dtype=torch.int32, device=table.device)
    place_of = torch.empty((max(A, 1),), dtype=torch.int32, device=table.device)
    tiles = torch.empty((max_tiles, 3), dtype=torch.int32, device=table.device)
    _call("jllm_moe_route", _ptr(token_ids), _ptr(table), T, top, experts, tile_rows, max_tiles, _ptr(sorted_), _ptr(tiles),
          _ptr(place_of), _stream())
    return MoeRouting(sorted_, tiles, place_of, max_tiles, tile_rows, top)


def moe_gemm(a: torch.Tensor, w: torch.Tensor, routing: MoeRouting, *, w2: Optional[torch.Tensor] = None,
             out: torch.Tensor, in_map: int, out_map: int, weight: float = 1.0, gate: int = 0, gate_limit: float = 0.0,
             exact: bool = False) -> torch.Tensor:
    """The grouped product of a routed feed-forward: every tile of ``routing`` multiplies its rows of ``a`` with its
    expert's weights ``w[e]`` ([experts, N, K]); with ``w2`` the gate function is applied to the two sums. ``in_map``
    0 / 1: a tile's input rows are its places in the sorted order / its assignments' token rows; ``out_map`` 0 / 1 / 2:
    output rows by place / by assignment / added, times ``weight``, into the fp32 row of the token (top = 1). With
    tiles of many rows (``routing.many``) the tiled matrix-core kernel takes the product; its output rows go by place."""
    _dev(a, w, w2, out)
    _rows2d(a, "moe input")
    _rows2d(out, "moe output")
    if w.dim() != 3 or not w.is_contiguous() or (w2 is not None and (w2.shape != w.shape or w2.dtype != w.dtype or not w2.is_contiguous())):
        raise KernelError("moe weights must be contiguous [experts, N, K] tensors of one shape and type")
    _, N, K = w.shape
    top = routing.top
    if a.shape[1] != K or out.shape[1] != N:
        raise KernelError(f"moe_gemm: rows of {a.shape[1]} -> {out.shape[1]} with weights {tuple(w.shape)}")
    epilogue = (EPI_GATED | (int(gate) << 8)) if w2 is not None else EPI_STORE
    if routing.many:
        if out_map != 0 or exact or a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
            raise KernelError("moe_gemm: tiles of many rows go through the bf16 tiled kernel and write their rows by place")
        if not _try("jllm_gemm_mfma_grouped_bf16", _ptr(a), a.stride(0), _ptr(w), _ptr(w2), _ptr(out), _code(out.dtype),
                    out.stride(0), routing.sorted.numel(), N, K, epilogue, float(gate_limit), _ptr(routing.tiles),
                    routing.max_tiles, routing.tile_rows, _ptr(routing.sorted) if in_map else None, int(top), _stream()):
            raise KernelError(f"moe_gemm: the tiled kernel does not take N {N}, K {K} (K must be a multiple of 64)")
        return out
    head = (_ptr(a), _code(a.dtype), a.stride(0), _ptr(w), _ptr(w2), _code(w.dtype), _ptr(out), _code(out.dtype),
            out.stride(0), N, K, _ptr(routing.sorted), _ptr(routing.tiles), routing.max_tiles, routing.tile_rows, int(top),
            int(in_map), int(out_map), float(weight), epilogue, float(gate_limit), _stream())
    if not exact and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and _try("jllm_moe_gemm_bf16", *head):
        return out
    if not exact:
        _count("general", "jllm_moe_gemm_generic")
    _call("jllm_moe_gemm_generic", *head)
    return out


def moe_combine(y: torch.Tensor, residual: torch.Tensor, top: int, weight: float, place_of: Optional[torch.Tensor] = None,
                weights: Optional[torch.Tensor] = None, shared: Optional[torch.Tensor] = None,
                shared_gate: Optional[torch.Tensor] = None, overwrite: bool = False) -> None:
    """residual[t] += weight * sum_k y[t * top + k] (fp32 both; k ascending); with ``place_of`` the k-th row of t is
    y[place_of[t * top + k]]; with ``weights`` (fp32 [T, top]) the k-th term is also multiplied by weights[t, k]. With
    ``shared`` (fp32 [T, width] with any row stride, a shared expert's rows) its row t joins the sum, times
    sigmoid(shared_gate[t]) where ``shared_gate`` (fp32 [T], any stride) is given; ``overwrite``: the rows of
    ``residual`` are written instead of added to."""
    _dev(y, residual, place_of, weights, shared, shared_gate)
    if shared is not None and (shared.dtype != torch.float32 or shared.dim() != 2 or shared.stride(1) != 1 or shared.shape != residual.shape):
        raise KernelError("moe_combine: the shared rows must be an fp32 tensor of the residual's shape with contiguous rows")
    if shared_gate is not None and (shared is None or shared_gate.dtype != torch.float32 or shared_gate.dim() != 1
                                    or shared_gate.shape[0] != residual.shape[0]):
        raise KernelError("moe_combine: the shared rows' gate is one fp32 number per row, beside the shared rows")
    T, width = residual.shape
    if y.dtype != torch.float32 or residual.dtype != torch.float32 or not y.is_contiguous() or not residual.is_contiguous() \
            or y.shape != (T * top, width):
        raise KernelError("moe_combine takes contiguous fp32 [T * top, width] rows and the fp32 residual [T, width]")
    _i32(place_of, T * top, "places")
    if weights is not None and (weights.dtype != torch.float32 or not weights.is_contiguous() or weights.numel() != T * top):
        raise KernelError("moe_combine: the weights must be a contiguous fp32 [T, top] tensor")
    _call("jllm_moe_combine", _ptr(y), _ptr(residual), T, width, int(top), float(weight), _ptr(place_of), _ptr(weights),
          _ptr(shared), _ptr(shared_gate), shared_gate.stride(0) if shared_gate is not None else 0, 1 if overwrite else 0,
          shared.stride(0) if shared is not None else 0, _stream())


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
