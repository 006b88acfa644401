"""Host layer: binds libflashcolsum.so (C ABI, include/flash_colsum.h) with ctypes.

PyTorch supplies device memory and the HIP stream; every byte of arithmetic happens in
the hand-written gfx950 kernels behind the C ABI.  There is no fallback: if the shared
library is missing or a launch fails this module raises.

The three private launchers keep the names and argument meaning of the reference's
(reference: flash_colsum/kernel_noncausal_batched.py:102, kernel_noncausal.py:95,
kernel_causal.py:94) and, like them, return fp16; the `*_f32` functions return the
kernels' fp32 means.
"""
import collections
import ctypes
import os
import threading
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libflashcolsum.so")
_ABI_VERSION = 5
_lib = None

_I64x4 = ctypes.c_int64 * 4
_MAX_HEAD_DIM = 256  # the library takes any multiple of 8 up to this


class _Call(ctypes.Structure):
    """fcs_call_t of include/flash_colsum.h: one call as a struct, filled once per tensor geometry."""
    _fields_ = [
        ("struct_bytes", ctypes.c_uint32), ("flags", ctypes.c_uint32),
        ("dtype", ctypes.c_int32), ("causal", ctypes.c_int32),
        ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("Hk", ctypes.c_int32),
        ("Sq", ctypes.c_int32), ("Sk", ctypes.c_int32), ("D", ctypes.c_int32),
        ("cls_n", ctypes.c_int32), ("k_past", ctypes.c_int32),
        ("scale", ctypes.c_float), ("reserved", ctypes.c_int32),
        ("q_strides", _I64x4), ("k_strides", _I64x4),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("out", ctypes.c_void_p), ("out_f16", ctypes.c_void_p),
        ("ws", ctypes.c_void_p), ("ws_bytes", ctypes.c_size_t), ("hip_stream", ctypes.c_void_p),
    ]


def lib() -> ctypes.CDLL:
    """Load the shared library once; raise loudly when it is absent or of another ABI."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} not found: build it with `make -C flash-colsum_amd` "
                "(hipcc, --offload-arch=gfx950). There is no fallback path."
            )
        cdll = ctypes.CDLL(_LIB_PATH)
        cdll.fcs_abi_version.restype = ctypes.c_int
        cdll.fcs_abi_version.argtypes = []
        cdll.fcs_strerror.restype = ctypes.c_char_p
        cdll.fcs_strerror.argtypes = [ctypes.c_int]
        cdll.fcs_workspace_bytes.restype = ctypes.c_size_t
        cdll.fcs_workspace_bytes.argtypes = [ctypes.c_int] * 7
        for fn in (cdll.fcs_colsum_noncausal_f16, cdll.fcs_colsum_noncausal_bf16):
            fn.restype = ctypes.c_int
            fn.argtypes = [
                ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                ctypes.c_float, ctypes.c_int, ctypes.c_void_p]
        cdll.fcs_colsum_noncausal_f16_static.restype = ctypes.c_int
        cdll.fcs_colsum_noncausal_f16_static.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
            ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
            ctypes.c_float, ctypes.c_int, ctypes.c_void_p]
        for fn in (cdll.fcs_colsum_causal_f16, cdll.fcs_colsum_causal_bf16):
            fn.restype = ctypes.c_int
            fn.argtypes = [
                ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                ctypes.c_float, ctypes.c_void_p]
        cdll.fcs_colsum_general.restype = ctypes.c_int
        cdll.fcs_colsum_general.argtypes = [
            ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_void_p, ctypes.c_size_t] + [ctypes.c_int] * 8 + [
            ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64), ctypes.c_float, ctypes.c_void_p]
        cdll.fcs_colsum_call.restype = ctypes.c_int
        cdll.fcs_colsum_call.argtypes = [ctypes.POINTER(_Call)]
        cdll.fcs_plan_describe.restype = ctypes.c_size_t
        cdll.fcs_plan_describe.argtypes = [ctypes.POINTER(_Call), ctypes.c_char_p, ctypes.c_size_t]
        cdll.fcs_static_scratch_init.restype = ctypes.c_int
        cdll.fcs_static_scratch_init.argtypes = []
        cdll.fcs_topk_f32.restype = ctypes.c_int
        cdll.fcs_topk_f32.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        cdll.fcs_threshold_f32.restype = ctypes.c_int
        cdll.fcs_threshold_f32.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p]
        got = cdll.fcs_abi_version()
        if got != _ABI_VERSION:
            raise RuntimeError(f"libflashcolsum.so has ABI {got}, this host layer needs {_ABI_VERSION}")
        _lib = cdll
    return _lib


def strerror(code: int) -> str:
    return lib().fcs_strerror(int(code)).decode()


def _check(code: int, what: str) -> None:
    if code != 0:
        raise RuntimeError(f"{what} failed with code {code}: {strerror(code)}")


def _as_kernel_input(t: torch.Tensor, dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """`dtype` (fp16 or bf16), unit last stride, 16-byte aligned rows/heads/base; copies only when it must."""
    if t.dtype != dtype:
        t = t.to(dtype)
    if t.is_contiguous() and t.shape[-1] % 8 == 0 and t.data_ptr() % 16 == 0 and t.shape[1] > 1 and t.shape[2] > 1:
        # the common case, decided without looking at the strides one by one (a dimension of size 1 may carry
        # any stride and still count as contiguous: those tensors take the checks below)
        return t
    ok = (
        t.stride(3) == 1
        and t.stride(2) % 8 == 0
        and t.stride(1) % 8 == 0
        and (t.shape[0] == 1 or t.stride(0) % 8 == 0)
        and t.data_ptr() % 16 == 0
    )
    if ok:
        return t
    if not t.is_contiguous():
        t = t.contiguous()
    elif t.data_ptr() % 16:
        t = t.clone()
    # contiguous now, but the stride of a size-1 dimension may still be anything: the same memory under the
    # dense strides
    b, h, s_, d = t.shape
    return t.as_strided(t.shape, (h * s_ * d, s_ * d, d, 1))


_ws_bytes_cache = {}


def workspace_bytes(causal: bool, b: int, h: int, s_q: int, s_k: int, d: int, cls_n: int = -1) -> int:
    key = (bool(causal), b, h, s_q, s_k, d, cls_n)
    n = _ws_bytes_cache.get(key)
    if n is None:
        n = int(lib().fcs_workspace_bytes(int(causal), b, h, s_q, s_k, d, cls_n))
        if len(_ws_bytes_cache) < 4096:
            _ws_bytes_cache[key] = n
    return n


# One workspace per (thread, device, stream), grown on demand and reused by later calls: calls on one
# stream execute in order, so the next call may overwrite what the previous one left behind; threads
# do not share workspaces, so calls that two threads enqueue on one stream cannot meet in one either.
# A thread keeps at most _WS_MAX_ENTRIES streams (least recently used goes first) and nothing
# above _WS_MAX_CACHED_BYTES: larger workspaces are allocated per call and returned to torch's
# allocator afterwards.  While a stream is capturing a HIP graph the cache is neither read nor
# filled: the workspace then comes from the graph's own pool and lives as long as the graph.
_tls = threading.local()
_WS_MIN_BYTES = 1 << 20
_WS_MAX_CACHED_BYTES = 64 << 20
_WS_MAX_ENTRIES = 16
_CALLS_MAX_ENTRIES = 256


def _workspace(device: torch.device, stream: int, n_bytes: int) -> torch.Tensor:
    if n_bytes > _WS_MAX_CACHED_BYTES or torch.cuda.is_current_stream_capturing():
        return torch.empty((max(n_bytes, 256),), dtype=torch.uint8, device=device)
    cache = getattr(_tls, "workspaces", None)
    if cache is None:
        cache = _tls.workspaces = collections.OrderedDict()
    key = (device.index, stream)
    ws = cache.get(key)
    if ws is None or ws.numel() < n_bytes:
        ws = torch.empty((max(n_bytes, _WS_MIN_BYTES),), dtype=torch.uint8, device=device)
        cache[key] = ws
        while len(cache) > _WS_MAX_ENTRIES:
            cache.popitem(last=False)
    elif len(cache) > 1:
        cache.move_to_end(key)
    return ws


def release_workspaces() -> None:
    """Drop the calling thread's cached per-stream workspaces (they are otherwise kept until the thread ends).

    Kernels already enqueued keep running on the memory they were given; torch's allocator
    reuses it for later allocations on the same stream in stream order."""
    cache = getattr(_tls, "workspaces", None)
    if cache is not None:
        cache.clear()


# the raw handle of the current stream without building a torch.cuda.Stream object (absent from some builds)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(dev: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


def _prepared_call(causal, q, k, scale, cls_n, k_past):
    """The calling thread's fcs_call_t for this tensor geometry (shape, strides, dtype and the scalar
    arguments filled in; pointers are set per call) and the workspace bytes it needs."""
    calls = getattr(_tls, "calls", None)
    if calls is None:
        calls = _tls.calls = {}
    key = (q.shape, k.shape, q.stride(), k.stride(), q.dtype, causal, cls_n, k_past, scale)
    ent = calls.get(key)
    if ent is None:
        b, h, s_q, d = q.shape
        c = _Call()
        c.struct_bytes = ctypes.sizeof(_Call)
        c.dtype = 1 if q.dtype == torch.bfloat16 else 0
        c.causal = int(causal)
        c.B, c.Hq, c.Hk, c.Sq, c.Sk, c.D = b, h, k.shape[1], s_q, k.shape[2], d
        c.cls_n, c.k_past, c.scale = int(cls_n), int(k_past), scale
        c.q_strides, c.k_strides = _I64x4(*q.stride()), _I64x4(*k.stride())
        ent = (c, ctypes.byref(c), workspace_bytes(causal, b, h, s_q, k.shape[2], d, cls_n))
        if len(calls) >= _CALLS_MAX_ENTRIES:
            calls.clear()
        calls[key] = ent
    return ent


def _enqueue(causal, q, k, scale, cls_n, k_past, want_f16, f16_only=False):
    c, c_ref, n_ws = _prepared_call(causal, q, k, scale, cls_n, k_past)
    b, s_k = c.B, c.Sk
    dev = q.device
    stream = _current_stream(dev)
    if f16_only:
        # the caller only wants the fp16 result: the kernels' fp32 means go to the tail of the workspace
        # instead of a tensor of their own (one allocation less per call)
        ws = _workspace(dev, stream, n_ws + 4 * b * s_k)
        ws_ptr = ws.data_ptr()
        out, out_ptr = None, ws_ptr + n_ws
    else:
        out = torch.empty((b, s_k), dtype=torch.float32, device=dev)
        ws = _workspace(dev, stream, n_ws)
        ws_ptr, out_ptr = ws.data_ptr(), out.data_ptr()
    out_h = torch.empty((b, s_k), dtype=torch.float16, device=dev) if want_f16 else None
    c.q, c.k, c.out, c.out_f16 = q.data_ptr(), k.data_ptr(), out_ptr, (out_h.data_ptr() if want_f16 else None)
    c.ws, c.ws_bytes, c.hip_stream = ws_ptr, n_ws, stream
    rc = (_lib or lib()).fcs_colsum_call(c_ref)
    if rc != 0:
        _check(rc, "fcs_colsum_call")
    if f16_only:
        return out_h
    return (out, out_h) if want_f16 else out


_FP16_MAX = 65504.0


def _wide_operands(q: torch.Tensor, k: torch.Tensor):
    """fp32 / fp64 operands.  The kernels' operand types are fp16 and bf16; the reference's kernels upcast whatever
    they are given (reference: flash_colsum/kernel_noncausal_batched.py:30-37,47-54, kernel_causal.py:26-32).
    Values inside fp16's range are rounded to fp16 (the mantissa of the reference's TF32 products).  Larger ones
    would become inf there: they run on the bf16 kernels instead, each operand split into a high and a low bf16
    part (16 mantissa bits together) laid side by side along the head dim, Q as [hi, hi, lo, lo] and K as
    [hi, lo, hi, lo], so that one dot product over 4 D channels adds up all four partial products.  That needs
    4 D <= 256; wider heads raise.  The range test reads one number back from the GPU; while a stream is
    capturing a graph it is skipped and the operands are rounded to fp16 unseen."""
    if torch.cuda.is_current_stream_capturing():
        return q.to(torch.float16), k.to(torch.float16), torch.float16
    amax = max(float(t.detach().abs().max()) if t.dtype not in (torch.float16, torch.bfloat16) else 0.0 for t in (q, k))
    if amax <= _FP16_MAX:  # (a NaN or an infinity fails this test too)
        return q.to(torch.float16), k.to(torch.float16), torch.float16
    if amax != amax or amax == float("inf"):
        raise ValueError("query / key hold NaN or infinite values")
    d = q.shape[-1]
    if 4 * d > _MAX_HEAD_DIM or d != k.shape[-1]:
        raise ValueError(
            f"query / key values reach {amax:.6g}, beyond fp16's range (+-{_FP16_MAX:g}); with head_dim {d} > "
            f"{_MAX_HEAD_DIM // 4} they cannot be split into bf16 parts either: pass bfloat16 tensors (same range "
            "as fp32, 8 mantissa bits) or rescale the operands and `scale`")

    def split(t):
        t = t.float()
        hi = t.bfloat16()
        return hi, (t - hi.float()).bfloat16()

    q_hi, q_lo = split(q)
    k_hi, k_lo = split(k)
    return torch.cat([q_hi, q_hi, q_lo, q_lo], dim=-1), torch.cat([k_hi, k_lo, k_hi, k_lo], dim=-1), torch.bfloat16


def _launch(causal: bool, q: torch.Tensor, k: torch.Tensor, scale: float, cls_n: int, k_past: int, want_f16: bool = False,
            f16_only: bool = False):
    """Enqueue one call; returns the fp32 means, (fp32, fp16) when `want_f16`, or the fp16 tensor alone
    when `f16_only` (which implies `want_f16`)."""
    want_f16 = want_f16 or f16_only
    if q.device.type != "cuda" or k.device != q.device:
        raise ValueError(f"query and key must live on the same GPU, got {q.device} and {k.device}")
    # fp16 and bf16 run natively (a mix of the two as fp16); wider types are rounded or split
    half = (torch.float16, torch.bfloat16)
    if q.dtype in half and k.dtype in half:
        dtype = torch.bfloat16 if (q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16) else torch.float16
    else:
        q, k, dtype = _wide_operands(q, k)
    # The library takes head dims that are a multiple of 8 (16-byte rows) up to 256 as they are.  Only a
    # head dim that is not a multiple of 8 is padded with zero channels to the next one (a copy), which
    # leaves every score unchanged; the caller's scale already reflects the real D.
    d = q.shape[-1]
    if d % 8 and d < _MAX_HEAD_DIM and d == k.shape[-1]:
        pad = 8 - d % 8
        q = torch.nn.functional.pad(q.to(dtype), (0, pad))
        k = torch.nn.functional.pad(k.to(dtype), (0, pad))
    q = _as_kernel_input(q, dtype)
    k = _as_kernel_input(k, dtype)
    # any k_past >= K_len means "no mask"; keep it inside the C int the library takes
    k_past = min(int(k_past), k.shape[2])
    if q.device.index == torch.cuda.current_device():
        return _enqueue(causal, q, k, float(scale), cls_n, k_past, want_f16, f16_only)
    with torch.cuda.device(q.device):
        return _enqueue(causal, q, k, float(scale), cls_n, k_past, want_f16, f16_only)


def plan_description(q_shape, k_shape, causal=False, cls_n=-1, k_past=None, scale=None, bf16=False) -> str:
    """Text of the launch plan (kernels, template arguments, grids) a call of these dense shapes gets."""
    b, h, s_q, d = q_shape
    c = _Call()
    c.struct_bytes = ctypes.sizeof(_Call)
    c.dtype, c.causal = int(bf16), int(causal)
    c.B, c.Hq, c.Hk, c.Sq, c.Sk, c.D = b, h, k_shape[1], s_q, k_shape[2], d
    c.cls_n = -1 if cls_n is None or cls_n < 0 else int(cls_n)
    c.k_past = (max(0, k_shape[2] - s_q) if k_past is None else min(int(k_past), k_shape[2])) if causal else 0
    c.scale = float(d ** -0.5 if scale is None else scale)
    c.q_strides = _I64x4(h * s_q * d, s_q * d, d, 1)
    c.k_strides = _I64x4(k_shape[1] * k_shape[2] * d, k_shape[2] * d, d, 1)
    buf = ctypes.create_string_buffer(1024)
    lib().fcs_plan_describe(ctypes.byref(c), buf, len(buf))
    return buf.value.decode()


def colsum_general(Q: torch.Tensor, K: torch.Tensor, scale: float, causal: bool = False, CLS_N: int = -1,
                   K_past: Optional[int] = None, want_f16: bool = False):
    """fcs_colsum_call in its general form: (B, S_k) fp32 means (or (fp32, fp16)) for grouped key heads,
    batched causal calls, causal calls restricted to the first CLS_N rows and non-causal calls with S_q != S_k."""
    if K_past is None:
        K_past = max(0, K.shape[2] - Q.shape[2]) if causal else 0
    return _launch(bool(causal), Q, K, scale, -1 if CLS_N is None or CLS_N < 0 else int(CLS_N), int(K_past) if causal else 0,
                   want_f16)


def colsum_noncausal_f32(Q: torch.Tensor, K: torch.Tensor, scale: float, CLS_N: int = -1) -> torch.Tensor:
    """(B, S) fp32 means over heads and the first min(CLS_N, S) rows (all rows if CLS_N < 0)."""
    return _launch(False, Q, K, scale, -1 if CLS_N is None or CLS_N < 0 else int(CLS_N), 0)


def colsum_causal_f32(Q: torch.Tensor, K: torch.Tensor, scale: float, K_past: Optional[int] = None) -> torch.Tensor:
    """(1, K_len) fp32 means; K_past defaults to max(0, K_len - Q_len) (reference: kernel_causal.py:113)."""
    if K_past is None:
        K_past = max(0, K.shape[2] - Q.shape[2])
    return _launch(True, Q, K, scale, -1, int(K_past))


def _flash_colsum_batched(Q, K, scale, CLS_N=-1):
    """(B, S) fp16, like the reference launcher; the rounding happens in the final kernel."""
    return _launch(False, Q, K, scale, -1 if CLS_N is None or CLS_N < 0 else int(CLS_N), 0, f16_only=True)


def _flash_colsum_non_batched(Q, K, scale, CLS_N=-1):
    """(1, S) fp16; the same kernels serve B = 1 and B > 1."""
    return _flash_colsum_batched(Q, K, scale, CLS_N)


def _flash_colsum_causal(Q, K, scale, K_past=None):
    """(1, K_len) fp16; K_past defaults to max(0, K_len - Q_len)."""
    if K_past is None:
        K_past = max(0, K.shape[2] - Q.shape[2])
    return _launch(True, Q, K, scale, -1, int(K_past), f16_only=True)


TOPK_SORT_MAX = 4096  # FCS_TOPK_SORT_MAX of include/flash_colsum.h


def topk_f32(means: torch.Tensor, k: int, sorted: bool = True):
    """(values fp32 (B,k), indices int64 (B,k)) of the k largest entries of every row of the fp32 (B,S)
    means, selected on the GPU on the current stream.  Ties at the k-th value go to the lower index."""
    if means.dtype != torch.float32 or means.ndim != 2 or means.device.type != "cuda":
        raise ValueError("means must be a 2-D fp32 GPU tensor")
    means = means.contiguous()
    b, s = means.shape
    idx = torch.empty((b, k), dtype=torch.int64, device=means.device)
    val = torch.empty((b, k), dtype=torch.float32, device=means.device)
    in_kernel_sort = sorted and k <= TOPK_SORT_MAX
    with torch.cuda.device(means.device):
        stream = _current_stream(means.device)
        _check(lib().fcs_topk_f32(means.data_ptr(), b, s, int(k), idx.data_ptr(), val.data_ptr(), int(in_kernel_sort), stream),
               "fcs_topk_f32")
    if sorted and not in_kernel_sort:
        # beyond the in-kernel sorting network: a stable sort of the (already index-ordered) selection
        order = torch.sort(val, dim=1, descending=True, stable=True).indices
        val, idx = val.gather(1, order), idx.gather(1, order)
    return val, idx


def threshold_f32(means: torch.Tensor, tau: float):
    """(indices int64 (B,S), counts int32 (B)): row b lists, ascending, the positions whose mean is >= tau
    in its first counts[b] entries."""
    if means.dtype != torch.float32 or means.ndim != 2 or means.device.type != "cuda":
        raise ValueError("means must be a 2-D fp32 GPU tensor")
    means = means.contiguous()
    b, s = means.shape
    idx = torch.empty((b, s), dtype=torch.int64, device=means.device)
    cnt = torch.empty((b,), dtype=torch.int32, device=means.device)
    with torch.cuda.device(means.device):
        stream = _current_stream(means.device)
        _check(lib().fcs_threshold_f32(means.data_ptr(), b, s, float(tau), idx.data_ptr(), cnt.data_ptr(), stream),
               "fcs_threshold_f32")
    return idx, cnt
