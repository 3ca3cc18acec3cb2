"""ctypes binding of libpdw.so, the C-ABI library of hand-written gfx950 kernels.

There is deliberately no fallback: if the library is missing and cannot be built, or a
tensor is not on a HIP device, the operators raise.
"""
from __future__ import annotations

import ctypes
import threading
import os
from ctypes import c_char_p, c_int, c_longlong, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpdw.so")

PDW_F32, PDW_F16, PDW_BF16 = 0, 1, 2
_DTYPES = {torch.float32: PDW_F32, torch.float16: PDW_F16, torch.bfloat16: PDW_BF16}

_lib = None

_CONV = [c_int] * 12  # B,H,W,C,KH,KW,SH,SW,PH,PW,DH,DW
_SIGS = {
    "pdw_version": (c_int, []),
    "pdw_launch_count": (ctypes.c_ulonglong, []),
    "pdw_last_error": (c_char_p, []),
    "pdw_conv_out_size": (c_int, [c_int] * 5),
    "pdw_dwconv_fwd": (c_int, [c_void_p] * 3 + _CONV + [c_int, c_void_p]),
    "pdw_dwconv_fwd_pool": (c_int, [c_void_p] * 4 + _CONV + [c_int, c_int, c_int, c_void_p]),
    "pdw_dwconv_dgrad": (c_int, [c_void_p] * 3 + _CONV + [c_int, c_void_p]),
    "pdw_reduce_defer_begin": (c_int, []),
    "pdw_reduce_defer_flush": (c_int, [c_void_p]),
    "pdw_dwconv_dgrad_addpool": (c_int, [c_void_p] * 4 + _CONV + [c_int, c_int, c_int, c_void_p]),
    "pdw_dwconv_wgrad_workspace_bytes": (c_size_t, _CONV + [c_int]),
    "pdw_dwconv_wgrad": (c_int, [c_void_p] * 4 + [c_size_t] + _CONV + [c_int, c_void_p]),
    "pdw_avgpool_fwd": (c_int, [c_void_p] * 2 + [c_int] * 7 + [c_void_p]),
    "pdw_avgpool_bwd": (c_int, [c_void_p] * 2 + [c_int] * 8 + [c_void_p]),
    "pdw_bilinear_fwd": (c_int, [c_void_p] * 2 + [c_int] * 8 + [c_void_p]),
    "pdw_bilinear_bwd": (c_int, [c_void_p] * 2 + [c_int] * 8 + [c_void_p]),
    "pdw_gate_fwd": (c_int, [c_void_p] * 2 + [c_longlong, c_int, c_int, c_int, c_void_p]),
    "pdw_gate_bwd": (c_int, [c_void_p] * 3 + [c_longlong, c_int, c_int, c_int, c_void_p]),
    "pdw_gate_pair_fwd": (c_int, [c_void_p] * 3 + [c_int] * 8 + [c_void_p]),
    "pdw_gate_pair_bwd": (c_int, [c_void_p] * 5 + [c_int] * 8 + [c_void_p]),
    "pdw_gate_bilinear_fwd": (c_int, [c_void_p] * 2 + [c_int] * 8 + [c_void_p]),
    "pdw_bilinear_gate_bwd": (c_int, [c_void_p] * 3 + [c_int] * 8 + [c_void_p]),
    "pdw_spatial_sum_workspace_bytes": (c_size_t, [c_int] * 3),
    "pdw_spatial_sum": (c_int, [c_void_p] * 3 + [c_size_t] + [c_int] * 4 + [c_void_p]),
    "pdw_add_rowbias": (c_int, [c_void_p] * 2 + [c_int] * 4 + [c_void_p]),
    "pdw_pool_branch_workspace_bytes": (c_size_t, [c_int] * 3),
    "pdw_pool_branch_fwd": (c_int, [c_void_p] * 7 + [c_size_t] + [c_int] * 4 + [c_void_p]),
    "pdw_pool_branch_fwd_parts": (c_int, [c_void_p, c_int] + [c_void_p] * 5 + [c_int] * 4 + [c_void_p]),
    "pdw_pool_branch_bwd_parts": (c_int, [c_void_p, c_int] + [c_void_p] * 7 + [c_size_t] + [c_int] * 4 + [c_void_p]),
    "pdw_dense_colsum_supported": (c_int, [c_int] * 3),
    "pdw_dense_colsum_rows": (c_int, []),
    "pdw_dense_fwd_colsum": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_longlong]
                             + [c_int] * 4 + [c_void_p]),
    "pdw_block_mid_fwd": (c_int, [c_void_p] * 3 + [c_int] * 7 + [c_void_p, c_int] + [c_void_p] * 5 + [c_int] * 3
                          + [c_void_p]),
    "pdw_block_mid_bwd": (c_int, [c_void_p] * 5 + [c_int] * 7 + [c_void_p, c_int] + [c_void_p] * 7 + [c_size_t]
                          + [c_int] * 3 + [c_void_p]),
    "pdw_pool_branch_bwd": (c_int, [c_void_p] * 8 + [c_size_t] + [c_int] * 4 + [c_void_p]),
    "pdw_dense_supported": (c_int, [c_int] * 3),
    "pdw_dense_fwd": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong] + [c_int] * 4
                      + [c_void_p]),
    "pdw_dense_fwd_flush": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong] + [c_int] * 4
                      + [c_void_p]),
    "pdw_dense_wgrad_workspace_bytes": (c_size_t, [c_longlong, c_int, c_int]),
    "pdw_dense_wgrad": (c_int, [c_void_p] * 4 + [c_size_t, c_longlong, c_int, c_int, c_int, c_void_p]),
}
EXPORTS = tuple(_SIGS)


def lib():
    """Loads libpdw.so (building it with hipcc only if it has never been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            from . import build as _build

            _build.build()
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(status: int, what: str = "libpdw") -> None:
    if status != 0:
        raise RuntimeError(f"{what}: {lib().pdw_last_error().decode()} (status {status})")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"pyramid dwconv kernels support float32/float16/bfloat16, got {dtype}") from None


def require_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError("pyramid dwconv kernels run on a HIP device only (tensor is on %s); "
                               "there is no CPU path" % t.device)
        if t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} vs {t.device}")
    return dev


def stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


class on_device:
    """Makes `dev` the current HIP device for the duration of a launch (no-op when it already is)."""

    def __init__(self, dev: torch.device):
        self.dev, self.prev = dev, None

    def __enter__(self):
        idx = self.dev.index if self.dev.index is not None else torch.cuda.current_device()
        cur = torch.cuda.current_device()
        if idx != cur:
            self.prev = cur
            torch.cuda.set_device(idx)
        return self

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


class _Recorder:  # process-wide: a backward pass makes its calls on the autograd engine's thread
    calls = None
    lock = threading.Lock()


_rec = _Recorder


def call(name: str, dev: torch.device, *args) -> None:
    """One stream-ordered entry point of the library: fn(*args, stream of `dev`), an error status raised as
    RuntimeError.  While a `recorded_calls` block is open on this thread the call is also noted down."""
    fn = getattr(lib(), name)
    with on_device(dev):
        check(fn(*args, stream_ptr(dev)), name)
    calls = _rec.calls
    if calls is not None:
        with _rec.lock:
            calls.append((fn, args, True, name))


class recorded_calls:
    """Collects the library calls made inside the block, by any thread, as (function, arguments, takes_stream,
    name), in order, for `replay_calls`.  The arguments are the raw pointers and extents of the calls: they stay
    meaningful only while the tensors behind them are alive and in place (as in a captured graph's memory pool).
    Nothing else may use the library while the block is open."""

    def __enter__(self):
        with _rec.lock:
            if _rec.calls is not None:
                raise RuntimeError("recorded_calls: already recording")
            _rec.calls = self.calls = []
        self.first_launch = lib().pdw_launch_count()
        return self

    def __exit__(self, *exc):
        _rec.calls = None
        self.kernels = lib().pdw_launch_count() - self.first_launch
        return False


def replay_calls(calls, dev: torch.device) -> None:
    """Issues recorded calls again, on `dev`'s current stream."""
    with on_device(dev):
        st = stream_ptr(dev)
        for fn, args, takes_stream, name in calls:
            status = fn(*args, st) if takes_stream else fn(*args)
            if status:
                check(status, name)


_defer = threading.local()


class deferred_reductions:
    """Within the block the final summation kernels of the weight-gradient calls are recorded and then run in one
    launch on `dev`'s current stream at exit; their results must not be read (or converted) before that."""

    def __init__(self, dev: torch.device):
        self.dev = dev

    def __enter__(self):
        check(lib().pdw_reduce_defer_begin(), "pdw_reduce_defer_begin")
        calls = _rec.calls
        if calls is not None:
            with _rec.lock:
                calls.append((lib().pdw_reduce_defer_begin, (), False, "pdw_reduce_defer_begin"))
        _defer.keep = []
        return self

    def __exit__(self, *exc):
        try:
            call("pdw_reduce_defer_flush", self.dev)
        finally:
            _defer.keep = None
        return False


def keep_until_flush(t: torch.Tensor) -> None:
    """A workspace whose contents a deferred reduction still has to read stays referenced until the flush."""
    keep = getattr(_defer, "keep", None)
    if keep is not None:
        keep.append(t)
