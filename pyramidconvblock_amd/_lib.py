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
    "pdw_last_error": (c_char_p, []),
    "pdw_conv_out_size": (c_int, [c_int] * 5),
    "pdw_dwconv_fwd": (c_int, [c_void_p] * 3 + _CONV + [c_int, c_void_p]),
    "pdw_dwconv_fwd_pool": (c_int, [c_void_p] * 4 + _CONV + [c_int, c_int, c_int, c_void_p]),
    "pdw_dwconv_fwd_gate": (c_int, [c_void_p] * 4 + [c_int] * 9 + [c_void_p]),
    "pdw_dwconv_dgrad": (c_int, [c_void_p] * 3 + _CONV + [c_int, c_void_p]),
    "pdw_reduce_defer_begin": (c_int, []),
    "pdw_reduce_defer_flush": (c_int, [c_void_p]),
    "pdw_dwconv_dgrad_addpool": (c_int, [c_void_p] * 4 + _CONV + [c_int, c_int, c_int, c_void_p]),
    "pdw_dwconv_wgrad_workspace_bytes": (c_size_t, _CONV + [c_int]),
    "pdw_dwconv_wgrad": (c_int, [c_void_p] * 4 + [c_size_t] + _CONV + [c_int, c_void_p]),
    "pdw_static_scratch_bytes": (c_size_t, []),
    "pdw_static_scratch_init": (c_int, []),
    "pdw_dwconv_wgrad_static": (c_int, [c_void_p] * 3 + _CONV + [c_int, c_void_p]),
    "pdw_dwconv_wgrad_pair": (c_int, ([c_void_p] * 4 + [c_size_t] + [c_int] * 2) * 2 + [c_int] * 4 + [c_void_p]),
    "pdw_convblock_supported": (c_int, [c_int] * 7),
    "pdw_convblock_fwd_workspace_bytes": (c_size_t, [c_int] * 7),
    "pdw_convblock_fwd": (c_int, [c_void_p] * 16 + [c_size_t] + [c_int] * 7 + [c_void_p]),
    "pdw_convblock_infer_workspace_bytes": (c_size_t, [c_int] * 7),
    "pdw_convblock_infer": (c_int, [c_void_p] * 10 + [c_size_t] + [c_int] * 7 + [c_void_p]),
    "pdw_convblock_bwd_workspace_bytes": (c_size_t, [c_int] * 7),
    "pdw_convblock_bwd": (c_int, [c_void_p] * 22 + [c_size_t] + [c_int] * 7 + [c_void_p]),
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
    "pdw_block_mid_infer": (c_int, [c_void_p] * 2 + [c_int] * 7 + [c_void_p, c_int] + [c_void_p] * 5 + [c_int] * 3
                            + [c_void_p]),
    "pdw_block_mid_fwd": (c_int, [c_void_p] * 3 + [c_int] * 7 + [c_void_p, c_int] + [c_void_p] * 5 + [c_int] * 3
                          + [c_void_p]),
    "pdw_block_mid_bwd": (c_int, [c_void_p] * 5 + [c_int] * 7 + [c_void_p, c_int] + [c_void_p] * 7 + [c_size_t]
                          + [c_int] * 3 + [c_void_p]),
    "pdw_pool_branch_bwd": (c_int, [c_void_p] * 8 + [c_size_t] + [c_int] * 4 + [c_void_p]),
    "pdw_sum_parts": (c_int, [c_void_p, c_void_p, c_int, c_longlong, c_int, c_void_p]),
    "pdw_dense_fwd_colsum_pool": (c_int, [c_void_p] * 6 + [c_int] * 6 + [c_void_p]),
    "pdw_dwconv_fwd2_supported": (c_int, [c_int] * 6),
    "pdw_dwconv_fwd2": (c_int, [c_void_p] * 6 + [c_int] * 6 + [c_void_p]),
    "pdw_dwconv_fwd2_mean": (c_int, [c_void_p] * 3 + [c_int] * 2 + [c_void_p] * 3 + [c_int] * 7 + [c_void_p, c_int]
                             + [c_void_p] * 5 + [c_int] * 3 + [c_void_p]),
    "pdw_dense_fwd_gated_supported": (c_int, [c_int] * 5),
    "pdw_dense_fwd_gated": (c_int, [c_void_p] * 7 + [c_int] * 7 + [c_void_p]),
    "pdw_dwconv_fwd2_gate": (c_int, [c_void_p] * 3 + [c_int] * 2 + [c_void_p] * 3 + [c_int] * 2 + [c_int] * 6 + [c_void_p]),
    "pdw_dwconv_bwd3_plan": (c_int, [c_int] * 6 + [c_void_p]),
    "pdw_dwconv_bwd3": (c_int, [c_void_p] * 7 + [c_size_t] + [c_void_p] * 4 + [c_size_t] + [c_int] * 6 + [c_void_p]),
    "pdw_dense_supported": (c_int, [c_int] * 3),
    "pdw_dense_fwd": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong] + [c_int] * 4
                      + [c_void_p]),
    "pdw_dense_fwd_flush": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong] + [c_int] * 4
                      + [c_void_p]),
    "pdw_dense_wgrad_workspace_bytes": (c_size_t, [c_longlong, c_int, c_int]),
    "pdw_dense_wgrad": (c_int, [c_void_p] * 4 + [c_size_t, c_longlong, c_int, c_int, c_int, c_void_p]),
    "pdw_dense_bwd_pair_supported": (c_int, [c_int] * 3),
    "pdw_dense_bwd_pair_colsum_supported": (c_int, [c_int] * 3),
    "pdw_dense_bwd_pair": (c_int, [c_void_p] * 7 + [c_size_t, c_void_p, c_int, c_longlong, c_int, c_int, c_int,
                                   c_void_p]),
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


_scope = threading.local()


def stream_ptr(dev: torch.device) -> int:
    held = getattr(_scope, "held", None)
    if held is not None and held[0] == dev:
        return held[1]
    return torch.cuda.current_stream(dev).cuda_stream


class on_device:
    """Makes `dev` the current HIP device for the duration of a launch (no-op when it already is)."""

    def __init__(self, dev: torch.device):
        self.dev, self.prev = dev, None

    def __enter__(self):
        held = getattr(_scope, "held", None)
        if held is not None and held[0] == self.dev:
            return self  # launch_scope made it current
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


class launch_scope:
    """A run of launches on one device from one host thread (an autograd node's forward or backward): `dev` is made
    current and its current stream looked up once instead of per launch.  The stream must not be switched inside."""

    def __init__(self, dev: torch.device):
        self.dev = dev
        self.guard = on_device(dev)
        self.outer = None

    def __enter__(self):
        self.outer = getattr(_scope, "held", None)
        _scope.held = None
        self.guard.__enter__()
        _scope.held = (self.dev, torch.cuda.current_stream(self.dev).cuda_stream)
        return self

    def __exit__(self, *exc):
        _scope.held = None
        self.guard.__exit__(*exc)
        _scope.held = self.outer
        return False


_defer = threading.local()


class deferred_reductions:
    """Within the block the final summation kernels of the weight-gradient calls are recorded and then run in one
    launch on `dev`'s current stream at exit; their results must not be read (or converted) before that."""

    def __init__(self, dev: torch.device):
        self.dev = dev

    def __enter__(self):
        check(lib().pdw_reduce_defer_begin(), "pdw_reduce_defer_begin")
        _defer.keep = []
        return self

    def __exit__(self, *exc):
        try:
            with on_device(self.dev):
                check(lib().pdw_reduce_defer_flush(stream_ptr(self.dev)), "pdw_reduce_defer_flush")
        finally:
            _defer.keep = None
        return False


def keep_until_flush(t: torch.Tensor) -> None:
    """A workspace whose contents a deferred reduction still has to read stays referenced until the flush."""
    keep = getattr(_defer, "keep", None)
    if keep is not None:
        keep.append(t)
