"""ctypes binding of libftadam.so -- the only way Python reaches the HIP kernels.

There is no Python or CPU fallback: if the library has not been built, or a call fails, an
exception is raised. Signatures mirror ``include/ft_adam.h`` one to one.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_uint64, c_void_p

import torch

F32, F16, BF16 = 0, 1, 2

DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libftadam.so")

class AdamSegment(ctypes.Structure):
    """Mirror of ``ft_adam_segment_t``: one contiguous piece of an in-place update."""

    _fields_ = [
        ("p", c_void_p), ("g", c_void_p), ("m", c_void_p), ("v", c_void_p), ("half_out", c_void_p),
        ("n", c_size_t), ("step", c_uint64),
        ("lr", c_float), ("beta1", c_float), ("beta2", c_float), ("eps", c_float), ("weight_decay", c_float),
        ("bias_correction", ctypes.c_int32), ("grad_mult", c_float), ("reserved", ctypes.c_int32),
        ("hyper", c_void_p),
    ]


class LinkProbe(ctypes.Structure):
    """Mirror of ``ft_link_probe_t`` (GB/s; ``both_*`` is the sum of the two directions)."""

    _fields_ = [(name, c_double) for name in ("h2d_copy", "d2h_copy", "both_copy", "h2d_kernel", "d2h_kernel", "both_kernel",
                                              "both_copy_in_kernel_out", "both_kernel_in_copy_out")]


EXPORTS = {
    # name: (restype, argtypes)
    "ft_last_error": (c_char_p, []),
    "ft_abi_version": (c_int, []),
    "ft_device_count": (c_int, []),
    "ft_adam_create": (c_int, [c_int, c_float, c_float, c_float, c_float, c_float, c_int, c_int]),
    "ft_adam_destroy": (c_int, [c_int]),
    "ft_adam_step": (c_int, [c_int, c_uint64, c_float, c_float, c_float, c_float, c_float, c_int, c_float,
                             c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_size_t,
                             c_void_p, c_void_p]),
    "ft_adam_hyper_fill": (c_int, [c_int, c_uint64, c_float, c_float, c_float, c_float, c_float, c_int, c_float, c_void_p]),
    "ft_adam_step_hyper": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_size_t,
                                   c_void_p, c_void_p]),
    "ft_adam_step_multi": (c_int, [c_int, POINTER(AdamSegment), c_int, c_int, c_int, c_void_p, c_void_p]),
    "ft_grad_stats_workspace_bytes": (c_size_t, []),
    "ft_grad_stats": (c_int, [c_void_p, c_int, c_size_t, c_float, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "ft_grad_accumulate_workspace_bytes": (c_size_t, [c_size_t]),
    "ft_grad_accumulate": (c_int, [c_void_p, c_int, c_void_p, c_int, c_size_t, c_float, c_int, c_float, c_void_p, c_int,
                                   c_void_p, c_size_t, c_void_p]),
    "ft_grad_decide": (c_int, [c_void_p, c_int, c_size_t, c_float, c_void_p, c_int, c_float, c_float, c_void_p, c_void_p, c_size_t,
                               c_void_p]),
    "ft_grad_decide_dev": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_size_t,
                                   c_void_p]),
    "ft_grad_accumulate_decide": (c_int, [c_void_p, c_int, c_void_p, c_int, c_size_t, c_float, c_int, c_float, c_void_p, c_int,
                                          c_float, c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ft_grad_accumulate_static": (c_int, [c_void_p, c_int, c_void_p, c_int, c_size_t, c_float, c_int, c_float, c_void_p, c_int,
                                          c_void_p]),
    "ft_grad_control": (c_int, [c_void_p, c_float, c_float, c_void_p, c_void_p]),
    "ft_pinned_alloc": (c_int, [c_size_t, POINTER(c_void_p)]),
    "ft_pinned_free": (c_int, [c_void_p]),
    "ft_offload_create": (c_int, [c_size_t, c_int, POINTER(c_void_p)]),
    "ft_offload_set_mode": (c_int, [c_void_p, c_int]),
    "ft_offload_set_window_piece": (c_int, [c_void_p, c_size_t]),
    "ft_offload_destroy": (c_int, [c_void_p]),
    "ft_offload_step": (c_int, [c_void_p, c_int, c_uint64, c_float, c_float, c_float, c_float, c_float, c_int,
                                c_float, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                c_int, c_size_t, c_void_p, c_void_p]),
    "ft_offload_window_open": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, POINTER(c_int)]),
    "ft_offload_window_close": (c_int, [c_void_p, c_int]),
    "ft_offload_stream_wait": (c_int, [c_void_p, c_void_p, c_int]),
    "ft_offload_wait": (c_int, [c_void_p]),
    "ft_offload_elapsed_ms": (c_int, [c_void_p, POINTER(c_float)]),
    "ft_link_probe": (c_int, [c_size_t, c_int, POINTER(LinkProbe)]),
    "ft_link_bandwidth": (c_int, [c_size_t, c_int, c_int, POINTER(c_double)]),
    "ft_synth_fill": (c_int, [c_void_p, c_int, c_size_t, c_uint64, c_uint32, c_uint64, c_int, c_float, c_void_p]),
    "ft_synth_fill_host": (c_int, [c_void_p, c_int, c_size_t, c_uint64, c_uint32, c_uint64, c_int, c_float]),
    "ft_set_launch_tuning": (c_int, [c_int, c_int]),
    "ft_set_cache_tuning": (c_int, [c_size_t]),
    "ft_set_stats_launches": (c_int, [c_int]),
    "ft_set_launch_limit": (c_int, [c_uint64]),
    "ft_launch_pieces": (c_int, [c_uint64, c_uint64, POINTER(c_uint64), POINTER(c_uint64), c_int]),
    "ft_segment_batches": (c_int, [POINTER(c_uint64), c_int, c_uint64, POINTER(c_int)]),
    "ft_relaxed_tile_start": (c_int, [POINTER(c_uint64), POINTER(c_uint32), POINTER(c_uint32), c_int, POINTER(c_uint32)]),
    "ft_release_stream_scratch": (c_int, [c_void_p]),
}


class FtError(RuntimeError):
    """A libftadam.so entry point returned a negative code."""

    def __init__(self, fn: str, code: int, message: str):
        super().__init__(f"{fn} failed ({code}): {message}")
        self.code = code


_lib = None


def lib() -> ctypes.CDLL:
    """Loads the library on first use. Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m flextrain_amd.build` "
                "(hipcc, gfx950). There is no CPU fallback for the optimizer step.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(fn: str, rc: int) -> int:
    if rc < 0:
        msg = lib().ft_last_error()
        err = FtError(fn, rc, msg.decode() if msg else "")
        if rc in (-1, -2):  # FT_EINVAL, FT_EALIGN
            raise ValueError(str(err))
        raise err
    return rc


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}; expected float32, float16 or bfloat16") from None


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_ptr(device=None) -> int:
    """Handle of torch's current stream on ``device`` (default: the current device)."""
    if _RAW_STREAM is not None:  # the same handle without building a Stream object (2 us -> 0.3 us)
        if device is None:
            index = torch.cuda.current_device()
        else:
            index = device.index if isinstance(device, torch.device) else torch.device(device).index
            if index is None:
                index = torch.cuda.current_device()
        return _RAW_STREAM(index)
    return torch.cuda.current_stream(device).cuda_stream
