"""CPU checker for the optimizer-step hot path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package, and only to check or to time the CPU side. The product package never does.

Contents
--------
``libftoracle.so``  C restatement of the reference CPU Adam (sources next to this file; what
                    follows which reference line is listed in ``ft_oracle.h``).
``_ref/*.so``       the reference's own two C++ files compiled untouched (``make ref``); used to
                    validate the restatement and as the "reference" CPU baseline.
this module         ctypes/numpy access to both, plus pure-Python restatements of the reference's
                    loss-scale state machine (flextrain/loss_scaler.py:134-179) and of the
                    closed forms that define the extensions (clip coefficient, skip rule).

bf16 has no numpy dtype: bf16 arrays travel as ``np.uint16`` bit patterns with dtype code BF16.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import subprocess
from typing import Optional, Sequence, Tuple

import numpy as np

F32, F16, BF16 = 0, 1, 2

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libftoracle.so")


class Scalars(ctypes.Structure):
    """Mirror of ``ft_oracle_scalars``."""

    _fields_ = [
        ("beta1", ctypes.c_float),
        ("beta2", ctypes.c_float),
        ("omb1", ctypes.c_float),
        ("omb2", ctypes.c_float),
        ("bias2", ctypes.c_float),
        ("eps", ctypes.c_float),
        ("step_size", ctypes.c_float),
        ("wd_coef", ctypes.c_float),
        ("wd_mode", ctypes.c_int32),
        ("beta1_t", ctypes.c_float),
        ("beta2_t", ctypes.c_float),
        ("bias1", ctypes.c_float),
    ]


def build(force: bool = False) -> str:
    """Compile ``libftoracle.so`` with the Makefile beside this file (gcc only)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-f", os.path.join(_HERE, "Makefile"), "oracle"] + (["-B"] if force else []),
                       check=True, cwd=_HERE, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = ctypes.CDLL(_LIB_PATH)
    vp, sz, f32, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_int
    L.ft_oracle_scalars_compute.argtypes = [ctypes.c_uint64, f32, f32, f32, f32, f32, i32, i32, i32,
                                            ctypes.POINTER(Scalars)]
    L.ft_oracle_scalars_compute.restype = None
    L.ft_oracle_adam_step.argtypes = [ctypes.POINTER(Scalars), f32, vp, vp, i32, vp, vp, vp, i32, sz, i32, i32]
    L.ft_oracle_adam_step.restype = i32
    L.ft_oracle_adam_trace.argtypes = [ctypes.POINTER(Scalars), f32, f32, f32, f32, f32,
                                       ctypes.POINTER(ctypes.c_float * 11)]
    L.ft_oracle_adam_trace.restype = None
    L.ft_oracle_grad_stats.argtypes = [vp, i32, sz, f32, ctypes.POINTER(ctypes.c_uint64),
                                       ctypes.POINTER(ctypes.c_double), i32]
    L.ft_oracle_grad_stats.restype = i32
    L.ft_oracle_grad_accumulate.argtypes = [vp, i32, vp, i32, sz, f32, i32]
    L.ft_oracle_grad_accumulate.restype = i32
    L.ft_oracle_convert.argtypes = [vp, i32, vp, i32, sz]
    L.ft_oracle_convert.restype = None
    L.ft_oracle_best_isa.restype = i32
    L.ft_oracle_max_threads.restype = i32
    _lib = L
    return L


def _ptr(a: Optional[np.ndarray]) -> Optional[int]:
    return None if a is None else a.ctypes.data


def _check(a: np.ndarray, dtype_code: int, n: int, name: str) -> None:
    want = np.float32 if dtype_code == F32 else (np.float16 if dtype_code == F16 else np.uint16)
    if dtype_code == F16 and a.dtype == np.uint16:
        want = np.uint16
    if a.dtype != want or a.ndim != 1 or a.shape[0] != n or not a.flags.c_contiguous:
        raise ValueError(f"{name}: need contiguous 1-D {want} of {n}, got {a.dtype} {a.shape}")


def scalars(step: int, lr: float, betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-8,
            weight_decay: float = 0.0, bias_correction: bool = True, adamw_mode: bool = True,
            double_sqrt: bool = False) -> Scalars:
    s = Scalars()
    lib().ft_oracle_scalars_compute(int(step), lr, betas[0], betas[1], eps, weight_decay,
                                    int(bool(bias_correction)), int(bool(adamw_mode)),
                                    int(bool(double_sqrt)), ctypes.byref(s))
    return s


def adam_step(p: np.ndarray, g: np.ndarray, m: np.ndarray, v: np.ndarray, *, step: int, lr: float,
              betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-8, weight_decay: float = 0.0,
              bias_correction: bool = True, adamw_mode: bool = True, grad_mult: float = 1.0,
              g_dtype: int = F32, half_out: Optional[np.ndarray] = None, half_dtype: int = F16,
              isa: int = -1, threads: int = 0, double_sqrt: bool = False) -> Scalars:
    """In-place step on numpy arrays (p, m, v float32; g per ``g_dtype``)."""
    n = p.shape[0]
    _check(p, F32, n, "p")
    _check(m, F32, n, "m")
    _check(v, F32, n, "v")
    _check(g, g_dtype, n, "g")
    if half_out is not None:
        _check(half_out, half_dtype, n, "half_out")
    s = scalars(step, lr, betas, eps, weight_decay, bias_correction, adamw_mode, double_sqrt)
    rc = lib().ft_oracle_adam_step(ctypes.byref(s), grad_mult, _ptr(p), _ptr(g), g_dtype, _ptr(m), _ptr(v),
                                   _ptr(half_out), half_dtype, n, isa, threads)
    if rc != 0:
        raise RuntimeError("ft_oracle_adam_step rejected its arguments (dtype or isa)")
    return s


TRACE_NAMES = ("g32", "m1", "m_new", "v1", "g2", "v_new", "sqrt", "denom", "update", "p1", "p_new")


def adam_trace(s: Scalars, p: float, g: float, m: float, v: float, grad_mult: float = 1.0) -> dict:
    out = (ctypes.c_float * 11)()
    lib().ft_oracle_adam_trace(ctypes.byref(s), grad_mult, p, g, m, v, ctypes.byref(out))
    return {k: np.float32(out[i]) for i, k in enumerate(TRACE_NAMES)}


def grad_stats(g: np.ndarray, g_dtype: int, pre_mult: float = 1.0, threads: int = 0) -> Tuple[int, float]:
    """(count of inf/nan elements, double-precision sum of squares of the finite g*pre_mult)."""
    _check(g, g_dtype, g.shape[0], "g")
    bad, acc = ctypes.c_uint64(0), ctypes.c_double(0.0)
    rc = lib().ft_oracle_grad_stats(_ptr(g), g_dtype, g.shape[0], pre_mult, ctypes.byref(bad),
                                    ctypes.byref(acc), threads)
    if rc != 0:
        raise RuntimeError("ft_oracle_grad_stats rejected its arguments")
    return int(bad.value), float(acc.value)


def grad_accumulate(acc: np.ndarray, acc_dtype: int, g: np.ndarray, g_dtype: int, scale: float = 1.0,
                    zero_g: bool = False) -> None:
    """acc = round(fma(g, scale, acc)) in place (16-bit types as uint16 bit patterns)."""
    n = acc.shape[0]
    _check(acc, acc_dtype, n, "acc")
    _check(g, g_dtype, n, "g")
    if lib().ft_oracle_grad_accumulate(_ptr(acc), acc_dtype, _ptr(g), g_dtype, n, scale, int(bool(zero_g))) != 0:
        raise RuntimeError("ft_oracle_grad_accumulate rejected its arguments")


def convert(src: np.ndarray, src_dtype: int, dst_dtype: int) -> np.ndarray:
    """Software conversion between f32 / f16 / bf16 bit patterns (16-bit types as uint16)."""
    src = np.ascontiguousarray(src)
    dst = np.empty(src.shape[0], dtype=np.float32 if dst_dtype == F32 else np.uint16)
    lib().ft_oracle_convert(_ptr(src), src_dtype, _ptr(dst), dst_dtype, src.shape[0])
    return dst


def best_isa() -> int:
    return int(lib().ft_oracle_best_isa())


def max_threads() -> int:
    return int(lib().ft_oracle_max_threads())


# --------------------------------------------------------------------------------------------
# Closed forms that define the extensions (no counterpart in the reference).
# --------------------------------------------------------------------------------------------

def clip_coefficient(total_norm: float, max_norm: Optional[float], eps: float = 1e-6) -> float:
    """torch.nn.utils.clip_grad_norm_ convention: min(1, max_norm / (norm + 1e-6))."""
    if max_norm is None or max_norm <= 0:
        return 1.0
    return min(1.0, float(max_norm) / (float(total_norm) + eps))


def combined_multiplier(loss_scale: float, clip_coef: float) -> np.float32:
    """grad_mult = fl32(clip_coef) * fl32(1/loss_scale), one fp32 multiply."""
    return np.float32(np.float32(clip_coef) * np.float32(1.0 / float(loss_scale)))


def loss_scale_trace(overflows: Sequence[bool], init_scale: float, scale_factor: float = 2.0,
                     scale_window: int = 1000, min_scale: float = 1.0, delayed_shift: int = 1,
                     consecutive_hysteresis: bool = False) -> list:
    """State machine of flextrain/loss_scaler.py:134-179 replayed on a list of overflow flags.

    Returns the loss scale seen by each step followed by the final scale."""
    cur_scale, cur_iter, last_overflow_iter, hyst = init_scale, 0, -1, delayed_shift
    seen = []
    for ov in overflows:
        seen.append(cur_scale)
        if ov:
            if delayed_shift == 1 or hyst == 1:
                cur_scale = max(cur_scale / scale_factor, min_scale)
            else:
                hyst -= 1
            last_overflow_iter = cur_iter
        else:
            if consecutive_hysteresis:
                hyst = delayed_shift
            if (cur_iter - last_overflow_iter) % scale_window == 0:
                if not consecutive_hysteresis:
                    hyst = delayed_shift
                cur_scale *= scale_factor
        cur_iter += 1
    seen.append(cur_scale)
    return seen


# --------------------------------------------------------------------------------------------
# The compiled reference (oracle/_ref), when it has been built and this CPU can run it.
# --------------------------------------------------------------------------------------------

def _cpu_flags() -> set:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


_ref_mod = None
_ref_tried = False


def reference_module():
    """The reference's pybind module (create_adam / adam_update / adam_update_copy /
    destroy_adam, flextrain/ops/csrc/adam/cpu_adam.cpp:8-16) built by ``make ref``, or None."""
    global _ref_mod, _ref_tried
    if _ref_tried:
        return _ref_mod
    _ref_tried = True
    flags = _cpu_flags()
    order = []
    if {"avx512f", "avx512bw", "avx512vl", "avx512dq", "fma", "f16c"} <= flags:
        order.append("ref_cpu_adam_avx512")
    if {"avx2", "fma", "f16c"} <= flags:
        order.append("ref_cpu_adam_avx256")
    for name in order:
        path = os.path.join(_HERE, "_ref", name + ".so")
        if not os.path.exists(path):
            continue
        import torch  # noqa: F401  (the module links against libtorch)
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.flavour = name
        _ref_mod = mod
        break
    return _ref_mod
