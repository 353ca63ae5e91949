"""Helpers shared by the tests: ULP distances on raw bit patterns and torch<->numpy views."""
from __future__ import annotations

import numpy as np
import torch

F32, F16, BF16 = 0, 1, 2
CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

# Tolerances of the hot path against the CPU oracle on identical inputs.
MASTER_ULP = 2      # fp32 master parameters, exp_avg, exp_avg_sq
HALF_ULP = 1        # bf16 / fp16 recast
NORM_RTOL = 1e-6    # global gradient norm against float64


def _ordered(bits: np.ndarray, width: int) -> np.ndarray:
    """Maps sign-magnitude float bit patterns to integers whose order is the floats' order."""
    b = bits.astype(np.int64)
    sign = np.int64(1) << (width - 1)
    return np.where(b & sign, sign - b, b)


def ulp_distance(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Element-wise distance in units in the last place between two arrays of the same float
    format given as float32/float16 arrays or uint16/uint32 bit patterns. Two NaNs are 0 apart;
    a NaN against a number is reported as a huge distance."""
    if a.dtype == np.float32:
        a, b, width, nan_lo = a.view(np.uint32), b.view(np.uint32), 32, 0x7f800000
    elif a.dtype == np.uint32:
        width, nan_lo = 32, 0x7f800000
    elif a.dtype == np.float16:
        a, b, width, nan_lo = a.view(np.uint16), b.view(np.uint16), 16, 0x7c00
    else:
        raise TypeError(a.dtype)
    mag = (1 << (width - 1)) - 1
    a_nan = (a.astype(np.int64) & mag) > nan_lo
    b_nan = (b.astype(np.int64) & mag) > nan_lo
    d = np.abs(_ordered(a, width) - _ordered(b, width))
    d = np.where(a_nan & b_nan, 0, d)
    d = np.where(a_nan ^ b_nan, np.int64(1) << 40, d)
    return d


def ulp_distance_bf16(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Same for bfloat16 bit patterns held in uint16 arrays."""
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    a_nan, b_nan = (a64 & 0x7fff) > 0x7f80, (b64 & 0x7fff) > 0x7f80
    d = np.abs(_ordered(a, 16) - _ordered(b, 16))
    d = np.where(a_nan & b_nan, 0, d)
    d = np.where(a_nan ^ b_nan, np.int64(1) << 40, d)
    return d


def max_ulp(a: np.ndarray, b: np.ndarray, bf16: bool = False, chunk: int = 1 << 24) -> int:
    """Largest ULP distance, computed chunk-wise to bound memory on large arrays."""
    worst = 0
    fn = ulp_distance_bf16 if bf16 else ulp_distance
    for lo in range(0, a.shape[0], chunk):
        d = fn(a[lo:lo + chunk], b[lo:lo + chunk])
        if d.size:
            worst = max(worst, int(d.max()))
    return worst


def to_np(t: torch.Tensor) -> np.ndarray:
    """Host numpy view/copy of a tensor; bf16 comes back as uint16 bit patterns."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def half_bits(t: torch.Tensor) -> np.ndarray:
    """uint16 bit patterns of an fp16/bf16 tensor."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def max_ulp_gpu(dev: torch.Tensor, host: np.ndarray, chunk: int = 1 << 26) -> int:
    """Largest ULP distance between a GPU tensor (fp32, or fp16/bf16) and host data of the same
    format (float32 array, or uint16 bit patterns), evaluated on the GPU chunk by chunk. NaN
    against NaN counts as equal, NaN against a number as a huge distance."""
    return ulp_histogram_gpu(dev, host, chunk)["max"]


def ulp_histogram_gpu(dev: torch.Tensor, host: np.ndarray, chunk: int = 1 << 26) -> dict:
    """How many elements of a GPU tensor lie 0, 1, 2 and more than 2 ULP from host data of the
    same format, plus the largest distance (see max_ulp_gpu for the conventions)."""
    n = dev.numel()
    assert host.shape[0] == n
    if dev.dtype == torch.float32:
        width, idt, exp_mask, view = 32, torch.int32, 0x7f800000, np.int32
    elif dev.dtype == torch.float16:
        width, idt, exp_mask, view = 16, torch.int16, 0x7c00, np.int16
    elif dev.dtype == torch.bfloat16:
        width, idt, exp_mask, view = 16, torch.int16, 0x7f80, np.int16
    else:
        raise TypeError(dev.dtype)
    mag = (1 << (width - 1)) - 1
    worst = 0
    counts = [0, 0, 0, 0]
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        a = dev[lo:hi].view(idt).to(torch.int64)
        b = torch.from_numpy(host[lo:hi].view(view)).to(dev.device).to(torch.int64)
        a_mag, b_mag = a & mag, b & mag
        a_nan, b_nan = a_mag > exp_mask, b_mag > exp_mask
        oa = torch.where(a < 0, -a_mag, a_mag)
        ob = torch.where(b < 0, -b_mag, b_mag)
        d = (oa - ob).abs()
        d = torch.where(a_nan & b_nan, torch.zeros_like(d), d)
        d = torch.where(a_nan ^ b_nan, torch.full_like(d, 1 << 40), d)
        worst = max(worst, int(d.max().item()))
        exact, one, two = int((d == 0).sum()), int((d == 1).sum()), int((d == 2).sum())
        counts = [counts[0] + exact, counts[1] + one, counts[2] + two, counts[3] + (hi - lo) - exact - one - two]
    return {"0": counts[0], "1": counts[1], "2": counts[2], ">2": counts[3], "max": worst}
