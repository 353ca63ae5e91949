"""Seeded synthetic inputs that are the same bits on the GPU and on the host.

Element ``i`` of a fill is a pure function of ``(seed, substream, first_index + i)``: filling a
GPU tensor, a host tensor, or any chunk of either gives identical values, so a partition of
billions of elements can be regenerated anywhere (for a checker, on another machine) instead of
being copied around. The reference draws its probe inputs with ``torch.randn``
(``flextrain/optimizer.py:71-95``), which ties them to one process.
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import _C

NORMAL = 0
UNIFORM = 1


def fill_(out: Tensor, seed: int, substream: int, *, kind: int = NORMAL, scale: float = 1.0, first_index: int = 0) -> Tensor:
    """Fills the flat contiguous fp32 / fp16 / bf16 tensor ``out`` in place and returns it.

    ``kind=NORMAL``: mean 0, standard deviation ``scale`` (rounded to ``out``'s type to nearest
    even); ``kind=UNIFORM``: ``(0, scale]``. A GPU tensor is filled by a kernel on torch's current
    stream, a host tensor by the calling thread."""
    if out.dim() != 1 or not out.is_contiguous():
        raise ValueError("out must be a flat contiguous tensor")
    code = _C.dtype_code(out.dtype)
    lib = _C.lib()
    if out.is_cuda:
        with torch.cuda.device(out.device):
            _C.check("ft_synth_fill", lib.ft_synth_fill(
                out.data_ptr(), code, out.numel(), int(seed), int(substream), int(first_index), int(kind), float(scale),
                _C.current_stream_ptr(out.device)))
    else:
        _C.check("ft_synth_fill_host", lib.ft_synth_fill_host(
            out.data_ptr(), code, out.numel(), int(seed), int(substream), int(first_index), int(kind), float(scale)))
    return out
