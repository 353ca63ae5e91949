"""On-disk layout of a unit's master parameters and optimizer states.

The reference swaps part of every unit's ``[master | exp_avg | exp_avg_sq]`` block to NVMe as two
headerless files per unit and rank (``flextrain/memory/coordinator/optimizer.py:219-235,296-348``):

    <dir>/rank{r}_OPTS_layer{i}.swp.0   forward share:  3 x fwd_numel master-dtype elements
    <dir>/rank{r}_OPTS_layer{i}.swp.1   backward share: 3 x bwd_numel elements, zero-padded to a
                                        whole number of 4096-byte pages

named by ``FlexTrainDataID.__str__`` (``flextrain/memory/__init__.py:30-49``) plus the index
suffix of ``NVMeGroup._rename`` (``flextrain/memory/nvme_swapper.py:181-182``); a share with no
elements has no file (``nvme_swapper.py:24-40``). Each file is the raw little-endian bytes of the
three equal-length arrays one after the other, exactly as they lie in the host buffer.

This module writes and reads those files with plain positional I/O so that the per-unit
optimizer pipeline can checkpoint and resume its state in the reference's own format. It is not
a swapping tier: there is no asynchronous engine here, calls return when the bytes are on their
way to the page cache (``os.fsync`` on request).
"""
from __future__ import annotations

import os
from enum import Enum
from typing import List, Sequence, Tuple

import numpy as np
import torch
from torch import Tensor

from .memory import get_page_aligned_padding_numel

FORWARD_SHARE, BACKWARD_SHARE = 0, 1


class FlexTrainDataType(Enum):
    """Kinds of swapped data (reference ``flextrain/memory/__init__.py:20-27``)."""
    CKPT = 0
    PARA = 1
    GRAD = 2
    OPTS = 3


class FlexTrainDataID:
    """Name of one unit's swap file (reference ``flextrain/memory/__init__.py:30-49``). The rank
    and the number of layers per unit are arguments here; the reference reads them from its
    process group and its global configuration."""

    def __init__(self, data_type: FlexTrainDataType, unit_index: int, *, rank: int = 0, checkpoint_interval: int = 1):
        self.data_type = data_type
        self.unit_index = unit_index
        self.rank = rank
        self.checkpoint_interval = checkpoint_interval

    def __str__(self) -> str:
        start = self.unit_index * self.checkpoint_interval
        end = start + self.checkpoint_interval - 1
        layer_index = f"{start}-{end}" if self.checkpoint_interval > 1 else start
        return f"rank{self.rank}_{self.data_type.name}_layer{layer_index}.swp"


def opts_file_name(unit_index: int, share: int, *, rank: int = 0, checkpoint_interval: int = 1) -> str:
    prefix = FlexTrainDataID(FlexTrainDataType.OPTS, unit_index, rank=rank, checkpoint_interval=checkpoint_interval)
    return f"{prefix}.{share}"


def opts_file_layout(share_numel: int, share: int, *, states_per_element: int = 2, itemsize: int = 4) -> Tuple[int, int, int]:
    """``(payload_numel, padding_numel, file_bytes)`` of one share's file. Only the backward share
    is padded to whole pages (reference ``coordinator/optimizer.py:223-235``)."""
    payload = share_numel * (1 + states_per_element)
    padding = get_page_aligned_padding_numel(payload, itemsize) if share == BACKWARD_SHARE else 0
    return payload, padding, (payload + padding) * itemsize


def _host_bytes(t: Tensor) -> np.ndarray:
    if t.is_cuda or not t.is_contiguous():
        raise ValueError("state arrays must be contiguous host tensors")
    return t.view(torch.uint8).numpy()


def _check_block(blocks: Sequence[Tensor]) -> int:
    if not blocks:
        raise ValueError("no arrays given")
    numel, dtype = blocks[0].numel(), blocks[0].dtype
    if any(b.numel() != numel or b.dtype != dtype for b in blocks):
        raise ValueError("master parameters and states of one share must have equal length and dtype")
    return numel


def write_unit_opts(directory: str, unit_index: int, blocks: Sequence[Tensor], *, share: int = BACKWARD_SHARE,
                    rank: int = 0, checkpoint_interval: int = 1, fsync: bool = False) -> str | None:
    """Writes ``blocks = [master, exp_avg, exp_avg_sq]`` (host tensors of one share of one unit)
    as that share's file; returns its path, or None when the share is empty (no file)."""
    numel = _check_block(blocks)
    if numel == 0:
        return None
    itemsize = blocks[0].dtype.itemsize
    _, padding, file_bytes = opts_file_layout(numel, share, states_per_element=len(blocks) - 1, itemsize=itemsize)
    os.makedirs(directory, exist_ok=True)
    path = os.path.join(directory, opts_file_name(unit_index, share, rank=rank, checkpoint_interval=checkpoint_interval))
    fd = os.open(path, os.O_WRONLY | os.O_CREAT | os.O_TRUNC, 0o644)
    try:
        offset = 0
        for b in blocks:
            view = memoryview(_host_bytes(b))
            while len(view):
                done = os.pwrite(fd, view[:1 << 30], offset)
                offset += done
                view = view[done:]
        if padding:
            os.pwrite(fd, bytes(padding * itemsize), offset)
            offset += padding * itemsize
        assert offset == file_bytes
        if fsync:
            os.fsync(fd)
    finally:
        os.close(fd)
    return path


def read_unit_opts(directory: str, unit_index: int, blocks: Sequence[Tensor], *, share: int = BACKWARD_SHARE,
                   rank: int = 0, checkpoint_interval: int = 1) -> None:
    """Fills ``blocks`` from that share's file. The file must have exactly the size the layout
    gives for these arrays (a different unit size or state count is an error, never a guess)."""
    numel = _check_block(blocks)
    if numel == 0:
        return
    itemsize = blocks[0].dtype.itemsize
    _, _, file_bytes = opts_file_layout(numel, share, states_per_element=len(blocks) - 1, itemsize=itemsize)
    path = os.path.join(directory, opts_file_name(unit_index, share, rank=rank, checkpoint_interval=checkpoint_interval))
    fd = os.open(path, os.O_RDONLY)
    try:
        size = os.fstat(fd).st_size
        if size != file_bytes:
            raise ValueError(f"{path}: {size} bytes on disk, {file_bytes} expected for {len(blocks)} arrays of {numel} elements")
        offset = 0
        for b in blocks:
            view = memoryview(_host_bytes(b))
            while len(view):
                done = os.preadv(fd, [view[:1 << 30]], offset)
                if done <= 0:
                    raise IOError(f"{path}: short read at byte {offset}")
                offset += done
                view = view[done:]
    finally:
        os.close(fd)


def list_unit_opts(directory: str, num_units: int, *, share: int = BACKWARD_SHARE, rank: int = 0,
                   checkpoint_interval: int = 1) -> List[str]:
    return [os.path.join(directory, opts_file_name(u, share, rank=rank, checkpoint_interval=checkpoint_interval))
            for u in range(num_units)]
