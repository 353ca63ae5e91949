"""Buffers for the optimizer step: pinned host memory, HBM buffers, rotation, side-stream copies.

Host-side mirror of the parts of the reference's ``flextrain/memory/__init__.py`` and
``flextrain/memory/pin_memory.py`` that feed the optimizer step (same public names and argument
meaning). What is different underneath:

* pinned host memory comes from ``hipHostMalloc`` through the C ABI in exactly the size asked
  for. The reference goes through torch's pinned allocator, which rounds every request up to a
  power of two, and therefore packs equal blocks into power-of-two chunks with a dynamic
  programme (``pin_memory.py:7-73``). ``allocate_optimal`` is kept for callers that still want
  that plan, but ``allocate_pin_memory_blocks`` no longer needs it: n blocks cost n x block bytes
  (rounded up to a page each), not the next power of two.
* ``FlexTrainDataStream.synchronize`` waits for the work that was launched through the stream
  (an event), not for the whole device (``__init__.py:394-395``), and ``wait()`` orders another
  stream behind it without blocking the host.
"""
from __future__ import annotations

import ctypes
import gc
import math
import weakref
from collections import defaultdict, deque
from math import ceil, prod
from typing import Callable, Dict, Iterable, List, Sequence, SupportsIndex, Tuple, Union

import torch
from torch import Tensor
from torch.nn import Parameter

from . import _C

_PAGE_SIZE = 4096

_ALLOCATED_VRAM_SIZE = 0
_ALLOCATED_DRAM_SIZE = 0


# ------------------------------------------------------------------------------------------------
# alignment and split arithmetic (pure integers)
# ------------------------------------------------------------------------------------------------
def _get_aligned_numel(original_numel: int, align_size: int) -> int:
    return -(-original_numel // align_size) * align_size


def get_partition_aligned_numel(numel: int, partition: int, itemsize: int) -> int:
    """Round up so that each of ``partition`` equal shares is a whole number of 4096-byte pages
    (reference ``__init__.py:322-323``)."""
    return _get_aligned_numel(numel, partition * _PAGE_SIZE // itemsize)


def get_page_aligned_numel(numel: int, itemsize: int, alignment_bytes: int = _PAGE_SIZE) -> int:
    """Round an element count up to whole pages (reference ``:326-333``)."""
    return _get_aligned_numel(numel, alignment_bytes // itemsize)


def get_page_aligned_padding_numel(numel: int, itemsize: int, alignment_bytes: int = _PAGE_SIZE) -> int:
    return get_page_aligned_numel(numel, itemsize, alignment_bytes) - numel


def get_split_numels(total_numel: int, ratios: Sequence[float], itemsize: int, num_levels: int = 3) -> Tuple[int, ...]:
    """Split ``total_numel`` over memory levels by ratio (reference ``:344-363``).

    Each of the first ``num_levels - 1`` levels gets ``ceil(total * ratio)`` rounded up to a page;
    if that over-commits, the excess is taken back from the last of them; the final level gets
    whatever remains.
    """
    ratios = list(ratios)[:num_levels - 1] if len(ratios) == num_levels else list(ratios)
    numels = [get_page_aligned_numel(ceil(total_numel * r), itemsize) for r in ratios]
    excess = sum(numels) - total_numel
    if excess > 0:
        numels[-1] -= excess
    numels.append(total_numel - sum(numels))
    return tuple(numels)


def allocate_optimal(n: int, size: int) -> Dict[int, int]:
    """Cheapest way to hold ``n`` blocks of ``size`` bytes in power-of-two chunks
    (reference ``pin_memory.py:7-73``): ``{chunk_bytes: how_many}`` minimising the total bytes.

    Candidate chunks run from the smallest power of two holding one block to the smallest holding
    all of them; ``best[x]`` is the least total for x blocks, built bottom-up. Among equally cheap
    plans the one met first (smaller chunk first) is kept, as in the reference.
    """
    if n <= 0:
        return {}

    def pow2_at_least(x: int) -> int:
        return max(0, (x - 1).bit_length())

    options = []
    for k in range(pow2_at_least(size), pow2_at_least(n * size) + 1):
        capacity = (1 << k) // size
        if capacity > 0:
            options.append((1 << k, capacity))

    best = [0] + [math.inf] * n
    pick: List[Tuple[int, int]] = [(0, 0)] * (n + 1)
    for x in range(1, n + 1):
        for chunk, capacity in options:
            cost = best[max(0, x - capacity)] + chunk
            if cost < best[x]:
                best[x], pick[x] = cost, (chunk, capacity)

    plan: Dict[int, int] = {}
    x = n
    while x > 0:
        chunk, capacity = pick[x]
        plan[chunk] = plan.get(chunk, 0) + 1
        x = max(0, x - capacity)
    return plan


def reshape_list(flat_list: List, shape: Sequence[int]) -> List:
    """Nest a flat list row-major into ``shape`` (reference ``pin_memory.py:76-97``)."""
    if len(shape) == 1:
        return flat_list
    stride = prod(shape[1:])
    return [reshape_list(flat_list[i * stride:(i + 1) * stride], shape[1:]) for i in range(shape[0])]


# ------------------------------------------------------------------------------------------------
# pinned host memory
# ------------------------------------------------------------------------------------------------
def pinned_bytes(nbytes: int) -> Tensor:
    """``nbytes`` of page-aligned pinned host memory as a uint8 tensor (uninitialised).

    The memory is released when the last tensor viewing it is gone."""
    if nbytes == 0:
        return torch.empty(0, dtype=torch.uint8)
    lib = _C.lib()
    # torch answers is_pinned() only once it has initialised the device itself
    torch.cuda.init()
    ptr = ctypes.c_void_p()
    _C.check("ft_pinned_alloc", lib.ft_pinned_alloc(nbytes, ctypes.byref(ptr)))
    carrier = (ctypes.c_uint8 * nbytes).from_address(ptr.value)
    weakref.finalize(carrier, lib.ft_pinned_free, ctypes.c_void_p(ptr.value))
    return torch.frombuffer(carrier, dtype=torch.uint8)


def pinned_empty(numel: int, dtype: torch.dtype) -> Tensor:
    return pinned_bytes(numel * dtype.itemsize).view(dtype)


def pinned_zeros(numel: int, dtype: torch.dtype) -> Tensor:
    t = pinned_empty(numel, dtype)
    t.view(torch.uint8).zero_()
    return t


def allocate_pin_memory_blocks(numel: int, dtype: torch.dtype, chunks: Union[int, Tuple[int, ...]]):
    """``prod(chunks)`` zero-filled pinned blocks of ``numel`` elements, nested as ``chunks``
    (reference ``pin_memory.py:100-171``). All blocks are carved out of one slab; each starts on a
    page boundary."""
    if isinstance(chunks, int):
        chunks = (chunks,)
    count = prod(chunks)
    if numel == 0:
        return reshape_list([torch.empty(0, dtype=dtype) for _ in range(count)], chunks)
    block_bytes = numel * dtype.itemsize
    stride = _get_aligned_numel(block_bytes, _PAGE_SIZE)
    slab = pinned_bytes(stride * count)
    slab.zero_()
    blocks = [slab[i * stride:i * stride + block_bytes].view(dtype) for i in range(count)]
    return reshape_list(blocks, chunks)


# ------------------------------------------------------------------------------------------------
# allocation with accounting
# ------------------------------------------------------------------------------------------------
def allocate_memory(numel: int, dtype: torch.dtype, device, pin_memory: bool = True) -> Tensor:
    """Zero-filled flat buffer on ``device``; host buffers are pinned unless asked otherwise
    (reference ``__init__.py:255-277``)."""
    global _ALLOCATED_DRAM_SIZE, _ALLOCATED_VRAM_SIZE
    device = torch.device(device)
    if device.type == "cpu":
        gc.collect()
        _ALLOCATED_DRAM_SIZE += numel * dtype.itemsize
        if pin_memory and numel > 0:
            return pinned_zeros(numel, dtype)
        return torch.zeros(numel, dtype=dtype)
    torch.cuda.empty_cache()
    _ALLOCATED_VRAM_SIZE += numel * dtype.itemsize
    return torch.zeros(numel, dtype=dtype, device=device)


def allocate_memory_chunks(numel: int, chunks: Union[int, Tuple[int, ...]], dtype: torch.dtype, device,
                           pin_memory: bool = True, mem_efficient: bool = True):
    """``chunks``-shaped collection of ``numel``-element buffers (reference ``:280-304``): a nested
    list of separate pinned blocks for efficient host allocation, one tensor viewed as
    ``(*chunks, numel)`` otherwise."""
    global _ALLOCATED_DRAM_SIZE
    if isinstance(chunks, int):
        chunks = (chunks,)
    device = torch.device(device)
    if device.type == "cpu" and pin_memory and mem_efficient:
        _ALLOCATED_DRAM_SIZE += numel * prod(chunks) * dtype.itemsize
        return allocate_pin_memory_blocks(numel, dtype, chunks)
    return allocate_memory(numel * prod(chunks), dtype, device, pin_memory).view(*chunks, numel)


_ARENA_ALIGN = 2 * 1024 * 1024
_ARENA_SKEW = 2 * 1024


def device_arena_layout(specs: Sequence[Tuple[int, torch.dtype]]) -> Tuple[List[int], int]:
    """Byte offsets of the arrays of ``allocate_device_arrays`` inside their one allocation, and
    its total size. Array k starts at the next 2 MiB boundary plus k x 2 KiB; arrays smaller than
    2 MiB are only 256-byte aligned."""
    offsets, cursor = [], 0
    for k, (numel, dtype) in enumerate(specs):
        nbytes = numel * dtype.itemsize
        if nbytes >= _ARENA_ALIGN:
            cursor = _get_aligned_numel(cursor, _ARENA_ALIGN) + (k * _ARENA_SKEW) % _ARENA_ALIGN
        else:
            cursor = _get_aligned_numel(cursor, 256)
        offsets.append(cursor)
        cursor += nbytes
    return offsets, max(cursor, 1)


def allocate_device_arrays(specs: Sequence[Tuple[int, torch.dtype]], device) -> List[Tensor]:
    """Zero-filled flat arrays for one update (parameters, moments, gradients, 16-bit copy ...),
    carved out of ONE device allocation.

    The update kernel streams all of its arrays at the same element index at once, and how their
    addresses relate decides how the streams collide in the memory system: arrays that torch
    happened to place badly have run the kernel 2-3 % slower than the same arrays in one
    allocation (855 M elements: 82 % against 84-85 % of peak bandwidth). One allocation with
    2 MiB-aligned starts and a 2 KiB stagger from array to array was the best or within 0.5 % of
    the best of the layouts measured, at every base address tried. The arrays keep the allocation
    alive; nothing else about them is special."""
    global _ALLOCATED_VRAM_SIZE
    device = torch.device(device)
    if device.type != "cuda":
        raise ValueError("allocate_device_arrays is for GPU memory; host state uses pinned_empty / allocate_memory")
    offsets, total = device_arena_layout(specs)
    total += _ARENA_ALIGN  # room to start the layout on a 2 MiB boundary wherever torch puts the block
    _ALLOCATED_VRAM_SIZE += total
    arena = torch.zeros(total, dtype=torch.uint8, device=device)
    lead = -arena.data_ptr() % _ARENA_ALIGN
    return [arena[lead + o:lead + o + numel * dtype.itemsize].view(dtype) for o, (numel, dtype) in zip(offsets, specs)]


def get_allocated_dram_size() -> int:
    return _ALLOCATED_DRAM_SIZE


def get_allocated_vram_size() -> int:
    return _ALLOCATED_VRAM_SIZE


# ------------------------------------------------------------------------------------------------
# tensor plumbing
# ------------------------------------------------------------------------------------------------
def free_tensor(tensor: Tensor, record_stream: bool = False) -> None:
    """Drop a tensor's storage but keep its device and dtype (reference ``:52-60``)."""
    if tensor.is_cuda and record_stream:
        tensor.record_stream(torch.cuda.current_stream())
    tensor.data = torch.empty(0, device=tensor.device, dtype=tensor.dtype)


def move_into_contiguous(srcs: Iterable[Tensor], dst: Tensor) -> None:
    """Pack tensors end to end into ``dst`` and re-point each at its slice (reference ``:63-84``)."""
    offset = 0
    for tensor in srcs:
        n, shape = tensor.numel(), tensor.shape
        target = dst[offset:offset + n]
        target.copy_(tensor.data.reshape(-1))
        free_tensor(tensor)
        tensor.data = target.view(shape)
        offset += n


def copy_segments(srcs: List[Tensor], dsts: List[Tensor], force_equal: bool = True) -> None:
    """Stream the concatenation of ``srcs`` into the concatenation of ``dsts`` without building
    either (reference ``:87-135``). Copies are ``non_blocking``; empty tensors are ignored; with
    ``force_equal=False`` the shorter side decides how much is copied."""
    srcs = [s.flatten() for s in srcs if s.numel() > 0]
    dsts = [d.flatten() for d in dsts if d.numel() > 0]
    if force_equal:
        assert sum(s.numel() for s in srcs) == sum(d.numel() for d in dsts)
    si = di = 0      # which tensor
    so = do = 0      # offset inside it
    while si < len(srcs) and di < len(dsts):
        src, dst = srcs[si], dsts[di]
        n = min(src.numel() - so, dst.numel() - do)
        dst[do:do + n].copy_(src[so:so + n], non_blocking=True)
        so += n
        do += n
        if so == src.numel():
            si, so = si + 1, 0
        if do == dst.numel():
            di, do = di + 1, 0


class ContiguousParaGroup:
    """Parameters kept in one flat buffer, ordered so that members of a parameter group are
    neighbours (reference ``:138-185``)."""

    def __init__(self, paras: Iterable[Parameter], param_grouping_mask: Iterable[int] = None):
        paras = list(paras)
        mask = list(param_grouping_mask) if param_grouping_mask is not None else [0] * len(paras)
        by_group = defaultdict(list)
        for key, para in zip(mask, paras):
            by_group[key].append(para)
        self.paras: List[Parameter] = [p for group in by_group.values() for p in group]
        self.numels = [p.numel() for p in self.paras]
        self.shapes = [p.shape for p in self.paras]

    def _views(self, contiguous_mem: Tensor):
        offset = 0
        for p, n, s in zip(self.paras, self.numels, self.shapes):
            yield p, contiguous_mem[offset:offset + n].view(s)
            offset += n

    def link_para_to(self, contiguous_mem: Tensor) -> None:
        for p, view in self._views(contiguous_mem):
            p.data = view

    def link_grad_to(self, contiguous_mem: Tensor) -> None:
        for p, view in self._views(contiguous_mem):
            if p.grad is None:
                p.grad = view
            else:
                p.grad.data = view

    def detach_para(self) -> None:
        for p in self.paras:
            free_tensor(p)

    def detach_grad(self) -> None:
        for p in self.paras:
            free_tensor(p.grad)


# ------------------------------------------------------------------------------------------------
# handles
# ------------------------------------------------------------------------------------------------
class Waitable:
    """Something that finishes later; ``wait()`` is idempotent (reference ``:188-203``)."""

    def __init__(self):
        self._finished = False

    def is_completed(self) -> bool:
        return self._finished

    def wait(self) -> None:
        if not self._finished:
            self._wait_task()
            self._finished = True

    def _wait_task(self) -> None:
        ...


class DummyHandle(Waitable):
    pass


class FunctionHandle(Waitable):
    def __init__(self, function: Callable, *args, **kwargs):
        super().__init__()
        self._call = (function, args, kwargs)

    def _wait_task(self) -> None:
        fn, args, kwargs = self._call
        fn(*args, **kwargs)


class AsyncIOHandle(Waitable):
    def __init__(self, handle: Waitable):
        super().__init__()
        self._handle = handle

    def _wait_task(self) -> None:
        self._handle.wait()


class FusedHandle(Waitable):
    def __init__(self, handles: Iterable[Waitable]):
        super().__init__()
        self._handles = list(handles)

    def _wait_task(self) -> None:
        for h in self._handles:
            h.wait()


class EventHandle(Waitable):
    """Completion of GPU work marked by an event (no counterpart in the reference, which waits
    for the whole device instead)."""

    def __init__(self, event: "torch.cuda.Event"):
        super().__init__()
        self._event = event

    def is_completed(self) -> bool:
        return self._finished or self._event.query()

    def _wait_task(self) -> None:
        self._event.synchronize()


class RotateContainer:
    """Buffer sets that trade places each step (reference ``:240-248``): after ``rotate()`` the
    item that was at index i is at index i + 1 and the last one is at index 0."""

    def __init__(self, items: Tuple):
        self._items = deque(items)

    def __getitem__(self, index: SupportsIndex):
        return self._items[index]

    def __len__(self) -> int:
        return len(self._items)

    def rotate(self) -> None:
        self._items.rotate(1)


# ------------------------------------------------------------------------------------------------
# side stream
# ------------------------------------------------------------------------------------------------
class FlexTrainDataStream:
    """Deferred copies on a side stream (reference ``:366-395``).

    ``submit`` queues closures; ``execute`` launches the stream tasks on the side stream (after
    everything already queued on the caller's stream, so a copy never overtakes the kernel that
    produced its source) and runs the normal tasks on the host; ``synchronize`` blocks the host
    until the launched work is done; ``wait`` makes a stream wait for it instead.
    """

    def __init__(self):
        self._stream = torch.cuda.Stream()  # default priority
        self._stream_tasks: List[Callable] = []
        self._normal_tasks: List[Callable] = []
        self._done = torch.cuda.Event()
        self._launched = False

    @property
    def stream(self) -> "torch.cuda.Stream":
        return self._stream

    def is_empty(self) -> bool:
        return not self._stream_tasks and not self._normal_tasks

    def submit(self, task: Callable, stream_execution: bool = True) -> None:
        (self._stream_tasks if stream_execution else self._normal_tasks).append(task)

    def execute(self) -> Waitable:
        if self._stream_tasks:
            self._stream.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(self._stream):
                for task in self._stream_tasks:
                    task()
                self._done.record(self._stream)
            self._launched = True
            self._stream_tasks.clear()
        for task in self._normal_tasks:
            task()
        self._normal_tasks.clear()
        return EventHandle(self._done) if self._launched else DummyHandle()

    def synchronize(self) -> None:
        if self._launched:
            self._done.synchronize()

    def wait(self, stream: "torch.cuda.Stream" = None) -> None:
        if self._launched:
            (stream or torch.cuda.current_stream()).wait_event(self._done)


_DATA_STREAM: FlexTrainDataStream = None


def get_data_stream() -> FlexTrainDataStream:
    """Process-wide side stream, created on first use (reference ``:398-412``)."""
    global _DATA_STREAM
    if _DATA_STREAM is None:
        _DATA_STREAM = FlexTrainDataStream()
    return _DATA_STREAM
