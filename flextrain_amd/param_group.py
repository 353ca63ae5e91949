"""Segment algebra that turns flat optimizer buffers into per-partition step contexts.

Host-side mirror of the reference's ``flextrain/param_group.py`` (same public names, argument
meaning and results), written around one idea: every plan is a sorted list of cut points on the
axis ``[0, total)``, and slicing, merging and regrouping are set operations on cut points.

Reference lines each function answers to are given in the docstrings. Differences, on purpose:
functions never mutate the ``GroupSegment`` objects they are given (the reference's
``merge_segments`` edits them in place, ``param_group.py:48-80``), and a request to slice more
than the segments cover raises instead of re-emitting the last segment (``:152-168``).
"""
from __future__ import annotations

from bisect import bisect_right
from dataclasses import dataclass
from itertools import accumulate
from typing import Dict, List, Optional, Sequence, Union

import numpy as np
import torch

ParamGroup = Dict


def reshape_list(lst: List, shape: Sequence[int]) -> np.ndarray:
    """Object array view of ``lst`` with ``shape`` (reference ``param_group.py:9-10``)."""
    out = np.empty(len(lst), dtype=object)
    for i, item in enumerate(lst):
        out[i] = item
    return out.reshape(shape)


def flatten_list(nested) -> List:
    """Depth-first flattening of nested lists (reference ``param_group.py:13-19``)."""
    if not isinstance(nested, list):
        return [nested]
    flat: List = []
    stack = [iter(nested)]
    while stack:
        for item in stack[-1]:
            if isinstance(item, list):
                stack.append(iter(item))
                break
            flat.append(item)
        else:
            stack.pop()
    return flat


@dataclass
class GroupSegment:
    """Half-open element range ``[start, end)`` that belongs to one parameter group."""
    param_group: ParamGroup
    start: int
    end: int

    @property
    def numel(self) -> int:
        return self.end - self.start


@dataclass
class StepContext:
    """Everything one optimizer call needs: the group's hyper-parameters and matching views."""
    param_group: ParamGroup
    half_parameter: Optional[torch.Tensor]
    full_parameter: torch.Tensor
    gradient: torch.Tensor
    optimizer_states: List[torch.Tensor]


def is_same_param_group(pg1: ParamGroup, pg2: ParamGroup) -> bool:
    """Groups are compared by identity, never by content (reference ``param_group.py:38-39``)."""
    return pg1 is pg2


def _cuts(lengths: Sequence[int]) -> List[int]:
    """Running totals of ``lengths``: the right edge of every piece."""
    return list(accumulate(lengths))


def merge_segments(segments: List[GroupSegment], is_remapping: bool = False) -> List[GroupSegment]:
    """Joins neighbouring segments of the same group (reference ``param_group.py:42-80``).

    Empty segments are dropped. Without remapping the input must start at 0 and be gap-free;
    with remapping it is first re-based to 0 with all gaps closed.
    """
    merged: List[GroupSegment] = []
    cursor = 0
    for seg in segments:
        length = seg.end - seg.start
        if length == 0:
            continue
        if is_remapping:
            start = cursor
        else:
            assert seg.start == cursor, f"segment starts at {seg.start}, expected {cursor}"
            start = seg.start
        cursor = start + length
        if merged and is_same_param_group(merged[-1].param_group, seg.param_group):
            merged[-1].end = cursor
        else:
            merged.append(GroupSegment(seg.param_group, start, cursor))
    return merged


def create_group_segments(params: List[torch.Tensor], groups: List[ParamGroup]) -> List[GroupSegment]:
    """One merged segment list for parameters laid end to end (reference ``:83-109``)."""
    assert len(params) == len(groups)
    edges = [0] + _cuts([p.numel() for p in params])
    raw = [GroupSegment(g, lo, hi) for g, lo, hi in zip(groups, edges[:-1], edges[1:]) if hi > lo]
    return merge_segments(raw)


def slice_segments(segments: List[GroupSegment], lengths: List[int]) -> List[List[GroupSegment]]:
    """Cuts a gap-free sorted segment list into consecutive windows (reference ``:112-173``).

    Window ``k`` covers ``lengths[k]`` elements right after window ``k-1``; the pieces inside a
    window keep their group and never straddle a segment boundary.
    """
    if not segments:
        assert sum(lengths) == 0
        return [[] for _ in lengths]
    origin = segments[0].start
    seg_ends = [s.end for s in segments]
    assert origin + sum(lengths) <= seg_ends[-1], "lengths exceed what the segments cover"

    windows: List[List[GroupSegment]] = []
    lo = origin
    idx = 0  # first segment that still has elements at or after `lo`
    for length in lengths:
        hi = lo + length
        pieces: List[GroupSegment] = []
        while lo < hi:
            while seg_ends[idx] <= lo:
                idx += 1
            stop = min(hi, seg_ends[idx])
            pieces.append(GroupSegment(segments[idx].param_group, lo, stop))
            lo = stop
        windows.append(pieces)
    return windows


def create_step_contexts(
    group_segments: List[GroupSegment],
    half_parameter: Optional[torch.Tensor],
    full_parameter: torch.Tensor,
    gradient: torch.Tensor,
    optimizer_states: List[torch.Tensor],
) -> List[StepContext]:
    """Views of whole flat buffers, one context per segment (reference ``:176-224``)."""
    live = [gs for gs in group_segments if gs.end > gs.start]
    sizes = [gs.end - gs.start for gs in live]
    halves = half_parameter.split(sizes) if half_parameter is not None else [None] * len(sizes)
    fulls = full_parameter.split(sizes)
    grads = gradient.split(sizes)
    states = [state.split(sizes) for state in optimizer_states]
    return [
        StepContext(gs.param_group, halves[i], fulls[i], grads[i], [pieces[i] for pieces in states])
        for i, gs in enumerate(live)
    ]


def merge_slice_plans(*plans: List[int]) -> List[int]:
    """Coarsest plan that refines every given plan: union of cut points (reference ``:227-267``)."""
    assert len(plans) >= 2
    total = sum(plans[0])
    cuts = set()
    for plan in plans:
        assert sum(plan) == total, f"plan sums to {sum(plan)}, expected {total}"
        cuts.update(_cuts(plan))
    cuts.discard(0)
    ordered = sorted(cuts)
    return [hi - lo for lo, hi in zip([0] + ordered[:-1], ordered)]


def create_tensor_split_plans(tensor_numels: List[int], merged_split_plan: List[int]) -> List[List[int]]:
    """Deals a common plan out to consecutive tensors (reference ``:270-316``).

    Every tensor boundary must be a cut point of ``merged_split_plan``.
    """
    sizes = [n for n in tensor_numels if n > 0]
    if not sizes:
        assert sum(merged_split_plan) == 0
        return []
    assert sum(sizes) == sum(merged_split_plan)
    plan_cuts = _cuts(merged_split_plan)
    out: List[List[int]] = []
    begin = 0  # index into merged_split_plan
    for edge in _cuts(sizes):
        end = bisect_right(plan_cuts, edge)
        assert end > begin and plan_cuts[end - 1] == edge, "a tensor boundary is not a cut point of the plan"
        out.append(list(merged_split_plan[begin:end]))
        begin = end
    assert begin == len(merged_split_plan)
    return out


def get_sliced_tensors(
    tensors: Union[torch.Tensor, List[torch.Tensor]], split_plan: List[List[int]]
) -> List[torch.Tensor]:
    """Applies per-tensor split plans and concatenates the views (reference ``:319-333``)."""
    if isinstance(tensors, torch.Tensor):
        tensors = [tensors]
    tensors = [t for t in tensors if t.numel() > 0]
    assert len(tensors) == len(split_plan), \
        f"Expected {[t.numel() for t in tensors]} to match {split_plan}"
    views: List[torch.Tensor] = []
    for t, splits in zip(tensors, split_plan):
        assert t.numel() == sum(splits), f"Expected {splits} to match {t.numel()}"
        views.extend(torch.split(t, splits))
    return views


def group_step_contexts(step_contexts: List[StepContext], split_plan: List[int]) -> List[List[StepContext]]:
    """Buckets consecutive contexts so that bucket ``k`` holds ``split_plan[k]`` elements
    (reference ``:336-363``)."""
    edges = _cuts([ctx.full_parameter.numel() for ctx in step_contexts])
    buckets: List[List[StepContext]] = []
    begin = 0
    for edge in _cuts(split_plan):
        end = bisect_right(edges, edge)
        assert end > begin and edges[end - 1] == edge, "a partition boundary cuts through a step context"
        buckets.append(step_contexts[begin:end])
        begin = end
    assert begin == len(step_contexts)
    return buckets


class StepContextContainer(Sequence):
    """Splits one unit's optimizer work into ``num_partitions`` equal shares (reference ``:365-477``).

    The physical buffers of the low-precision parameters, the master parameters / states and the
    gradients may each come in several pieces; the container cuts everything at the union of all
    boundaries (equal shares, parameter groups, buffer pieces) so that each resulting context lies
    inside one group and one piece of every buffer, then hands the contexts out share by share.
    ``plan()`` re-binds the same cut pattern to a new set of tensors.
    """

    def __init__(
        self,
        num_partitions: int,
        group_segments: List[GroupSegment],
        device_param_numels: List[int],
        master_param_numels: List[int],
        gradient_numels: List[int],
    ):
        group_segments = merge_segments(group_segments, is_remapping=True)
        self._empty = not group_segments
        self._grouped_step_contexts: List[List[StepContext]] = []
        if self._empty:
            self._grouped_step_contexts = [[] for _ in range(num_partitions)]
            return

        total = group_segments[-1].end
        assert sum(device_param_numels) == total
        assert sum(master_param_numels) == total
        assert sum(gradient_numels) == total
        assert total % num_partitions == 0

        self._ep_slice_plan = [total // num_partitions] * num_partitions
        self._merged_plan = merge_slice_plans(
            self._ep_slice_plan,
            [gs.end - gs.start for gs in group_segments],
            device_param_numels, master_param_numels, gradient_numels,
        )
        self._group_segments: List[GroupSegment] = flatten_list(slice_segments(group_segments, self._merged_plan))
        self._half_parameter_splits = create_tensor_split_plans(device_param_numels, self._merged_plan)
        self._full_parameter_splits = create_tensor_split_plans(master_param_numels, self._merged_plan)
        self._gradient_splits = create_tensor_split_plans(gradient_numels, self._merged_plan)

    def plan(
        self,
        half_parameter: Union[None, torch.Tensor, List[torch.Tensor]],
        full_parameter: Union[torch.Tensor, List[torch.Tensor]],
        gradient: Union[torch.Tensor, List[torch.Tensor]],
        optimizer_states: List[Union[torch.Tensor, List[torch.Tensor]]],
    ) -> None:
        if self._empty:
            return
        pieces = len(self._group_segments)
        self.extra_copy = half_parameter is not None
        self.half_parameter = get_sliced_tensors(half_parameter, self._half_parameter_splits) \
            if self.extra_copy else [None] * pieces
        self.full_parameter = get_sliced_tensors(full_parameter, self._full_parameter_splits)
        self.gradient = get_sliced_tensors(gradient, self._gradient_splits)
        self.optimizer_states = [get_sliced_tensors(s, self._full_parameter_splits) for s in optimizer_states]

        assert len(self.half_parameter) == pieces
        assert len(self.full_parameter) == pieces
        assert len(self.gradient) == pieces
        assert all(len(s) == pieces for s in self.optimizer_states)

        self._step_contexts = [
            StepContext(
                param_group=self._group_segments[i].param_group,
                half_parameter=self.half_parameter[i],
                full_parameter=self.full_parameter[i],
                gradient=self.gradient[i],
                optimizer_states=[s[i] for s in self.optimizer_states],
            )
            for i in range(pieces)
        ]
        self._grouped_step_contexts = group_step_contexts(self._step_contexts, self._ep_slice_plan)

    def __getitem__(self, index: int) -> List[StepContext]:
        assert self._grouped_step_contexts
        assert 0 <= index < len(self._grouped_step_contexts)
        return self._grouped_step_contexts[index]

    def __len__(self) -> int:
        return len(self._grouped_step_contexts)

    def __iter__(self):
        return iter(self._grouped_step_contexts)
