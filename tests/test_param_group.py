"""Segment algebra: hand-derived answers from the reference's semantics, brute force against a
per-element labelling, and the reference's own assertions turned into properties."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from flextrain_amd.param_group import (
    GroupSegment,
    StepContext,
    StepContextContainer,
    create_group_segments,
    create_step_contexts,
    create_tensor_split_plans,
    flatten_list,
    get_sliced_tensors,
    group_step_contexts,
    merge_segments,
    merge_slice_plans,
    reshape_list,
    slice_segments,
)

A, B, C = {"name": "A"}, {"name": "B"}, {"name": "C"}


def seg(group, lo, hi):
    return GroupSegment(group, lo, hi)


def as_tuples(segments):
    return [(s.param_group["name"], s.start, s.end) for s in segments]


def test_known_answers():
    assert merge_slice_plans([4, 4], [3, 5]) == [3, 1, 4]
    assert merge_slice_plans([8], [8]) == [8]
    assert merge_slice_plans([2, 0, 6], [8]) == [2, 6]  # empty pieces vanish
    assert create_tensor_split_plans([3, 5], [3, 1, 4]) == [[3], [1, 4]]
    assert create_tensor_split_plans([0, 3, 0, 5], [3, 1, 4]) == [[3], [1, 4]]  # empty tensors are dropped
    assert create_tensor_split_plans([], []) == []
    got = slice_segments([seg(A, 0, 5), seg(B, 5, 8)], [3, 1, 4])
    assert [as_tuples(w) for w in got] == [[("A", 0, 3)], [("A", 3, 4)], [("A", 4, 5), ("B", 5, 8)]]
    assert slice_segments([], [0, 0]) == [[], []]
    assert [as_tuples(w) for w in slice_segments([seg(A, 0, 4)], [0, 4, 0])] == [[], [("A", 0, 4)], []]
    with pytest.raises(AssertionError):
        create_tensor_split_plans([4, 4], [3, 5])  # boundary 4 is not a cut point
    with pytest.raises(AssertionError):
        merge_slice_plans([4, 4], [3, 4])  # different totals
    with pytest.raises(AssertionError):
        merge_slice_plans([8])  # needs two plans


def test_merge_segments_identity_and_remapping():
    a2 = {"name": "A"}  # equal content, different object: must NOT merge
    assert as_tuples(merge_segments([seg(A, 0, 2), seg(A, 2, 5), seg(a2, 5, 6), seg(B, 6, 6), seg(B, 6, 9)])) == \
        [("A", 0, 5), ("A", 5, 6), ("B", 6, 9)]
    assert merge_segments([]) == [] and merge_segments([seg(A, 3, 3)]) == []
    with pytest.raises(AssertionError):
        merge_segments([seg(A, 1, 2)])  # must start at 0 without remapping
    with pytest.raises(AssertionError):
        merge_segments([seg(A, 0, 2), seg(B, 3, 4)])  # gap
    # remapping re-bases to 0 and closes gaps
    assert as_tuples(merge_segments([seg(A, 10, 12), seg(A, 20, 23), seg(B, 40, 41)], is_remapping=True)) == \
        [("A", 0, 5), ("B", 5, 6)]
    # inputs are left untouched
    s0 = seg(A, 10, 12)
    merge_segments([s0, seg(A, 12, 14)], is_remapping=True)
    assert (s0.start, s0.end) == (10, 12)


def test_create_group_segments_and_contexts():
    params = [torch.zeros(3), torch.zeros(0), torch.zeros(2, 2), torch.zeros(5)]
    segs = create_group_segments(params, [A, B, A, B])
    assert as_tuples(segs) == [("A", 0, 7), ("B", 7, 12)]
    full, grad = torch.arange(12.0), torch.arange(12.0) * 10
    half = torch.arange(12.0).half()
    states = [torch.zeros(12), torch.ones(12)]
    ctxs = create_step_contexts(segs, half, full, grad, states)
    assert [c.param_group["name"] for c in ctxs] == ["A", "B"]
    assert ctxs[1].full_parameter.tolist() == list(range(7, 12))
    assert ctxs[1].full_parameter.data_ptr() == full[7:].data_ptr()  # views, not copies
    assert ctxs[0].half_parameter.numel() == 7 and len(ctxs[0].optimizer_states) == 2
    assert all(c.half_parameter is None for c in create_step_contexts(segs, None, full, grad, states))


def test_small_helpers():
    assert flatten_list([1, [2, [3, 4]], [], [[5]]]) == [1, 2, 3, 4, 5]
    assert flatten_list(7) == [7]
    arr = reshape_list(list(range(6)), [2, 3])
    assert arr.shape == (2, 3) and arr[1, 2] == 5
    assert reshape_list([[1], [2, 3]], [2]).shape == (2,)  # ragged items stay objects
    t = torch.arange(8)
    assert [x.tolist() for x in get_sliced_tensors(t, [[3, 5]])] == [[0, 1, 2], [3, 4, 5, 6, 7]]
    with pytest.raises(AssertionError):
        get_sliced_tensors([t], [[3, 4]])


plans = st.lists(st.integers(min_value=0, max_value=9), min_size=1, max_size=8)


@st.composite
def plans_with_total(draw, count):
    total = draw(st.integers(min_value=1, max_value=60))
    out = []
    for _ in range(count):
        k = draw(st.integers(min_value=1, max_value=6))
        cuts = sorted(draw(st.lists(st.integers(min_value=0, max_value=total), min_size=k - 1, max_size=k - 1)))
        edges = [0] + cuts + [total]
        out.append([b - a for a, b in zip(edges[:-1], edges[1:])])
    return total, out


@given(plans_with_total(3))
@settings(max_examples=200, deadline=None)
def test_merged_plan_is_the_union_of_cut_points(arg):
    total, ps = arg
    merged = merge_slice_plans(*ps)
    assert sum(merged) == total and all(x > 0 for x in merged)
    cuts = set(np.cumsum(merged).tolist())
    want = set()
    for p in ps:
        want |= set(np.cumsum(p).tolist())
    want.discard(0)
    assert cuts == want
    # every original plan can be dealt out of the merged plan
    for p in ps:
        dealt = create_tensor_split_plans(p, merged)
        assert [sum(d) for d in dealt] == [x for x in p if x > 0]
        assert [y for d in dealt for y in d] == merged


@given(plans_with_total(2))
@settings(max_examples=200, deadline=None)
def test_slice_segments_against_element_labels(arg):
    """Brute force: label every element with its group, slice, and read the labels back."""
    total, (seg_plan, win_plan) = arg
    groups = [{"name": f"g{i}"} for i in range(len(seg_plan))]
    segments, off = [], 0
    for g, n in zip(groups, seg_plan):
        if n:
            segments.append(GroupSegment(g, off, off + n))
        off += n
    labels = np.empty(total, dtype=object)
    for s in segments:
        labels[s.start:s.end] = s.param_group["name"]
    windows = slice_segments(segments, win_plan)
    assert len(windows) == len(win_plan)
    pos = 0
    for pieces, length in zip(windows, win_plan):
        assert sum(p.end - p.start for p in pieces) == length
        for p in pieces:
            assert p.start == pos and p.end > p.start
            assert (labels[p.start:p.end] == p.param_group["name"]).all()  # one group per piece
            pos = p.end
    assert pos == total


@given(plans_with_total(4), st.integers(min_value=1, max_value=6))
@settings(max_examples=150, deadline=None)
def test_step_context_container_partitions_evenly(arg, parts):
    """Every element is stepped exactly once, in the share that owns it, with the hyper-parameters of
    its group, through views of the right physical pieces."""
    total, (group_plan, dev_plan, master_plan, grad_plan) = arg
    total_p = total * parts  # make the total divisible by the number of partitions
    scale = lambda plan: [x * parts for x in plan]  # noqa: E731
    group_plan, dev_plan, master_plan, grad_plan = map(scale, (group_plan, dev_plan, master_plan, grad_plan))
    groups = [{"name": f"g{i}"} for i in range(len(group_plan))]
    # segments arrive with arbitrary offsets and gaps: the container remaps them
    segments, off = [], 100
    for g, n in zip(groups, group_plan):
        segments.append(GroupSegment(g, off, off + n))
        off += n + 3
    container = StepContextContainer(parts, segments, dev_plan, master_plan, grad_plan)

    def pieces(plan, dtype, base):
        out, o = [], 0
        for n in plan:
            out.append((torch.arange(o, o + n) + base).to(dtype))
            o += n
        return out
    half = pieces(dev_plan, torch.float64, 0)
    full = pieces(master_plan, torch.float64, 0)
    grad = pieces(grad_plan, torch.float64, 0)
    states = [pieces(master_plan, torch.float64, 0), pieces(master_plan, torch.float64, 0)]
    container.plan(half, full, grad, states)
    assert len(container) == parts
    owner = np.empty(total_p, dtype=object)
    o = 0
    for g, n in zip(groups, group_plan):
        owner[o:o + n] = g["name"]
        o += n
    seen = np.zeros(total_p, dtype=int)
    share = total_p // parts
    for k in range(parts):
        got = 0
        for ctx in container[k]:
            idx = ctx.full_parameter.long().numpy()
            assert np.array_equal(idx, np.arange(idx[0], idx[0] + len(idx)))           # contiguous
            assert k * share <= idx[0] and idx[-1] < (k + 1) * share                       # inside its share
            assert np.array_equal(ctx.gradient.long().numpy(), idx)                        # aligned buffers
            assert np.array_equal(ctx.half_parameter.long().numpy(), idx)
            assert all(np.array_equal(s.long().numpy(), idx) for s in ctx.optimizer_states)
            assert (owner[idx] == ctx.param_group["name"]).all()                            # one group
            seen[idx] += 1
            got += len(idx)
        assert got == share
    assert (seen == 1).all()
    # iterating the container goes over its parts and ends (indexing asserts its range, as the reference's does)
    assert [id(part) for part in container] == [id(container[k]) for k in range(parts)]
    # re-planning with half_parameter=None yields contexts without a copy-out
    container.plan(None, full, grad, states)
    assert all(ctx.half_parameter is None for k in range(parts) for ctx in container[k])


def test_empty_container_and_grouping_errors():
    c = StepContextContainer(3, [], [], [], [])
    c.plan(None, [], [], [[], []])
    assert len(c) == 3 and all(c._grouped_step_contexts[i] == [] for i in range(3))
    full = torch.arange(6.0)
    ctxs = create_step_contexts([seg(A, 0, 4), seg(B, 4, 6)], None, full, full, [full, full])
    assert [len(b) for b in group_step_contexts(ctxs, [4, 2])] == [1, 1]
    with pytest.raises(AssertionError):
        group_step_contexts(ctxs, [3, 3])  # a share boundary inside a context
    with pytest.raises(AssertionError):
        StepContextContainer(4, [seg(A, 0, 6)], [6], [6], [6])  # 6 % 4 != 0
