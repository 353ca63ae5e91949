"""Host-side buffer logic that needs no GPU: split / alignment arithmetic, the power-of-two
packing plan, segment copies, rotation, handles."""
import itertools

import pytest
import torch

from flextrain_amd.memory import (
    ContiguousParaGroup,
    DummyHandle,
    FunctionHandle,
    FusedHandle,
    RotateContainer,
    allocate_optimal,
    copy_segments,
    device_arena_layout,
    get_page_aligned_numel,
    get_page_aligned_padding_numel,
    get_partition_aligned_numel,
    get_split_numels,
    move_into_contiguous,
    reshape_list,
)


def test_alignment_known_answers():
    assert get_page_aligned_numel(1, 4) == 1024
    assert get_page_aligned_numel(1024, 4) == 1024
    assert get_page_aligned_numel(1025, 4) == 2048
    assert get_page_aligned_numel(0, 2) == 0
    assert get_page_aligned_padding_numel(1000, 2) == 2048 - 1000
    assert get_page_aligned_numel(3, 2, alignment_bytes=16) == 8
    assert get_partition_aligned_numel(1, 4, 2) == 4 * 2048
    assert get_partition_aligned_numel(202_383_360, 4, 2) == 202_383_360  # the 7B layer needs no padding
    n = 202_383_360 + 1
    assert get_partition_aligned_numel(n, 4, 2) % (4 * 2048) == 0 and get_partition_aligned_numel(n, 4, 2) >= n


def test_split_numels_known_answers():
    assert get_split_numels(1000, (0.0, 1.0), 2) == (0, 1000, 0)
    assert get_split_numels(10000, (0.0, 0.5), 2) == (0, 6144, 3856)
    assert get_split_numels(10000, (0.0, 0.5, 0.5), 2) == (0, 6144, 3856)  # a third ratio is ignored
    assert get_split_numels(4096, (0.5, 0.5), 4) == (2048, 2048, 0)
    assert get_split_numels(100, (0.3,), 4, num_levels=2) == (100, 0)  # over-commit is clipped
    for total in (1, 4095, 4096, 123_457, 10 ** 7):
        for ratios in ((0.0, 0.0), (0.25, 0.5), (1.0, 0.0), (0.9, 0.9)):
            parts = get_split_numels(total, ratios, 2)
            assert sum(parts) == total and len(parts) == 3 and all(p >= 0 for p in parts[:1])


def brute_force_cost(n, size):
    k1 = max(0, (size - 1).bit_length())
    k2 = max(0, (n * size - 1).bit_length())
    chunks = [(1 << k, (1 << k) // size) for k in range(k1, k2 + 1)]
    best = None
    for counts in itertools.product(range(n + 1), repeat=len(chunks)):
        if sum(c * cap for c, (_, cap) in zip(counts, chunks)) >= n:
            cost = sum(c * ch for c, (ch, _) in zip(counts, chunks))
            best = cost if best is None else min(best, cost)
    return best


@pytest.mark.parametrize("size", [1, 3, 5, 1000, 4096, 4097, 6000])
def test_allocate_optimal_is_minimal(size):
    for n in range(1, 9):
        plan = allocate_optimal(n, size)
        assert all(ch & (ch - 1) == 0 for ch in plan)  # powers of two
        assert sum(cnt * (ch // size) for ch, cnt in plan.items()) >= n
        assert sum(cnt * ch for ch, cnt in plan.items()) == brute_force_cost(n, size), (n, size, plan)
    assert allocate_optimal(0, size) == {}


def test_allocate_optimal_examples():
    assert allocate_optimal(1, 4096) == {4096: 1}
    assert allocate_optimal(3, 4096) == {4096: 1, 8192: 1} or allocate_optimal(3, 4096) == {4096: 3}
    # 3 blocks of 5 bytes: 8 + 8 + 8 = 24 beats 16 (3 blocks) ... no: 16 holds 3 blocks for 16 bytes
    assert allocate_optimal(3, 5) == {16: 1}
    assert reshape_list(list(range(6)), (2, 3)) == [[0, 1, 2], [3, 4, 5]]
    assert reshape_list(list(range(4)), (4,)) == [0, 1, 2, 3]
    assert reshape_list(list(range(8)), (2, 2, 2))[1][0] == [4, 5]


def test_copy_segments_equals_concatenate_then_split():
    torch.manual_seed(0)
    for sizes_src, sizes_dst in (([5, 0, 3, 8], [4, 4, 8]), ([16], [1] * 16), ([1] * 7, [7]), ([2, 3], [5])):
        srcs = [torch.randn(n) for n in sizes_src]
        dsts = [torch.zeros(n) for n in sizes_dst]
        copy_segments(srcs, dsts)
        assert torch.equal(torch.cat(dsts), torch.cat(srcs))
    srcs = [torch.arange(6.0).reshape(2, 3)]  # shapes are flattened
    dsts = [torch.zeros(3, 2)]
    copy_segments(srcs, dsts)
    assert dsts[0].flatten().tolist() == list(range(6))
    with pytest.raises(AssertionError):
        copy_segments([torch.zeros(3)], [torch.zeros(4)])
    dst = torch.zeros(4)
    copy_segments([torch.ones(3)], [dst], force_equal=False)
    assert dst.tolist() == [1, 1, 1, 0]


def test_rotate_container_and_handles():
    r = RotateContainer(("recv", "step", "offload"))
    assert (r[0], r[1], r[2]) == ("recv", "step", "offload")
    r.rotate()
    assert (r[0], r[1], r[2]) == ("offload", "recv", "step")  # each item moves one slot up
    r.rotate()
    r.rotate()
    assert (r[0], r[1], r[2]) == ("recv", "step", "offload") and len(r) == 3
    calls = []
    h = FunctionHandle(lambda x, y=0: calls.append((x, y)), 1, y=2)
    assert not h.is_completed()
    h.wait()
    h.wait()
    assert calls == [(1, 2)] and h.is_completed()
    fused = FusedHandle([FunctionHandle(calls.append, "a"), DummyHandle(), FunctionHandle(calls.append, "b")])
    fused.wait()
    assert calls[1:] == ["a", "b"]


def test_move_into_contiguous_and_para_group():
    a, b = torch.arange(6.0).reshape(2, 3), torch.arange(4.0) + 10
    dst = torch.zeros(10)
    move_into_contiguous([a, b], dst)
    assert dst.tolist() == [0, 1, 2, 3, 4, 5, 10, 11, 12, 13]
    assert a.shape == (2, 3) and a.data_ptr() == dst.data_ptr() and b.data_ptr() == dst[6:].data_ptr()
    params = [torch.nn.Parameter(torch.full((2,), float(i))) for i in range(4)]
    group = ContiguousParaGroup(params, [1, 0, 1, 0])
    assert [int(p[0].item()) for p in group.paras] == [0, 2, 1, 3]  # grouped by mask, order of first sight
    flat = torch.arange(8.0)
    group.link_para_to(flat)
    assert params[2].tolist() == [2.0, 3.0] and params[1].tolist() == [4.0, 5.0]
    grads = torch.zeros(8)
    group.link_grad_to(grads)
    params[3].grad += 1
    assert grads.tolist() == [0, 0, 0, 0, 0, 0, 1, 1]
    group.detach_para()
    assert all(p.numel() == 0 for p in params)


def test_device_arena_layout_staggers_large_arrays_and_packs_small_ones():
    """Arrays of 2 MiB and more start on a 2 MiB boundary plus 2 KiB times their index and never
    overlap; small ones are only 256-byte aligned; the total covers the last array."""
    mib2 = 2 * 1024 * 1024
    specs = [(202_383_360, torch.float32)] * 3 + [(202_383_360, torch.bfloat16)] * 2
    offsets, total = device_arena_layout(specs)
    assert [o % mib2 for o in offsets] == [0, 2048, 4096, 6144, 8192]
    ends = [o + n * dt.itemsize for o, (n, dt) in zip(offsets, specs)]
    assert all(ends[k] <= offsets[k + 1] for k in range(4)) and total == ends[-1]
    assert total - sum(n * dt.itemsize for n, dt in specs) < 5 * mib2          # padding is bounded

    offsets, total = device_arena_layout([(7, torch.float32), (3, torch.float16), (1 << 20, torch.float32), (5, torch.float32)])
    assert offsets[0] == 0 and offsets[1] == 256 and offsets[2] == mib2 + 2 * 2048
    assert offsets[3] == -(-(offsets[2] + (4 << 20)) // 256) * 256 and total == offsets[3] + 20
    assert device_arena_layout([]) == ([], 1)
