"""How work is cut into launches, as arithmetic (no GPU): the update, the accumulation pass and the
many-segment call take their "workgroups per launch" decision from one host function whose limit
follows from what the HIP runtime accepts (gridDim.x * blockDim.x <= 2^32 - 1, blocks of 64 lanes).
Checked here with small artificial limits and at the real one: every workgroup is covered exactly
once, pieces are full except the last, and a piece's first workgroup is what the kernel receives as
its tile offset."""
import ctypes

import pytest

MAX_WORKGROUPS = (2 ** 32 - 1) // 64


@pytest.fixture(scope="module")
def lib():
    from flextrain_amd import _C
    return _C.lib()


def _pieces(lib, workgroups, limit, capacity=4096):
    first = (ctypes.c_uint64 * capacity)()
    count = (ctypes.c_uint64 * capacity)()
    n = lib.ft_launch_pieces(workgroups, limit, first, count, capacity)
    assert 0 <= n <= capacity
    return [(int(first[k]), int(count[k])) for k in range(n)]


@pytest.mark.parametrize("limit", [1, 2, 7, 64, 1000])
@pytest.mark.parametrize("workgroups", [0, 1, 6, 7, 8, 63, 64, 65, 999, 1000, 1001, 2999])
def test_pieces_cover_every_workgroup_exactly_once(lib, workgroups, limit):
    pieces = _pieces(lib, workgroups, limit)
    assert len(pieces) == -(-workgroups // limit)
    covered = []
    for k, (first, count) in enumerate(pieces):
        assert first == k * limit                      # the tile offset the k-th launch is given
        assert 1 <= count <= limit
        assert count == limit or k == len(pieces) - 1  # only the last piece may be short
        covered.extend(range(first, first + count))
    assert covered == list(range(workgroups))


def test_the_real_limit_is_what_the_runtime_accepts(lib):
    """Default limit: (2^32 - 1) // 64 workgroups. One more tile than that makes two launches; a
    2^36-element update (2^28 tiles) makes five, the last one short."""
    assert _pieces(lib, MAX_WORKGROUPS, 0) == [(0, MAX_WORKGROUPS)]
    assert _pieces(lib, MAX_WORKGROUPS + 1, 0) == [(0, MAX_WORKGROUPS), (MAX_WORKGROUPS, 1)]
    big = _pieces(lib, 2 ** 28, 0)
    assert len(big) == 5 and sum(c for _, c in big) == 2 ** 28
    assert all(c * 64 <= 2 ** 32 - 1 for _, c in big)
    assert big[-1] == (4 * MAX_WORKGROUPS, 2 ** 28 - 4 * MAX_WORKGROUPS)
    # a limit above what the runtime takes is refused; 0 restores the default
    assert lib.ft_set_launch_limit(MAX_WORKGROUPS + 1) < 0
    assert lib.ft_set_launch_limit(5) == 0
    try:
        assert _pieces(lib, 12, 0) == [(0, 5), (5, 5), (10, 2)]
    finally:
        assert lib.ft_set_launch_limit(0) == 0
    assert _pieces(lib, 12, 0) == [(0, 12)]


def _batches(lib, wgs, limit):
    arr = (ctypes.c_uint64 * len(wgs))(*wgs)
    out = (ctypes.c_int * len(wgs))()
    n = lib.ft_segment_batches(arr, len(wgs), limit, out)
    return n, [int(x) for x in out]


def test_segment_batches_respect_both_limits(lib):
    """Many-segment launches: at most 16 segments and `limit` workgroups per launch, in order."""
    n, batch_of = _batches(lib, [1] * 40, 1000)
    assert n == 3 and batch_of == [0] * 16 + [1] * 16 + [2] * 8
    n, batch_of = _batches(lib, [600, 300, 200, 1000, 1, 999, 1], 1000)
    assert batch_of == [0, 0, 1, 2, 3, 3, 4] and n == 5
    # brute force: any list, the greedy rule never overfills a launch and never splits early
    import random
    rng = random.Random(0)
    for _ in range(200):
        limit = rng.randrange(1, 50)
        wgs = [rng.randrange(1, limit + 1) for _ in range(rng.randrange(0, 60))]
        n, batch_of = _batches(lib, wgs, limit)
        assert batch_of == sorted(batch_of) and (n == 0) == (not wgs)
        for b in range(n):
            members = [w for w, k in zip(wgs, batch_of) if k == b]
            assert 1 <= len(members) <= 16 and sum(members) <= limit
            if b + 1 < n:  # the next segment did not fit
                nxt = wgs[batch_of.index(b + 1)]
                assert len(members) == 16 or sum(members) + nxt > limit
    # the default limit of a many-segment launch is the smaller of the table's encoding (2^28 - 1)
    # and what the runtime accepts
    n, batch_of = _batches(lib, [MAX_WORKGROUPS - 1, 1, 1], 0)
    assert batch_of == [0, 0, 1]


# ---- where relaxed-alignment tiles start -----------------------------------------------------------
def _tile_start(lib, arrays):
    """arrays: [(address, element bytes, weight)] -> (head, set of array indices whose tiles start on lines)"""
    n = len(arrays)
    addr = (ctypes.c_uint64 * n)(*[a for a, _, _ in arrays])
    width = (ctypes.c_uint32 * n)(*[w for _, w, _ in arrays])
    weight = (ctypes.c_uint32 * n)(*[w for _, _, w in arrays])
    mask = ctypes.c_uint32(0xffffffff)
    head = lib.ft_relaxed_tile_start(addr, width, weight, n, ctypes.byref(mask))
    assert 0 <= head < 64, head
    on = {k for k in range(n) if mask.value >> k & 1}
    assert mask.value >> n == 0
    for k, (a, w, _) in enumerate(arrays):  # the mask says exactly which arrays sit on 128-byte lines behind the head
        assert ((a + head * w) % 128 == 0) == (k in on), (k, head)
    return head, on


BASE = 0x7f00_0000_0000


def test_arrays_with_a_common_phase_all_start_on_lines(lib):
    for cut in (0, 1, 5, 31, 33, 63, 64, 100, 255):
        arrays = [(BASE + (k << 30) + cut * w, w, 4) for k, w in enumerate((4, 4, 4, 2, 2))]
        head, on = _tile_start(lib, arrays)
        assert on == {0, 1, 2, 3, 4} and head == (-cut) % 64, (cut, head)


@pytest.mark.parametrize("odd", range(5))
@pytest.mark.parametrize("shift", [1, 2, 3, 7, 40])
def test_one_array_off_leaves_the_others_on_lines(lib, odd, shift):
    widths = (4, 4, 4, 2, 2)
    arrays = [(BASE + (k << 30) + (shift * w if k == odd else 0), w, 8 if k < 3 else 2) for k, w in enumerate(widths)]
    head, on = _tile_start(lib, arrays)
    assert head == 0 and on == set(range(5)) - {odd}


def test_the_heavier_side_wins_and_ties_take_the_smaller_head(lib):
    # written state (weight 8 each) three elements in, gradient and copy (weight 2 each) at the start
    arrays = [(BASE + 12, 4, 8), (BASE + (1 << 30) + 12, 4, 8), (BASE + (2 << 30), 2, 2), (BASE + (3 << 30), 2, 2)]
    head, on = _tile_start(lib, arrays)
    assert head == 29 and on == {0, 1}
    # equal weights on both sides: both heads score the same, the smaller one is taken
    arrays = [(BASE + 12, 4, 8), (BASE + (1 << 30), 4, 8)]
    head, on = _tile_start(lib, arrays)
    assert head == 0 and on == {1}
    # nothing can be put on a line (dword-aligned fp32 arrays at different phases of 16 bytes):
    # the head that at least makes the heavier one's 4-element units whole vectors
    arrays = [(BASE + 4, 4, 8), (BASE + (1 << 30) + 8, 4, 2)]
    head, on = _tile_start(lib, arrays)
    assert on == {0} and head == 31  # 31 elements later the first array IS on a line


def test_tile_start_refuses_bad_arguments(lib):
    mask = ctypes.c_uint32()
    a, w, g = (ctypes.c_uint64 * 1)(BASE), (ctypes.c_uint32 * 1)(3), (ctypes.c_uint32 * 1)(1)
    assert lib.ft_relaxed_tile_start(a, w, g, 1, ctypes.byref(mask)) < 0
    w[0] = 4
    assert lib.ft_relaxed_tile_start(a, w, g, 0, ctypes.byref(mask)) < 0
    assert lib.ft_relaxed_tile_start(a, w, g, 1, ctypes.byref(mask)) == 0 and mask.value == 1
