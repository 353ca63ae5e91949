"""GPU tests of the pinned-host <-> HBM pipeline: the streamed step must give the bits of the
resident step (and so of the oracle), whatever the chunking, slot count, or where gradients and
the low-precision copy live."""
import numpy as np
import pytest
import torch

from _util import CODE, F16, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)


def _host_state(n, seed):
    from flextrain_amd.memory import pinned_empty
    rng = np.random.default_rng(seed)
    p, m, v = (pinned_empty(n, torch.float32) for _ in range(3))
    p.copy_(torch.from_numpy(rng.normal(0, 0.02, n).astype(np.float32)))
    m.copy_(torch.from_numpy(rng.normal(0, 1e-4, n).astype(np.float32)))
    v.copy_(torch.from_numpy(rng.uniform(0, 1e-6, n).astype(np.float32)))
    return p, m, v


def _oracle(oracle, p, g, m, v, step, half_dtype, grad_mult=1.0):
    pn, mn, vn = p.numpy().copy(), m.numpy().copy(), v.numpy().copy()
    gn = to_np(g)
    if g.dtype == torch.float16:
        gn = gn.view(np.uint16)
    hn = np.zeros(pn.shape[0], np.uint16) if half_dtype is not None else None
    oracle.adam_step(pn, gn, mn, vn, step=step, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                     weight_decay=HP["weight_decay"], g_dtype=CODE[g.dtype], grad_mult=grad_mult, half_out=hn,
                     half_dtype=CODE[half_dtype] if half_dtype is not None else F16)
    return pn, mn, vn, hn


def _assert_equal_bits(tag, p, m, v, h, want, half_dtype):
    pn, mn, vn, hn = want
    worst = dict(p=max_ulp(p.numpy(), pn), m=max_ulp(m.numpy(), mn), v=max_ulp(v.numpy(), vn))
    if h is not None:
        hb = half_bits(h)
        worst["h"] = max_ulp(hb, hn, bf16=True) if half_dtype == torch.bfloat16 else max_ulp(hb.view(np.float16), hn.view(np.float16))
    print(f"[{tag}] worst ULP distance: {worst}", flush=True)
    assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst.get("h", 0) <= HALF_ULP, (tag, worst)


def test_pinned_allocations(cuda):
    from flextrain_amd.memory import allocate_memory, allocate_memory_chunks, allocate_pin_memory_blocks, pinned_empty
    t = pinned_empty(1_000_003, torch.float32)
    assert t.is_pinned() and t.numel() == 1_000_003 and t.data_ptr() % 4096 == 0
    z = allocate_memory(12345, torch.float32, "cpu")
    assert z.is_pinned() and not z.any()
    blocks = allocate_pin_memory_blocks(1000, torch.float16, (2, 3))
    assert len(blocks) == 2 and len(blocks[0]) == 3
    flat = [b for row in blocks for b in row]
    assert all(b.is_pinned() and b.numel() == 1000 and b.dtype == torch.float16 and not b.any() for b in flat)
    assert all(b.data_ptr() % 4096 == 0 for b in flat)
    spans = sorted((b.data_ptr(), b.data_ptr() + 2000) for b in flat)
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))  # disjoint
    nested = allocate_memory_chunks(64, (2, 2), torch.float32, "cpu")
    assert nested[1][1].is_pinned()
    dev = allocate_memory_chunks(64, 3, torch.float32, cuda)
    assert dev.shape == (3, 64) and dev.is_cuda
    empty = allocate_pin_memory_blocks(0, torch.float32, 2)
    assert len(empty) == 2 and empty[0].numel() == 0
    # round trip through the GPU
    t.copy_(torch.arange(1_000_003, dtype=torch.float32))
    d = t.to(cuda, non_blocking=True)
    torch.cuda.synchronize()
    assert d[-1].item() == 1_000_002.0


def test_data_stream_orders_copies_behind_their_producer(cuda):
    from flextrain_amd.memory import FlexTrainDataStream, pinned_empty
    ds = FlexTrainDataStream()
    n = 8_000_000
    src = torch.zeros(n, device=cuda)
    dst = pinned_empty(n, torch.float32)
    dst.zero_()
    ran = []
    for i in range(3):
        src.add_(1.0)  # producer on the current stream
        ds.submit(lambda: dst.copy_(src, non_blocking=True))
        ds.submit(lambda: ran.append(i), stream_execution=False)
        handle = ds.execute()
        ds.wait()  # the producer of the next round must not overwrite src before the copy has read it
        handle.wait()
        assert dst[0].item() == float(i + 1) and dst[-1].item() == float(i + 1)
    assert ran == [0, 1, 2] and ds.is_empty()
    ds.synchronize()


@pytest.mark.parametrize("slots", [2, 3])
@pytest.mark.parametrize("n,chunk", [(1_000_003, 1 << 16), (300_000, 1 << 20), (4 * (1 << 16), 1 << 16)])
def test_streamed_step_device_grads(cuda, oracle, n, chunk, slots, mode=1):
    """Master state in pinned host memory, bf16 grads and bf16 copy on the GPU (the offloaded
    configuration), several chunks, ragged last chunk, two steps in a row."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(offload_chunk_elems=chunk, offload_slots=slots, offload_mode=mode, **HP)
    p, m, v = _host_state(n, seed=n)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    gen = torch.Generator(device=cuda).manual_seed(1)
    for t in (1, 2):
        g = (torch.randn(n, device=cuda, generator=gen) * 1e-3).to(torch.bfloat16)
        want = _oracle(oracle, p, g, m, v, t, torch.bfloat16)
        eng._step({"step": t}, h, p, g, m, v)
        _assert_equal_bits(f"offload n={n} chunk={chunk} slots={slots} t={t}", p, m, v, h, want, torch.bfloat16)


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_streamed_step_reference_layout(cuda, oracle, mode):
    """Everything in pinned host memory with fp32 gradients and an fp16 copy: the layout the
    reference's coordinator hands to the step."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.memory import pinned_empty
    n = 700_001
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 17, offload_slots=2, offload_mode=mode, **HP)
    p, m, v = _host_state(n, seed=3)
    g = pinned_empty(n, torch.float32)
    g.copy_(torch.randn(n) * 1e-3)
    h = pinned_empty(n, torch.float16)
    h.zero_()
    want = _oracle(oracle, p, g, m, v, 9, torch.float16)
    eng._step({"step": 9}, h, p, g, m, v)
    _assert_equal_bits("host layout", p, m, v, h, want, torch.float16)
    assert eng.last_offload_ms() > 0


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_streamed_equals_resident_bit_for_bit(cuda, mode):
    """Every transfer mode (automatic, staged, direct, staged-in, staged-out) gives the resident
    kernel's bits."""
    from flextrain_amd import FlexTrainCPUAdam
    n = 3_000_017
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 18, offload_slots=3, offload_mode=mode, **HP)
    p, m, v = _host_state(n, seed=8)
    g = (torch.randn(n, device=cuda) * 1e-3 * 512).to(torch.float16)
    dp, dm, dv = p.to(cuda), m.to(cuda), v.to(cuda)
    dh = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    for t in range(1, 4):
        eng._step({"step": t}, dh, dp, g, dm, dv, grad_mult=1.0 / 512)
        eng._step({"step": t}, h, p, g, m, v, grad_mult=1.0 / 512)
    torch.cuda.synchronize()
    assert torch.equal(dp.cpu(), p) and torch.equal(dm.cpu(), m) and torch.equal(dv.cpu(), v) and torch.equal(dh, h)


def test_non_blocking_step_and_explicit_wait(cuda, oracle):
    from flextrain_amd import FlexTrainCPUAdam
    n = 2_000_000
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 18, **HP)
    p, m, v = _host_state(n, seed=5)
    g = (torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16)
    want = _oracle(oracle, p, g, m, v, 1, None)
    eng._step({"step": 1}, None, p, g, m, v, blocking=False)
    eng.synchronize()
    _assert_equal_bits("non-blocking", p, m, v, None, want, None)


def test_pageable_host_memory_is_refused(cuda):
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 16, **HP)
    n = 1000
    p, m, v = (torch.zeros(n) for _ in range(3))
    g = torch.zeros(n, device=cuda)
    with pytest.raises(ValueError, match="pinned"):
        eng._step({"step": 1}, None, p, g, m, v)


def test_a_refused_step_leaves_nothing_enqueued(cuda, oracle):
    """Whatever can refuse a streamed step is checked before anything is enqueued: a gradient pointer
    off its element alignment in a step of several chunks returns FT_EALIGN with the host state
    untouched and the engine idle, and the next good step runs as if nothing had happened."""
    from flextrain_amd import FlexTrainCPUAdam, _C
    n, chunk = 300_000, 1 << 16
    eng = FlexTrainCPUAdam(offload_chunk_elems=chunk, offload_mode=1, **HP)
    p, m, v = _host_state(n, 41)
    before = [t.clone() for t in (p, m, v)]
    gbuf = (torch.randn(n + 8, device=cuda) * 1e-3).to(torch.bfloat16)
    g = gbuf[:n]
    engine = eng._offload_engine()
    lib = _C.lib()
    rc = lib.ft_offload_step(engine, eng.opt_id, 3, 1e-4, 0.9, 0.999, 1e-8, 0.01, 1, 1.0, p.data_ptr(), gbuf.data_ptr() + 1,
                             _C.BF16, 0, m.data_ptr(), v.data_ptr(), None, _C.F16, 0, n, None, _C.current_stream_ptr())
    assert rc == -2 and b"aligned" in lib.ft_last_error()
    bad_ctl = torch.zeros(8, dtype=torch.float32, device=cuda)
    rc = lib.ft_offload_step(engine, eng.opt_id, 3, 1e-4, 0.9, 0.999, 1e-8, 0.01, 1, 1.0, p.data_ptr(), g.data_ptr(),
                             _C.BF16, 0, m.data_ptr(), v.data_ptr(), None, _C.F16, 0, n, bad_ctl.data_ptr() + 4, _C.current_stream_ptr())
    assert rc == -2
    eng.synchronize()
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip((p, m, v), before))
    want = _oracle(oracle, p, g, m, v, 3, None)
    eng._step({"step": 3}, None, p, g, m, v)
    _assert_equal_bits("after refused steps", p, m, v, None, want, None)


def test_link_probe_reports_sane_numbers(cuda):
    import ctypes
    from flextrain_amd import _C
    lib = _C.lib()
    out = ctypes.c_double()
    for direction in (0, 1, 2):
        _C.check("ft_link_bandwidth", lib.ft_link_bandwidth(256 << 20, 4, direction, ctypes.byref(out)))
        print(f"[link] direction {direction}: {out.value:.1f} GB/s", flush=True)
        assert 1.0 < out.value < 1000.0


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_steps_on_disjoint_memory_overlap_and_same_memory_stay_ordered(cuda, oracle, mode):
    """Per-unit use: many non-blocking steps in a row, each on its own host arrays, then two on the
    same arrays; every result must equal the oracle's, and more steps than the engine tracks
    individually (8) must still be ordered correctly."""
    from flextrain_amd import FlexTrainCPUAdam
    n, units = 400_000, 12
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 17, offload_slots=2, offload_mode=mode, **HP)
    state = [_host_state(n, seed=50 + u) for u in range(units)]
    grads = [(torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16) for _ in range(units)]
    halves = [torch.zeros(n, dtype=torch.bfloat16, device=cuda) for _ in range(units)]
    want = [_oracle(oracle, *(state[u][0], grads[u], state[u][1], state[u][2]), 3, torch.bfloat16) for u in range(units)]
    for u in range(units):
        p, m, v = state[u]
        eng._step({"step": 3}, halves[u], p, grads[u], m, v, blocking=False, guard_stream=False)
    # unit 0 again, twice, on the same memory: must see the result of the earlier step
    p, m, v = state[0]
    pn, mn, vn, _ = want[0]
    for t in (4, 5):
        eng._step({"step": t}, halves[0], p, grads[0], m, v, blocking=False, guard_stream=False)
        hn = np.zeros(n, np.uint16)
        oracle.adam_step(pn, to_np(grads[0]), mn, vn, step=t, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                         weight_decay=HP["weight_decay"], g_dtype=CODE[torch.bfloat16], half_out=hn, half_dtype=CODE[torch.bfloat16])
    want[0] = (pn, mn, vn, hn)
    eng.stream_wait()
    eng.synchronize()
    for u in range(units):
        p, m, v = state[u]
        _assert_equal_bits(f"unit {u}", p, m, v, halves[u], want[u], torch.bfloat16)


@pytest.mark.parametrize("mode", [1, 2])
def test_buffers_poisoned_as_soon_as_the_engine_says_they_are_free(cuda, oracle, mode):
    """Event dependencies of the streamed step, made visible with poison. The gradient buffer is
    filled by a copy enqueued just before the step (the step must wait for its producer), is
    overwritten with NaN right after a device-side wait for the step's kernels (nothing may read it
    after that), and the host arrays are read back by a copy ordered only by the device-side wait
    for the write-back. 46 chunks through 2 slots, no host synchronisation until the end."""
    from flextrain_amd import FlexTrainCPUAdam
    n = 3_000_001
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 16, offload_slots=2, offload_mode=mode, **HP)
    p, m, v = _host_state(n, seed=77)
    real = (torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16)
    want = _oracle(oracle, p, real, m, v, 2, torch.bfloat16)
    g = torch.full((n,), float("nan"), dtype=torch.bfloat16, device=cuda)
    h = torch.full((n,), float("nan"), dtype=torch.bfloat16, device=cuda)
    mirror = torch.zeros(n, device=cuda)
    torch.cuda.synchronize()
    g.copy_(real)                                   # producer on the current stream
    eng._step({"step": 2}, h, p, g, m, v, blocking=False)
    eng.stream_wait()                               # kernels done -> g is free, h is final
    g.fill_(float("nan"))                           # poison
    h_seen = h.clone()
    eng.stream_wait(write_back=True)                # write-back done -> host arrays are final
    mirror.copy_(p, non_blocking=True)
    torch.cuda.synchronize()
    eng.synchronize()
    _assert_equal_bits(f"poison mode={mode}", p, m, v, h_seen, want, torch.bfloat16)
    assert torch.equal(mirror.cpu(), p)
    assert torch.isnan(g).all()


def test_window_keeps_a_unit_on_the_device_between_open_and_close(cuda, oracle):
    """One large copy in, many small in-place steps, one large copy out: results equal the oracle's,
    the host arrays stay untouched while steps are still missing (the write-back of a piece starts
    when its last element has been stepped, the rest goes at the close), and misuse is refused."""
    from flextrain_amd import FlexTrainCPUAdam, _C
    n, shares = 1_000_000, 8
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 16, **HP)
    p, m, v = _host_state(n, seed=31)
    before = p.clone()
    g = (torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    want = _oracle(oracle, p, g, m, v, 4, torch.bfloat16)
    token = eng.open_window(p, m, v)
    per = n // shares
    for k in range(shares):
        if k == shares - 1:
            eng.stream_wait()
            torch.cuda.synchronize()
            assert torch.equal(p, before)  # nothing has come back yet
            assert np.array_equal(half_bits(h)[:k * per], want[3][:k * per])  # but the kernels have run
        sl = slice(k * per, (k + 1) * per)
        eng._step({"step": 4}, h[sl], p[sl], g[sl], m[sl], v[sl], blocking=False)
    eng.stream_wait()
    torch.cuda.synchronize()
    assert np.array_equal(half_bits(h), want[3])
    with pytest.raises(ValueError, match="offset inside the open window"):
        eng._step({"step": 4}, None, p[8:16], g[8:16], m[8:16], v[0:8], blocking=False)
    sp, sm, sv = _host_state(64, seed=1)
    small = eng.open_window(sp[:32], sm[:32], sv[:32])
    with pytest.raises(ValueError, match="inside or entirely outside"):
        eng._step({"step": 4}, None, sp[16:48], g[16:48], sm[16:48], sv[16:48], blocking=False)
    eng.close_window(small)
    with pytest.raises(_C.FtError, match="already belongs"):
        eng.open_window(p, m, v)
    eng.close_window(token)
    eng.synchronize()
    _assert_equal_bits("window", p, m, v, h, want, torch.bfloat16)
    with pytest.raises(_C.FtError, match="not open"):
        eng.close_window(token)

    # windows are reused and grow; a second round on the same memory sees the first one's result
    p2, m2, v2 = _host_state(2 * n, seed=32)
    g2 = (torch.randn(2 * n, device=cuda) * 1e-3).to(torch.bfloat16)
    want2 = _oracle(oracle, p2, g2, m2, v2, 1, None)
    pn, mn, vn, hn = want
    oracle.adam_step(pn, to_np(g), mn, vn, step=5, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                     weight_decay=HP["weight_decay"], g_dtype=CODE[torch.bfloat16], half_out=hn, half_dtype=CODE[torch.bfloat16])
    t1, t2 = eng.open_window(p, m, v), eng.open_window(p2, m2, v2)
    eng._step({"step": 5}, h, p, g, m, v, blocking=False)
    eng._step({"step": 1}, None, p2, g2, m2, v2, blocking=False)
    eng.close_window(t2)
    eng.close_window(t1)
    eng.synchronize()
    _assert_equal_bits("window again", p, m, v, h, (pn, mn, vn, hn), torch.bfloat16)
    _assert_equal_bits("second window", p2, m2, v2, None, want2, None)
    tokens = [eng.open_window(*_host_state(64, seed=s)) for s in range(4)]
    with pytest.raises(_C.FtError, match="windows are open"):
        eng.open_window(*_host_state(64, seed=9))
    for t in tokens:
        eng.close_window(t)
    eng.synchronize()


def test_window_pieces_go_back_as_their_steps_complete(cuda, oracle):
    """A window cut into several pieces: a piece is written back as soon as its last element has been
    stepped, the rest at the close; a piece stepped again after its write-back goes back again.
    Shares in scrambled order, one of them stepped a second time; the host arrays hold the oracle's
    result after the close, whichever way each piece travelled."""
    from flextrain_amd import FlexTrainCPUAdam
    share, shares = 1 << 19, 7
    n = share * shares  # 3.5 Mi elements: four pieces of 0.875 Mi, none aligned with the shares
    with pytest.raises(ValueError, match="refused"):
        FlexTrainCPUAdam(offload_window_piece_elems=4096, **HP)._offload_engine()
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 16, offload_window_piece_elems=1 << 20, **HP)
    p, m, v = _host_state(n, seed=77)
    g = (torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    pn, mn, vn, hn = _oracle(oracle, p, g, m, v, 4, torch.bfloat16)
    again = slice(1 * share, 2 * share)  # share 1 once more, at step 5, after its pieces have gone back
    ps, ms, vs, hs = pn[again].copy(), mn[again].copy(), vn[again].copy(), hn[again].copy()
    oracle.adam_step(ps, to_np(g[again]), ms, vs, step=5, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                     weight_decay=HP["weight_decay"], g_dtype=CODE[torch.bfloat16], half_out=hs, half_dtype=CODE[torch.bfloat16])
    pn[again], mn[again], vn[again], hn[again] = ps, ms, vs, hs
    token = eng.open_window(p, m, v)
    for k in (3, 0, 6, 1, 5, 2, 4):
        sl = slice(k * share, (k + 1) * share)
        eng._step({"step": 4}, h[sl], p[sl], g[sl], m[sl], v[sl], blocking=False)
    eng._step({"step": 5}, h[again], p[again], g[again], m[again], v[again], blocking=False)
    eng.close_window(token)
    eng.synchronize()
    _assert_equal_bits("window in pieces", p, m, v, h, (pn, mn, vn, hn), torch.bfloat16)


def test_write_through_window(cuda, oracle):
    """A window whose steps write their results straight to the host arrays: nothing is copied
    back at the close, the host arrays fill in share by share."""
    from flextrain_amd import FlexTrainCPUAdam
    n, shares = 1_000_000, 5
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 16, **HP)
    p, m, v = _host_state(n, seed=41)
    before = p.clone()
    g = (torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    want = _oracle(oracle, p, g, m, v, 2, torch.bfloat16)
    token = eng.open_window(p, m, v, write_through=True)
    per = n // shares
    for k in range(shares - 1):
        sl = slice(k * per, (k + 1) * per)
        eng._step({"step": 2}, h[sl], p[sl], g[sl], m[sl], v[sl], blocking=False)
    eng.synchronize()
    done = (shares - 1) * per
    assert np.array_equal(p.numpy()[:done].view(np.uint32), want[0][:done].view(np.uint32))  # already on the host
    assert torch.equal(p[done:], before[done:])                                              # not stepped yet
    eng._step({"step": 2}, h[done:], p[done:], g[done:], m[done:], v[done:], blocking=False)
    eng.close_window(token)
    eng.synchronize()
    _assert_equal_bits("write-through window", p, m, v, h, want, torch.bfloat16)


def _control(cuda, skip, grad_mult):
    """A device ft_step_control_t: {u32 skip, f32 grad_mult, f32 grad_norm, f32 clip_coef}."""
    ctl = torch.zeros(4, dtype=torch.float32, device=cuda)
    ctl[1], ctl[3] = grad_mult, 1.0
    ctl.view(torch.int32)[0] = int(skip)
    return ctl


@pytest.mark.parametrize("half_on_host", [True, False])
@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_device_side_skip_and_multiplier_in_every_transfer_mode(cuda, oracle, mode, half_on_host):
    """A control record on an offloaded step. Skipped: the host master state and the low-precision
    copy (in pinned host memory or on the GPU) keep their bits, although the engine's staging slots
    hold another unit's data from the step before (the poison). Not skipped: the record's
    multiplier replaces grad_mult and the result equals the oracle's."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.memory import pinned_empty
    n = 900_001
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 17, offload_slots=2, offload_mode=mode, **HP)

    def half_buffer():
        if half_on_host:
            t = pinned_empty(n, torch.float16)
            t.fill_(3.0)
            return t
        return torch.full((n,), 3.0, dtype=torch.float16, device=cuda)

    # poison: a step on other memory leaves its values in the slots (p, m, v and the copy)
    pp, pm, pv = _host_state(n, seed=90)
    pp.fill_(777.0)
    ph = half_buffer()
    eng._step({"step": 1}, ph, pp, torch.zeros(n, dtype=torch.float16, device=cuda), pm, pv)

    p, m, v = _host_state(n, seed=91)
    g = (torch.randn(n, device=cuda) * 1e-3 * 1024).to(torch.float16)
    h = half_buffer()
    before = tuple(t.clone() for t in (p, m, v))
    eng._step({"step": 7}, h, p, g, m, v, control=_control(cuda, 1, 1.0 / 1024))
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip((p, m, v), before)), "a skipped step changed the master state"
    assert bool((h == 3.0).all()), "a skipped step changed the low-precision copy"

    want = _oracle(oracle, p, g, m, v, 7, torch.float16, grad_mult=1.0 / 1024)
    eng._step({"step": 7}, h, p, g, m, v, grad_mult=55.0, control=_control(cuda, 0, 1.0 / 1024))
    torch.cuda.synchronize()
    _assert_equal_bits(f"control mode={mode} half_on_host={half_on_host}", p, m, v, h, want, torch.float16)


@pytest.mark.parametrize("write_through", [False, True])
def test_device_side_skip_inside_a_window(cuda, oracle, write_through):
    """Shares of a unit stepped inside a window under a control record: a skipped iteration leaves
    host state and copy alone after the close (copy-back and write-through windows), the next one
    steps normally."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.memory import pinned_empty
    n, shares = 800_000, 4
    per = n // shares
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 16, **HP)
    warm = _host_state(n, seed=95)  # the window's device arrays hold this unit's values afterwards
    token = eng.open_window(*warm)
    eng.close_window(token)
    p, m, v = _host_state(n, seed=96)
    before = tuple(t.clone() for t in (p, m, v))
    g = (torch.randn(n, device=cuda) * 1e-3 * 256).to(torch.float16)
    h = pinned_empty(n, torch.bfloat16)
    h.fill_(5.0)
    for skip in (1, 0):
        ctl = _control(cuda, skip, 1.0 / 256)
        want = _oracle(oracle, p, g, m, v, 3, torch.bfloat16, grad_mult=1.0 / 256)
        token = eng.open_window(p, m, v, write_through=write_through)
        for k in range(shares):
            sl = slice(k * per, (k + 1) * per)
            eng._step({"step": 3}, h[sl], p[sl], g[sl], m[sl], v[sl], control=ctl, blocking=False)
        eng.close_window(token)
        eng.synchronize()
        torch.cuda.synchronize()
        if skip:
            assert all(torch.equal(a, b) for a, b in zip((p, m, v), before))
            assert bool((h == 5.0).all())
        else:
            _assert_equal_bits(f"window control write_through={write_through}", p, m, v, h, want, torch.bfloat16)


@pytest.mark.parametrize("mode", [1, 3, 4])
def test_engine_grows_its_chunk_for_long_steps(cuda, oracle, mode):
    """A step that would need more than 96 chunks makes the engine enlarge its chunk first (long
    bursts of copies run slowly); results are unaffected, also for the steps that follow."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(offload_chunk_elems=1 << 12, offload_slots=2, offload_mode=mode, **HP)
    h = None
    for n, t in ((300_000, 1), (1_000_003, 2), (5_000, 3), (2_500_000, 4)):  # 74, then 245 (grows), 1, 3 chunks
        p, m, v = _host_state(n, seed=60 + t)
        g = (torch.randn(n, device=cuda) * 1e-3).to(torch.bfloat16)
        h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
        want = _oracle(oracle, p, g, m, v, t, torch.bfloat16)
        eng._step({"step": t}, h, p, g, m, v)
        _assert_equal_bits(f"grown chunk mode={mode} n={n}", p, m, v, h, want, torch.bfloat16)


CFG5_MIN_LAYERS = 24  # a machine that cannot pin even this much of the 32-layer optimizer fails the test


def test_config5_offloaded_7b_optimizer(cuda, oracle, summary_line):
    """The offloaded Llama-7B optimizer: 32 layers + embedding + lm_head = 6,738,411,520 elements,
    81 GB of pinned fp32 state, 101 chunks of 64 Mi elements, one AdamW step at t = 100. A machine
    that refuses to pin that much in one piece (the measured ones stop near 64 GiB) covers it in two
    passes over the largest slab it can pin: pass 1 streams the elements from 0 up, pass 2 the
    elements up to the end of the optimizer starting at a chunk boundary, so that every chunk 0..100
    is streamed with its true extent and its true element indices (the inputs are a function of the
    element index). Fewer than 24 layers' worth of slab is a failure, not a smaller test.
    Each pass is checked by (1) the oracle on three whole chunks (first, middle, last) and (2)
    bit-equality with the resident kernel on every chunk. The reached size goes into the summary."""
    import gc
    from flextrain_amd import FlexTrainCPUAdam, _C, synth
    from flextrain_amd.memory import pinned_empty
    layer, chunk = 202_383_360, 64 * 1024 * 1024
    n_full = 32 * layer + 2 * 4096 * 32000
    total_chunks = -(-n_full // chunk)
    assert total_chunks == 101
    layers, state = 32, None
    while state is None:
        n = layers * layer + 2 * 4096 * 32000
        try:
            state = tuple(pinned_empty(n, torch.float32) for _ in range(3))
            del_me = pinned_empty(1 << 30, torch.uint8)
            del del_me
        except _C.FtError:
            state = None
            gc.collect()
            layers -= 1
            assert layers >= CFG5_MIN_LAYERS, f"this machine cannot pin {CFG5_MIN_LAYERS} layers of optimizer state"
    P, M, V = state
    G = torch.empty(n, dtype=torch.bfloat16, device=cuda)
    H = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    scratch = torch.empty(chunk, dtype=torch.float32, device=cuda)
    res = FlexTrainCPUAdam(**HP)
    eng = FlexTrainCPUAdam(offload_chunk_elems=chunk, offload_slots=3, **HP)

    # pass 1: elements [0, n); pass 2: [first2, n_full), first2 the first chunk boundary that fits
    first2 = -(-(n_full - n) // chunk) * chunk if n < n_full else n_full
    passes = [(0, n)] + ([(first2, n_full - first2)] if first2 < n_full else [])
    seen_chunks = set()
    for number, (first, count) in enumerate(passes, 1):
        p, m, v, g, h = P[:count], M[:count], V[:count], G[:count], H[:count]
        for lo in range(0, count, chunk):  # element i of the optimizer is a function of i alone
            hi = min(count, lo + chunk)
            k = hi - lo
            p[lo:hi].copy_(synth.fill_(scratch[:k], 0, 0, scale=0.02, first_index=first + lo))
            m[lo:hi].copy_(synth.fill_(scratch[:k], 0, 1, scale=1e-4, first_index=first + lo))
            v[lo:hi].copy_(synth.fill_(scratch[:k], 0, 2, kind=synth.UNIFORM, scale=1e-6, first_index=first + lo))
        synth.fill_(g, 0, 3, scale=1e-3, first_index=first)
        h.zero_()
        torch.cuda.synchronize()
        nchunks = -(-count // chunk)
        probes = sorted({0, nchunks // 2, nchunks - 1})
        want = {}
        for c in probes:
            lo, hi = c * chunk, min(count, (c + 1) * chunk)
            want[c] = _oracle(oracle, p[lo:hi], g[lo:hi], m[lo:hi], v[lo:hi], 100, torch.bfloat16)
        # resident results for every chunk, kept as 64-bit checksums of the raw bits
        sums = []
        for lo in range(0, count, chunk):
            hi = min(count, lo + chunk)
            dp, dm, dv = p[lo:hi].to(cuda), m[lo:hi].to(cuda), v[lo:hi].to(cuda)
            dh = torch.empty(hi - lo, dtype=torch.bfloat16, device=cuda)
            res._step({"step": 100}, dh, dp, g[lo:hi], dm, dv)
            sums.append(tuple(int(t.view(torch.int32).to(torch.int64).sum().item()) for t in (dp, dm, dv)) +
                        (int(dh.view(torch.int16).to(torch.int64).sum().item()),))
        eng._step({"step": 100}, h, p, g, m, v)
        rate = count * 12 / eng.last_offload_ms() / 1e6
        print(f"[cfg5 pass {number}] elements [{first}, {first + count}): {eng.last_offload_ms():.1f} ms, {rate:.1f} GB/s each way", flush=True)
        for c in probes:
            lo, hi = c * chunk, min(count, (c + 1) * chunk)
            _assert_equal_bits(f"cfg5 pass {number} chunk {first // chunk + c}", p[lo:hi], m[lo:hi], v[lo:hi], h[lo:hi], want[c], torch.bfloat16)
        for i, lo in enumerate(range(0, count, chunk)):
            hi = min(count, lo + chunk)
            got = tuple(int(t[lo:hi].to(cuda).view(torch.int32).to(torch.int64).sum().item()) for t in (p, m, v)) + \
                (int(h[lo:hi].view(torch.int16).to(torch.int64).sum().item()),)
            assert got == sums[i], f"pass {number} chunk {i}: streamed and resident results differ"
            if first % chunk == 0 and (hi - lo == chunk or first + hi == n_full):
                seen_chunks.add(first // chunk + i)  # streamed with its true extent
        summary_line(f"cfg5 pass {number}: streamed elements [{first:,}, {first + count:,}) of {n_full:,} "
                     f"({3 * count * 4 / 1e9:.1f} GB pinned state, {nchunks} chunks) at {rate:.1f} GB/s each way")
    assert seen_chunks == set(range(total_chunks)), sorted(set(range(total_chunks)) - seen_chunks)
    summary_line(f"cfg5: {layers} of 32 layers fit one pinned slab; all {total_chunks} chunks of the full optimizer streamed "
                 f"in {len(passes)} pass(es)")
