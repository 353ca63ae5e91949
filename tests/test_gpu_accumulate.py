"""GPU tests of the fused gradient accumulation pass (accumulate [+ scale] [+ clear source]
[+ statistics]) against the oracle: bit-exact accumulators, exact inf/nan counts, norm within 1e-6."""
import math

import numpy as np
import pytest
import torch

from _util import CODE, NORM_RTOL, half_bits, max_ulp_gpu, to_np

pytestmark = pytest.mark.gpu

N_7B_LAYER = 4 * 4096 ** 2 + 3 * 4096 * 11008 + 2 * 4096


def _bits(t):
    n = to_np(t)
    return n.view(np.uint16) if n.dtype == np.float16 else n


@pytest.mark.parametrize("acc_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("g_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale,zero", [(1.0, False), (0.25, True), (0.3, False)])
def test_accumulate_matrix(cuda, oracle, acc_dtype, g_dtype, scale, zero):
    from flextrain_amd.loss_scaler import GradientGuard
    guard = GradientGuard(cuda)
    gen = torch.Generator(device=cuda).manual_seed(3)
    for n, offset in ((1, 0), (5, 3), (1000, 1), (4096, 0), (4099, 1), (70_001, 37), (300_007, 2)):
        A = torch.randn(n + offset + 8, device=cuda, generator=gen).to(acc_dtype)
        G = (torch.randn(n + offset + 8, device=cuda, generator=gen) * 0.1).to(g_dtype)
        a, g = A[offset:offset + n], G[offset:offset + n]
        an, gn = _bits(a).copy(), _bits(g).copy()
        oracle.grad_accumulate(an, CODE[acc_dtype], gn, CODE[g_dtype], scale=scale, zero_g=zero)
        outside = (A[:offset].clone(), A[offset + n:].clone(), G[:offset].clone(), G[offset + n:].clone())
        guard.accumulate(a, g, scale=scale, zero_grads=zero)
        assert max_ulp_gpu(a, an) == 0, (n, offset)
        assert np.array_equal(_bits(g), gn)  # cleared, or untouched
        assert torch.equal(A[:offset], outside[0]) and torch.equal(A[offset + n:], outside[1])
        assert torch.equal(G[:offset], outside[2]) and torch.equal(G[offset + n:], outside[3])


def test_fused_statistics_equal_a_separate_pass(cuda, oracle):
    from flextrain_amd.loss_scaler import GradientGuard
    guard, check = GradientGuard(cuda), GradientGuard(cuda)
    n, scale_loss = 1_000_003, 1024.0
    acc = torch.zeros(n, device=cuda)
    gen = torch.Generator(device=cuda).manual_seed(5)
    micro = [(torch.randn(n, device=cuda, generator=gen) * 0.01 * scale_loss).to(torch.float16) for _ in range(4)]
    micro[2][12345] = float("inf")
    micro[3][0] = float("nan")
    micro[3][n - 1] = float("-inf")
    an = np.zeros(n, np.float32)
    guard.begin()
    for k, g in enumerate(micro):
        last = k == len(micro) - 1
        oracle.grad_accumulate(an, CODE[torch.float32], _bits(g).copy(), CODE[g.dtype], scale=0.25)
        guard.accumulate(acc, g, scale=0.25, zero_grads=True, with_stats=last, loss_scale=scale_loss)
        assert not g.any()
    d = guard.decide(loss_scale=scale_loss, max_grad_norm=1.0)
    assert max_ulp_gpu(acc, an) == 0
    bad, sumsq = oracle.grad_stats(an, CODE[torch.float32], pre_mult=1.0 / scale_loss)
    assert d.nonfinite == bad == 3 and d.overflow
    assert abs(d.sumsq - sumsq) <= 2 * NORM_RTOL * sumsq
    check.begin()
    check.add(acc, loss_scale=scale_loss)
    d2 = check.decide(loss_scale=scale_loss, max_grad_norm=1.0)
    assert d2.nonfinite == d.nonfinite and abs(d2.sumsq - d.sumsq) <= 2 * NORM_RTOL * d.sumsq


@pytest.mark.parametrize("acc_dtype,g_dtype", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.float16)])
@pytest.mark.parametrize("zero", [False, True])
def test_gradients_off_the_accumulators_alignment(cuda, oracle, acc_dtype, g_dtype, zero):
    """acc and g cut at different element offsets of their buffers: g is then read (and cleared)
    through accesses that assume element alignment only; the same bits, statistics included,
    nothing outside the views touched. Lengths that differ are refused."""
    from flextrain_amd.loss_scaler import GradientGuard
    guard = GradientGuard(cuda)
    gen = torch.Generator(device=cuda).manual_seed(11)
    n = 200_003
    for a_off, g_off in ((0, 1), (2, 0), (3, 1), (1, 2), (0, 3)):
        A = torch.randn(n + 8, device=cuda, generator=gen).to(acc_dtype)
        G = (torch.randn(n + 8, device=cuda, generator=gen) * 0.1).to(g_dtype)
        a, g = A[a_off:a_off + n], G[g_off:g_off + n]
        an, gn = _bits(a).copy(), _bits(g).copy()
        oracle.grad_accumulate(an, CODE[acc_dtype], gn, CODE[g_dtype], scale=0.5, zero_g=zero)
        outside = (A[:a_off].clone(), A[a_off + n:].clone(), G[:g_off].clone(), G[g_off + n:].clone())
        guard.begin()
        guard.accumulate(a, g, scale=0.5, zero_grads=zero, with_stats=True)
        d = guard.decide()
        assert max_ulp_gpu(a, an) == 0, (a_off, g_off)
        assert np.array_equal(_bits(g), gn)
        assert torch.equal(A[:a_off], outside[0]) and torch.equal(A[a_off + n:], outside[1])
        assert torch.equal(G[:g_off], outside[2]) and torch.equal(G[g_off + n:], outside[3])
        bad, sumsq = oracle.grad_stats(an, CODE[acc_dtype])
        assert d.nonfinite == bad == 0 and abs(d.sumsq - sumsq) <= 2 * NORM_RTOL * sumsq
    with pytest.raises(ValueError):
        guard.accumulate(torch.zeros(1000, device=cuda), torch.zeros(1001, device=cuda, dtype=torch.bfloat16))  # lengths differ


@pytest.mark.parametrize("g_off", [1, 4, 32])
def test_micro_batches_into_an_accumulator_the_gradients_are_off(cuda, oracle, g_off):
    """Four micro-batches in a row, the gradient buffer off the accumulator's cache lines (by one
    element, by 8 bytes, by 64): it is read through the caches and cleared by every pass, refilled by
    another kernel in between; the accumulator stays bit for bit with the oracle and the buffer ends
    cleared."""
    from flextrain_amd.loss_scaler import GradientGuard
    guard = GradientGuard(cuda)
    n = 1_000_003
    A = torch.zeros(n + 64, device=cuda)
    G = torch.zeros(n + 64, device=cuda, dtype=torch.bfloat16)
    a, g = A[:n], G[g_off:g_off + n]
    an = np.zeros(n, np.float32)
    for mb in range(4):
        g.copy_((torch.randn(n, device=cuda, generator=torch.Generator(device=cuda).manual_seed(100 + mb)) * 0.1).to(torch.bfloat16))
        gn = _bits(g).copy()
        oracle.grad_accumulate(an, CODE[torch.float32], gn, CODE[torch.bfloat16], scale=0.25, zero_g=True)
        guard.begin()
        guard.accumulate(a, g, scale=0.25, zero_grads=True, with_stats=mb == 3)
        assert max_ulp_gpu(a, an) == 0, mb
        assert not bool(G.view(torch.int16).any()), mb
    d = guard.decide()
    bad, sumsq = oracle.grad_stats(an, CODE[torch.float32])
    assert d.nonfinite == bad == 0 and abs(d.sumsq - sumsq) <= 2 * NORM_RTOL * sumsq


def test_accumulate_llama7b_layer(cuda, oracle):
    """Full-size: fp32 accumulator += bf16 gradients over the 7B-layer partition, with the
    statistics of the result gathered in the same pass."""
    from flextrain_amd.loss_scaler import GradientGuard
    n = N_7B_LAYER
    guard = GradientGuard(cuda)
    gen = torch.Generator(device=cuda).manual_seed(9)
    acc = torch.randn(n, device=cuda, generator=gen) * 1e-3
    g = (torch.randn(n, device=cuda, generator=gen) * 1e-3).to(torch.bfloat16)
    an, gn = to_np(acc).copy(), _bits(g).copy()
    oracle.grad_accumulate(an, CODE[torch.float32], gn, CODE[torch.bfloat16], scale=1.0)
    guard.begin()
    guard.accumulate(acc, g, with_stats=True)
    d = guard.decide()
    assert max_ulp_gpu(acc, an) == 0
    bad, sumsq = oracle.grad_stats(an, CODE[torch.float32])
    assert d.nonfinite == bad == 0
    assert abs(math.sqrt(d.sumsq) - math.sqrt(sumsq)) <= NORM_RTOL * math.sqrt(sumsq)


def test_accumulate_with_decision_in_one_call(cuda, oracle):
    """GradientGuard.accumulate(decide=True): accumulate + statistics + decision, then the update of
    the same buffer under that decision (the accumulator's tail is stored with caching stores for
    it); against the oracle, with a clip below 1."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import GradientGuard
    n = 3_000_017
    gen = torch.Generator(device=cuda).manual_seed(77)
    acc = torch.randn(n, device=cuda, generator=gen) * 0.01
    g = (torch.randn(n, device=cuda, generator=gen) * 0.02 * 32).to(torch.float16)
    p = torch.randn(n, device=cuda, generator=gen) * 0.02
    m, v = torch.zeros(n, device=cuda), torch.zeros(n, device=cuda)
    p0 = to_np(p).copy()
    accn = to_np(acc).copy()
    oracle.grad_accumulate(accn, CODE[torch.float32], half_bits(g).copy(), CODE[torch.float16], scale=0.5)
    guard = GradientGuard(cuda)
    guard.begin()
    ctl = guard.accumulate(acc, g, scale=0.5, decide=True, loss_scale=32.0, max_grad_norm=1.0)
    eng = FlexTrainCPUAdam(lr=1e-3, weight_decay=0.01)
    eng._step({"step": 1}, None, p, acc, m, v, control=ctl)
    d = guard.read()
    assert np.array_equal(to_np(acc).view(np.uint32), accn.view(np.uint32))
    bad, sumsq = oracle.grad_stats(accn, CODE[torch.float32], pre_mult=1.0 / 32)
    assert d.nonfinite == bad == 0 and abs(d.sumsq - sumsq) <= 2e-6 * sumsq and d.clip_coef < 1.0
    pn, mn, vn = p0, np.zeros(n, np.float32), np.zeros(n, np.float32)
    oracle.adam_step(pn, accn, mn, vn, step=1, lr=1e-3, weight_decay=0.01, grad_mult=d.grad_mult)
    assert np.array_equal(to_np(p).view(np.uint32), pn.view(np.uint32))
    assert np.array_equal(to_np(m).view(np.uint32), mn.view(np.uint32)) and np.array_equal(to_np(v).view(np.uint32), vn.view(np.uint32))
