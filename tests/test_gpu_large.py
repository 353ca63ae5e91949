"""More than 2**32 elements in one call: element indices, byte offsets and grid sizes beyond 32 bits.

No host can hold an oracle copy of 69 GB, so the check uses that the update is purely elementwise:
every array is one 2**20-element period repeated 4097 times plus three more elements; the first
period is compared with the oracle bit for bit, and every other period with the first one on the
GPU. The statistics must count non-finite values planted beyond element 2**32 and sum 4097 periods.
"""
import math

import numpy as np
import pytest
import torch

from _util import CODE, NORM_RTOL, half_bits, max_ulp_gpu, to_np

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)
PERIOD = 1 << 20
REPEATS = 4097
TAIL = 3
N = PERIOD * REPEATS + TAIL  # 4,296,015,875 > 2**32


def _tiled(pattern: torch.Tensor) -> torch.Tensor:
    out = torch.empty(N, dtype=pattern.dtype, device=pattern.device)
    out[:PERIOD * REPEATS].view(REPEATS, PERIOD).copy_(pattern.unsqueeze(0).expand(REPEATS, PERIOD))
    out[PERIOD * REPEATS:] = pattern[:TAIL]
    return out


def _every_period_equals_the_first(t: torch.Tensor) -> bool:
    bits = t.view(torch.int32 if t.dtype == torch.float32 else torch.int16)
    first = bits[:PERIOD]
    rows = bits[:PERIOD * REPEATS].view(REPEATS, PERIOD)
    for lo in range(0, REPEATS, 256):
        if not torch.equal(rows[lo:lo + 256], first.unsqueeze(0).expand(min(256, REPEATS - lo), PERIOD)):
            return False
    return torch.equal(bits[PERIOD * REPEATS:], first[:TAIL])


def test_step_statistics_and_accumulation_beyond_2_pow_32_elements(cuda, oracle):
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import GradientGuard
    free, _ = torch.cuda.mem_get_info(cuda)
    if free < 90 << 30:
        pytest.skip("needs 90 GB of free device memory")
    assert N > 1 << 32
    gen = torch.Generator(device=cuda).manual_seed(33)
    pat = dict(p=torch.randn(PERIOD, device=cuda, generator=gen) * 0.02,
               m=torch.randn(PERIOD, device=cuda, generator=gen) * 1e-4,
               v=torch.rand(PERIOD, device=cuda, generator=gen) * 1e-6,
               g=(torch.randn(PERIOD, device=cuda, generator=gen) * 1e-3).to(torch.bfloat16))
    p, m, v, g = (_tiled(pat[k]) for k in "pmvg")
    h = torch.zeros(N, dtype=torch.bfloat16, device=cuda)

    # statistics: exact count of values planted past element 2**32, sum over all periods
    guard = GradientGuard(cuda)
    _, period_sumsq = oracle.grad_stats(half_bits(pat["g"]), CODE[torch.bfloat16])
    _, tail_sumsq = oracle.grad_stats(half_bits(pat["g"][:TAIL]), CODE[torch.bfloat16])
    guard.begin()
    guard.add(g)
    d = guard.decide(max_grad_norm=1.0)
    want = REPEATS * period_sumsq + tail_sumsq
    assert d.nonfinite == 0 and abs(math.sqrt(d.sumsq) - math.sqrt(want)) <= NORM_RTOL * math.sqrt(want)
    planted = [(1 << 32) + 5, N - 1, N - PERIOD - 7]
    saved = [g[i].clone() for i in planted]
    for i, bad in zip(planted, (float("inf"), float("nan"), float("-inf"))):
        g[i] = bad
    guard.begin()
    guard.add(g)
    assert guard.decide().nonfinite == 3
    for i, s in zip(planted, saved):
        g[i] = s

    # the update
    eng = FlexTrainCPUAdam(**HP)
    eng._step({"step": 7}, h, p, g, m, v)
    pn, mn, vn = (to_np(pat[k]).copy() for k in "pmv")
    hn = np.zeros(PERIOD, np.uint16)
    oracle.adam_step(pn, half_bits(pat["g"]), mn, vn, step=7, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                     weight_decay=HP["weight_decay"], g_dtype=CODE[torch.bfloat16], half_out=hn, half_dtype=CODE[torch.bfloat16])
    for name, t, want_first in (("p", p, pn), ("m", m, mn), ("v", v, vn), ("h", h, hn)):
        assert max_ulp_gpu(t[:PERIOD], want_first) == 0, name
        assert _every_period_equals_the_first(t), name

    # a second step through the many-contexts launch: two contexts of one group, cut at an odd element
    # beyond 2**31, the second one longer than 2**31 elements and ending beyond 2**32
    from flextrain_amd.param_group import StepContext
    cut = PERIOD * 2049 + 1
    group = {"step": 8}
    eng._step_many([StepContext(group, h[:cut], p[:cut], g[:cut], [m[:cut], v[:cut]]),
                    StepContext(group, h[cut:], p[cut:], g[cut:], [m[cut:], v[cut:]])])
    oracle.adam_step(pn, half_bits(pat["g"]), mn, vn, step=8, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                     weight_decay=HP["weight_decay"], g_dtype=CODE[torch.bfloat16], half_out=hn, half_dtype=CODE[torch.bfloat16])
    for name, t, want_first in (("p", p, pn), ("m", m, mn), ("v", v, vn), ("h", h, hn)):
        assert max_ulp_gpu(t[:PERIOD], want_first) == 0, name
        assert _every_period_equals_the_first(t), name
    del h, m, v

    # accumulation into the (now updated) fp32 array, source cleared, statistics in the same pass
    acc_first = to_np(p[:PERIOD]).copy()
    oracle.grad_accumulate(acc_first, CODE[torch.float32], half_bits(pat["g"]).copy(), CODE[torch.bfloat16], scale=0.5)
    _, period_sumsq = oracle.grad_stats(acc_first, CODE[torch.float32])
    _, tail_sumsq = oracle.grad_stats(acc_first[:TAIL].copy(), CODE[torch.float32])
    guard.begin()
    guard.accumulate(p, g, scale=0.5, zero_grads=True, with_stats=True)
    d = guard.decide()
    want = REPEATS * period_sumsq + tail_sumsq
    assert d.nonfinite == 0 and abs(math.sqrt(d.sumsq) - math.sqrt(want)) <= NORM_RTOL * math.sqrt(want)
    assert max_ulp_gpu(p[:PERIOD], acc_first) == 0 and _every_period_equals_the_first(p)
    for lo in range(0, N, 1 << 30):
        assert not g[lo:lo + (1 << 30)].any()
