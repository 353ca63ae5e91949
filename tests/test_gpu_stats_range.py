"""The sum of squares over the whole fp32 range: finite gradients whose squares leave the fp32 range
(|g| above 1.8e19 or below 1e-23) must neither turn the norm into inf -- which would make the clip
coefficient 0 and let the update run on zeroed gradients with no overflow flagged -- nor vanish from
it, and an element must contribute the same whether it falls into the vector body of a pass or into
its head / tail. Checked against the CPU checker's fp64 sums (themselves pinned by exact rationals)
through ft_grad_stats / ft_grad_decide and through the statistics of ft_grad_accumulate.

Bar: inf/nan count exact (0 here), norm within 1e-6 relative.
"""
import math

import numpy as np
import pytest
import torch

from _util import CODE, NORM_RTOL, to_np

pytestmark = pytest.mark.gpu

MAGNITUDES = (1e-25, 1e-20, 1e19, 1e20, 3e38)
FLT_MAX = 3.4028234663852886e38


def _bits(t):
    n = to_np(t)
    return n.view(np.uint16) if n.dtype == np.float16 else n


def _planted(cuda, dtype, n, offset, magnitude, where, background):
    """A gradient view of n elements cut `offset` elements into a larger buffer, zero or N(0, 1e-3)
    everywhere except for +-magnitude at positions that lie in the head, the body and the tail."""
    gen = torch.Generator(device=cuda).manual_seed(int(n + offset))
    buf = torch.randn(n + offset + 16, device=cuda, generator=gen) * 1e-3 if background else torch.zeros(n + offset + 16, device=cuda)
    buf = buf.to(dtype)
    g = buf[offset:offset + n]
    pos = {"head": [0, 1], "body": [n // 2, n // 2 + 1, n // 3], "tail": [n - 1, n - 2], "all": [0, 1, n // 3, n // 2, n - 2, n - 1]}[where]
    for k, i in enumerate(pos):
        g[i] = magnitude if k % 2 == 0 else -magnitude
    return g


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("magnitude", MAGNITUDES)
@pytest.mark.parametrize("where", ["head", "body", "tail", "all"])
@pytest.mark.parametrize("background", [False, True])
def test_statistics_pass_over_the_fp32_range(cuda, oracle, dtype, magnitude, where, background):
    from flextrain_amd.loss_scaler import GradientGuard
    n, offset = 300_007, 3
    g = _planted(cuda, dtype, n, offset, magnitude, where, background)
    guard = GradientGuard(cuda)
    guard.begin()
    guard.add(g)
    d = guard.decide(max_grad_norm=1.0)
    bad, sumsq = oracle.grad_stats(_bits(g), CODE[dtype])
    assert bad == 0 and d.nonfinite == 0 and not d.overflow
    assert math.isfinite(d.sumsq) and d.sumsq > 0
    assert abs(math.sqrt(d.sumsq) - math.sqrt(sumsq)) <= NORM_RTOL * math.sqrt(sumsq), (d.sumsq, sumsq)
    assert math.isfinite(d.grad_norm) and math.isfinite(d.clip_coef) and d.clip_coef > 0
    assert np.float32(d.grad_norm) == np.float32(min(math.sqrt(d.sumsq), FLT_MAX))
    assert np.float32(d.clip_coef) == np.float32(min(1.0, 1.0 / (math.sqrt(d.sumsq) + 1e-6)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_contribution_does_not_depend_on_the_position(cuda, oracle, dtype):
    """The same values at other element offsets of the buffer (other splits into head, body and
    tail) give the same sum to fp64 rounding: one element of 1e19 among a million ordinary ones, then
    one of 1e-25 alone."""
    from flextrain_amd.loss_scaler import GradientGuard
    n = 1_000_003
    guard = GradientGuard(cuda)
    for magnitude, background in ((1e19, True), (1e-25, False)):
        gen = torch.Generator(device=cuda).manual_seed(11)
        base = (torch.randn(n, device=cuda, generator=gen) * 1e-3 if background else torch.zeros(n, device=cuda)).to(dtype)
        sums = []
        for offset, where in ((0, 0), (1, 0), (5, n - 1), (7, n // 2), (2, 3)):
            vals = base.clone()
            vals[where] = magnitude
            buf = torch.zeros(n + 16, dtype=dtype, device=cuda)
            buf[offset:offset + n] = vals
            guard.begin()
            guard.add(buf[offset:offset + n])
            sums.append(guard.decide().sumsq)
        want = oracle.grad_stats(_bits(vals), CODE[dtype])[1]
        for s in sums:
            assert abs(s - want) <= 1e-12 * want, (sums, want)


@pytest.mark.parametrize("acc_dtype,g_dtype", [(torch.float32, torch.bfloat16), (torch.float32, torch.float32),
                                               (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("magnitude", MAGNITUDES)
@pytest.mark.parametrize("background", [False, True])
def test_accumulation_statistics_over_the_fp32_range(cuda, oracle, acc_dtype, g_dtype, magnitude, background):
    """The same through the fused accumulation pass: the statistics are those of the new accumulator."""
    from flextrain_amd.loss_scaler import GradientGuard
    n, offset = 300_007, 1
    g = _planted(cuda, g_dtype, n, offset, magnitude, "all", background)
    accbuf = torch.zeros(n + offset + 16, dtype=acc_dtype, device=cuda)
    acc = accbuf[offset:offset + n]
    guard = GradientGuard(cuda)
    guard.begin()
    guard.accumulate(acc, g, with_stats=True)
    d = guard.decide(max_grad_norm=1.0)
    bad, sumsq = oracle.grad_stats(_bits(acc), CODE[acc_dtype])
    assert sumsq > 0  # the planted values reached the accumulator
    assert bad == 0 and d.nonfinite == 0 and not d.overflow
    assert math.isfinite(d.sumsq)
    assert abs(math.sqrt(d.sumsq) - math.sqrt(sumsq)) <= NORM_RTOL * math.sqrt(sumsq), (d.sumsq, sumsq)
    assert math.isfinite(d.grad_norm) and math.isfinite(d.clip_coef) and d.clip_coef > 0


def test_norm_beyond_the_fp32_range_still_clips(cuda, oracle):
    """Two elements of 3e38: the norm (4.2e38) is no fp32 number. The decision is taken in fp64, the
    informational fp32 copy of the norm saturates, and the update that follows multiplies by a
    finite, non-zero coefficient."""
    from flextrain_amd.loss_scaler import GradientGuard
    g = torch.zeros(4096, device=cuda)
    g[7] = 3e38
    g[4000] = -3e38
    guard = GradientGuard(cuda)
    guard.begin()
    guard.add(g)
    d = guard.decide(max_grad_norm=1.0)
    norm = math.sqrt(oracle.grad_stats(to_np(g), 0)[1])
    assert norm > FLT_MAX and not d.overflow
    assert np.float32(d.grad_norm) == np.float32(FLT_MAX)
    assert np.float32(d.clip_coef) == np.float32(1.0 / (norm + 1e-6)) and d.clip_coef > 0
