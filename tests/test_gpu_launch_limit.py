"""The cutting of work into launches, exercised on the GPU with an artificially small limit: an
update of a few hundred thousand elements then takes dozens of launches (aligned and relaxed tile
kernels, the many-segment launch, the accumulation pass), and must give the bits it gives in one."""
import numpy as np
import pytest
import torch

from _util import CODE, to_np

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)


@pytest.fixture
def lib():
    from flextrain_amd import _C
    L = _C.lib()
    yield L
    L.ft_set_launch_limit(0)


def _state(cuda, n, seed, off=(0, 0, 0, 0, 0)):
    gen = torch.Generator(device=cuda).manual_seed(seed)
    mk = lambda s, o: (torch.randn(n + 16, device=cuda, generator=gen) * s)[o:o + n]
    p, m, g = mk(0.02, off[0]), mk(1e-4, off[1]), mk(1e-3, off[3]).to(torch.bfloat16)
    v = (torch.rand(n + 16, device=cuda, generator=gen) * 1e-6)[off[2]:off[2] + n]
    h = torch.zeros(n + 16, dtype=torch.bfloat16, device=cuda)[off[4]:off[4] + n]
    return p, g, m, v, h


@pytest.mark.parametrize("limit", [1, 37, 1000])
@pytest.mark.parametrize("offsets", [(0, 0, 0, 0, 0), (3, 3, 3, 3, 3), (0, 0, 0, 0, 1), (1, 2, 1, 1, 1)])
def test_update_in_many_launches(cuda, oracle, lib, limit, offsets):
    """Aligned arrays, arrays cut at a common odd element (edges in the many-segment kernel, which
    falls back to separate launches once its grid would exceed the limit) and arrays whose
    alignments disagree (relaxed tiles)."""
    from flextrain_amd import FlexTrainCPUAdam
    n = 300_003
    eng = FlexTrainCPUAdam(**HP)
    results = []
    for lim in (0, limit):
        lib.ft_set_launch_limit(lim)
        p, g, m, v, h = _state(cuda, n, 5, offsets)
        if lim == 0:
            pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
            hn = np.zeros(n, np.uint16)
            oracle.adam_step(pn, to_np(g), mn, vn, step=9, g_dtype=CODE[g.dtype], half_out=hn, half_dtype=oracle.BF16,
                             **{k: HP[k] for k in ("lr", "betas", "eps", "weight_decay")})
        eng._step({"step": 9}, h, p, g, m, v)
        torch.cuda.synchronize()
        results.append([to_np(t).copy() for t in (p, m, v, h)])
    for a, b in zip(*results):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    for got, want in zip(results[1], (pn, mn, vn, hn)):
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_many_segments_in_many_launches(cuda, lib):
    """40 ragged contexts: with a limit of 50 workgroups per launch the batches hold two or three
    contexts each, and a context of more tiles than that is stepped by launches of its own."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.param_group import StepContext
    rng = np.random.default_rng(1)
    lengths = [int(x) for x in rng.integers(1, 9000, size=39)] + [100_000]
    n = sum(lengths)
    eng = FlexTrainCPUAdam(**HP)
    results = []
    for lim in (0, 50):
        lib.ft_set_launch_limit(lim)
        p, g, m, v, h = _state(cuda, n, 8)
        ctxs, lo = [], 0
        for k, ln in enumerate(lengths):
            group = dict(HP, step=3 + k % 5, weight_decay=0.01 * (k % 3))
            ctxs.append(StepContext(group, h[lo:lo + ln], p[lo:lo + ln], g[lo:lo + ln], [m[lo:lo + ln], v[lo:lo + ln]]))
            lo += ln
        eng._step_many(ctxs)
        torch.cuda.synchronize()
        results.append([to_np(t).copy() for t in (p, m, v, h)])
    for a, b in zip(*results):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.parametrize("acc_dtype", [torch.float32, torch.bfloat16])
def test_accumulation_with_a_capped_grid(cuda, oracle, lib, acc_dtype):
    """The accumulation pass caps its grid at the limit and lets its workgroups stride over the
    tiles: same accumulator, same cleared source, same statistics."""
    from flextrain_amd.loss_scaler import GradientGuard
    n = 500_011
    results = []
    for lim in (0, 13):
        lib.ft_set_launch_limit(lim)
        gen = torch.Generator(device=cuda).manual_seed(2)
        acc = (torch.randn(n, device=cuda, generator=gen) * 0.1).to(acc_dtype)
        g = (torch.randn(n, device=cuda, generator=gen) * 0.1).to(torch.bfloat16)
        guard = GradientGuard(cuda)
        guard.begin()
        guard.accumulate(acc, g, scale=0.5, zero_grads=True, with_stats=True)
        d = guard.decide(max_grad_norm=1.0)
        results.append((to_np(acc).copy(), to_np(g).copy(), d.nonfinite, d.sumsq))
    (a0, g0, bad0, s0), (a1, g1, bad1, s1) = results
    assert np.array_equal(a0.view(np.uint8), a1.view(np.uint8)) and not g1.any() and not g0.any()
    assert bad0 == bad1 == 0
    assert abs(s0 - s1) <= 1e-12 * s0  # the order of the fp64 additions follows the grid
    want = oracle.grad_stats(a1.view(np.uint16) if acc_dtype != torch.float32 else a1, CODE[acc_dtype])[1]
    assert abs(s1 - want) <= 1e-9 * want
