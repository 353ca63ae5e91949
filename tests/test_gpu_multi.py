"""GPU parity of the many-segments-in-one-launch update (ft_adam_step_multi) against the CPU oracle.

The reference steps a share of a unit context by context, each context one native call with its
group's own hyper-parameters (flextrain/optimizer.py:44-69 over the contexts that
flextrain/param_group.py:365-477 cuts). Here the contexts of a call are one kernel launch; what is
checked is that every element comes out as the oracle's per-context step has it (0 ULP is what the
kernels give; the bars are 2 ULP fp32, 1 ULP for the 16-bit copy), whatever the segment's length,
start offset, group or position in the table, and that nothing outside the segments is touched.
"""
import ctypes

import numpy as np
import pytest
import torch

from _util import CODE, F16, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu

BASE = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)

# 21 ragged segment lengths: below one tile, exactly one, just above, many tiles, empty
LENGTHS = [1, 3, 255, 256, 257, 0, 1000, 4096, 65_536, 5, 300_001, 64, 2049, 7, 1_048_576 + 3, 511, 513, 12, 100_000, 260, 33]


def _groups():
    """Four parameter groups with different learning rate, decay, betas, epsilon, bias correction and
    step count, as a caller with per-group schedules would have them."""
    return [
        dict(BASE, step=100),
        dict(BASE, lr=3e-4, weight_decay=0.0, step=7),
        dict(BASE, lr=5e-5, betas=(0.8, 0.99), eps=1e-6, weight_decay=0.1, step=1),
        dict(BASE, lr=2e-4, bias_correction=False, step=1000),
    ]


def _flat_buffers(cuda, total, g_dtype, half_dtype, seed):
    gen = torch.Generator(device=cuda).manual_seed(seed)
    P = torch.randn(total, device=cuda, generator=gen) * 0.02
    G = (torch.randn(total, device=cuda, generator=gen) * 1e-3).to(g_dtype)
    M = torch.randn(total, device=cuda, generator=gen) * 1e-4
    V = torch.rand(total, device=cuda, generator=gen) * 1e-6
    H = torch.full((total,), 7.0, dtype=half_dtype, device=cuda) if half_dtype is not None else None
    return P, G, M, V, H


def _contexts(P, G, M, V, H, lengths, groups, gap=1):
    """Consecutive segments of the flat buffers with `gap` untouched elements between them, so the
    segments start at every element offset modulo 4 and their neighbours show any stray write."""
    from flextrain_amd.param_group import StepContext
    ctxs, spans, lo = [], [], 2
    for k, n in enumerate(lengths):
        sl = slice(lo, lo + n)
        ctxs.append(StepContext(groups[k % len(groups)], H[sl] if H is not None else None, P[sl], G[sl], [M[sl], V[sl]]))
        spans.append(sl)
        lo += n + gap
    return ctxs, spans


def _oracle_segment(oracle, ctx, half_dtype, grad_mult=1.0, adamw_mode=True):
    g = ctx.gradient
    pn, mn, vn = (to_np(t).copy() for t in (ctx.full_parameter, *ctx.optimizer_states))
    gn = to_np(g)
    if g.dtype == torch.float16:
        gn = gn.view(np.uint16)
    hn = np.zeros(pn.shape[0], np.uint16) if half_dtype is not None else None
    hp = ctx.param_group
    oracle.adam_step(pn, gn, mn, vn, step=hp["step"], lr=hp["lr"], betas=hp["betas"], eps=hp["eps"],
                     weight_decay=hp["weight_decay"], bias_correction=hp["bias_correction"], adamw_mode=adamw_mode,
                     grad_mult=grad_mult, g_dtype=CODE[g.dtype], half_out=hn,
                     half_dtype=CODE[half_dtype] if half_dtype is not None else F16)
    return pn, mn, vn, hn


def _check_segments(tag, ctxs, wants, half_dtype):
    worst = dict(p=0, m=0, v=0, h=0)
    for ctx, (pn, mn, vn, hn) in zip(ctxs, wants):
        if not pn.shape[0]:
            continue
        worst["p"] = max(worst["p"], max_ulp(to_np(ctx.full_parameter), pn))
        worst["m"] = max(worst["m"], max_ulp(to_np(ctx.optimizer_states[0]), mn))
        worst["v"] = max(worst["v"], max_ulp(to_np(ctx.optimizer_states[1]), vn))
        if hn is not None:
            hb = half_bits(ctx.half_parameter)
            worst["h"] = max(worst["h"], max_ulp(hb, hn, bf16=True) if half_dtype == torch.bfloat16
                             else max_ulp(hb.view(np.float16), hn.view(np.float16)))
    print(f"[{tag}] worst ULP distance over {len(ctxs)} segments: {worst}", flush=True)
    assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP, (tag, worst)


def _outside(spans, total, device):
    keep = torch.ones(total, dtype=torch.bool, device=device)
    for sl in spans:
        keep[sl] = False
    return keep


@pytest.mark.parametrize("g_dtype,half_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                                 (torch.float32, None), (torch.float32, torch.bfloat16)])
def test_ragged_segments_with_mixed_groups_in_one_call(cuda, oracle, g_dtype, half_dtype):
    """21 segments (20 live: more than one launch's table of 16 holds), four groups with different
    lr / betas / eps / weight decay / bias correction / step, every start offset modulo 4."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(**BASE)
    total = sum(LENGTHS) + 2 * len(LENGTHS) + 16
    P, G, M, V, H = _flat_buffers(cuda, total, g_dtype, half_dtype, seed=11)
    groups = _groups()
    ctxs, spans = _contexts(P, G, M, V, H, LENGTHS, groups)
    assert {c.full_parameter.data_ptr() % 16 // 4 for c in ctxs if c.full_parameter.numel()} == {0, 1, 2, 3}
    wants = [_oracle_segment(oracle, c, half_dtype) for c in ctxs]
    before = [t.clone() for t in (P, M, V)] + ([H.clone()] if H is not None else [])
    eng._step_many(ctxs)
    torch.cuda.synchronize()
    _check_segments(f"multi g={g_dtype} h={half_dtype}", ctxs, wants, half_dtype)
    keep = _outside(spans, total, cuda)
    for now, old in zip([P, M, V] + ([H] if H is not None else []), before):
        assert torch.equal(now[keep], old[keep]), "an element outside every segment changed"


def test_some_segments_with_a_copy_and_some_without(cuda, oracle):
    """Segments with and without a low-precision copy in one call (two kernel variants behind it)."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(**BASE)
    lengths = [5000, 257, 70_000, 1023, 4]
    total = sum(lengths) + 32
    P, G, M, V, H = _flat_buffers(cuda, total, torch.bfloat16, torch.bfloat16, seed=12)
    ctxs, spans = _contexts(P, G, M, V, H, lengths, _groups())
    for k in (1, 3):
        ctxs[k].half_parameter = None
    wants = [_oracle_segment(oracle, c, torch.bfloat16 if c.half_parameter is not None else None) for c in ctxs]
    eng._step_many(ctxs)
    torch.cuda.synchronize()
    _check_segments("with and without copy", ctxs, wants, torch.bfloat16)
    keep = _outside([spans[k] for k in (0, 2, 4)], total, cuda)
    assert bool((H[keep] == 7.0).all()), "a copy was written for a segment that has none"


@pytest.mark.parametrize("g_dtype", [torch.float32, torch.float16])
def test_equals_one_call_per_context_bit_for_bit(cuda, g_dtype):
    """The contexts of a call stepped together and one at a time (`_step`) give the same bits, over
    three consecutive steps; Adam (not AdamW) mode."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(adamw_mode=False, **BASE)
    total = sum(LENGTHS) + 2 * len(LENGTHS) + 16
    A = _flat_buffers(cuda, total, g_dtype, torch.float16, seed=13)
    B = tuple(t.clone() for t in A)
    groups_a, groups_b = _groups(), _groups()
    ctx_a, _ = _contexts(*A, LENGTHS, groups_a)
    ctx_b, _ = _contexts(*B, LENGTHS, groups_b)
    for it in range(3):
        for ga, gb in zip(groups_a, groups_b):
            ga["step"] += 1
            gb["step"] += 1
        eng._step_many(ctx_a, grad_mult=0.5)
        for c in ctx_b:
            if c.gradient.numel():
                eng._step(c.param_group, c.half_parameter, c.full_parameter, c.gradient, *c.optimizer_states, grad_mult=0.5)
        torch.cuda.synchronize()
        for ta, tb in zip(A, B):
            assert torch.equal(ta.view(torch.int32 if ta.dtype == torch.float32 else torch.int16),
                               tb.view(torch.int32 if tb.dtype == torch.float32 else torch.int16)), it


def test_control_record_applies_to_every_segment(cuda, oracle):
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(**BASE)
    lengths = [3, 9000, 256, 123_457, 1]
    total = sum(lengths) + 32
    P, G, M, V, H = _flat_buffers(cuda, total, torch.float16, torch.bfloat16, seed=14)
    G.mul_(512)
    ctxs, _ = _contexts(P, G, M, V, H, lengths, _groups())
    ctl = torch.zeros(4, dtype=torch.float32, device=cuda)
    ctl[1], ctl[3] = 1.0 / 512, 1.0
    ctl.view(torch.int32)[0] = 1
    before = [t.clone() for t in (P, M, V, H)]
    eng._step_many(ctxs, control=ctl)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip((P, M, V, H), before)), "a skipped call changed something"
    ctl.view(torch.int32)[0] = 0
    wants = [_oracle_segment(oracle, c, torch.bfloat16, grad_mult=1.0 / 512) for c in ctxs]
    eng._step_many(ctxs, grad_mult=99.0, control=ctl)  # the record's multiplier wins
    torch.cuda.synchronize()
    _check_segments("control", ctxs, wants, torch.bfloat16)


def test_segment_whose_arrays_disagree_in_alignment(cuda, oracle):
    """Gradient cut at another element offset than the parameters: that segment goes through
    launches of its own (the tile kernel that assumes element alignment only), its neighbours
    through the table."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.param_group import StepContext
    eng = FlexTrainCPUAdam(**BASE)
    n = 10_000
    P, G, M, V, H = _flat_buffers(cuda, 3 * n + 64, torch.bfloat16, torch.bfloat16, seed=15)
    g = _groups()
    ctxs = [
        StepContext(g[0], H[0:n], P[0:n], G[0:n], [M[0:n], V[0:n]]),
        StepContext(g[1], H[n:2 * n], P[n:2 * n], G[n + 1:2 * n + 1], [M[n:2 * n], V[n:2 * n]]),
        StepContext(g[2], H[2 * n + 8:3 * n + 8], P[2 * n + 8:3 * n + 8], G[2 * n + 8:3 * n + 8], [M[2 * n + 8:3 * n + 8], V[2 * n + 8:3 * n + 8]]),
    ]
    wants = [_oracle_segment(oracle, c, torch.bfloat16) for c in ctxs]
    eng._step_many(ctxs)
    torch.cuda.synchronize()
    _check_segments("misaligned segment", ctxs, wants, torch.bfloat16)


def test_optimizer_step_takes_the_single_launch_path(cuda, oracle, monkeypatch):
    """FlexTrainCPUOptimizer.step over several resident contexts goes through `_step_many` (no
    per-context `_step`), including the device-side overflow decision."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(**BASE)
    lengths = [700, 70_001, 2]
    total = sum(lengths) + 16
    P, G, M, V, H = _flat_buffers(cuda, total, torch.float16, torch.float16, seed=16)
    G.mul_(256)
    ctxs, _ = _contexts(P, G, M, V, H, lengths, _groups())
    wants = [_oracle_segment(oracle, c, torch.float16, grad_mult=1.0 / 256) for c in ctxs]
    calls = []
    real = eng._step
    monkeypatch.setattr(eng, "_step", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    decision = eng.step(ctxs, loss_scale=256.0, check_overflow=True)
    torch.cuda.synchronize()
    assert not calls and not decision.overflow
    _check_segments("optimizer.step", ctxs, wants, torch.float16)
    before = [t.clone() for t in (P, M, V, H)]
    ctxs[1].gradient[5] = float("inf")
    decision = eng.step(ctxs, loss_scale=256.0, check_overflow=True)
    torch.cuda.synchronize()
    assert decision.overflow and decision.nonfinite == 1
    assert all(torch.equal(a, b) for a, b in zip((P, M, V, H), before))


def test_bad_segments_are_refused_before_anything_runs(cuda):
    from flextrain_amd import FlexTrainCPUAdam, _C
    eng = FlexTrainCPUAdam(**BASE)
    lib = _C.lib()
    n = 1024
    P, G, M, V, _ = _flat_buffers(cuda, n, torch.float32, None, seed=17)
    before = P.clone()
    segs = (_C.AdamSegment * 2)()
    for s in segs:
        s.p, s.g, s.m, s.v, s.n = P.data_ptr(), G.data_ptr(), M.data_ptr(), V.data_ptr(), n // 2
        s.step, s.lr, s.beta1, s.beta2, s.eps, s.weight_decay, s.bias_correction, s.grad_mult = 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0
    segs[1].p = P.data_ptr() + 2  # not a float address
    stream = _C.current_stream_ptr(cuda)
    assert lib.ft_adam_step_multi(eng.opt_id, segs, 2, _C.F32, _C.F16, None, stream) == -2
    segs[1].p, segs[1].m = P.data_ptr() + 4 * (n // 2), None
    assert lib.ft_adam_step_multi(eng.opt_id, segs, 2, _C.F32, _C.F16, None, stream) == -1
    assert lib.ft_adam_step_multi(eng.opt_id + 12345, segs, 2, _C.F32, _C.F16, None, stream) == -3
    assert lib.ft_adam_step_multi(eng.opt_id, segs, 2, 9, _C.F16, None, stream) == -1
    assert lib.ft_adam_step_multi(eng.opt_id, None, 0, _C.F32, _C.F16, None, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(P, before), "a refused call must not have stepped its first segment"
    assert ctypes.sizeof(_C.AdamSegment) == 96
