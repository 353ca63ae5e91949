"""GPU tests of the gradient statistics pass, the skip / clip decision and the two mixed-precision
scenarios at full size (overflow skipping on the 7B-layer partition; norm clipping on the
70B-shaped layer).

Bars: inf/nan counts and skip decisions bit-exact; global norm within 1e-6 relative of a float64
reference; state after a skipped step bit-identical; applied steps within the Adam tolerances.
These features have no counterpart in the reference (parity unpinned by it); they are pinned by
the closed forms in the oracle's header.
"""
import math

import numpy as np
import pytest
import torch

from _util import CODE, F16, HALF_ULP, MASTER_ULP, NORM_RTOL, half_bits, max_ulp_gpu, to_np, ulp_histogram_gpu

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)
N_7B_LAYER = 4 * 4096 ** 2 + 3 * 4096 * 11008 + 2 * 4096
N_70B_LAYER = 2 * 8192 ** 2 + 2 * 8192 * 1024 + 3 * 8192 * 28672 + 2 * 8192


def _bits(t):
    n = to_np(t)
    return n.view(np.uint16) if n.dtype == np.float16 else n


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,offset", [(1, 0), (7, 1), (8, 0), (9, 3), (63, 5), (1000, 2), (4096, 0), (100_003, 1), (1_000_000, 7)])
def test_stats_match_oracle(cuda, oracle, dtype, n, offset):
    from flextrain_amd.loss_scaler import GradientGuard
    gen = torch.Generator(device=cuda).manual_seed(n + offset)
    buf = (torch.randn(n + offset + 8, device=cuda, generator=gen) * 3.0).to(dtype)
    g = buf[offset:offset + n]
    guard = GradientGuard(cuda)
    scale = 128.0
    guard.begin()
    guard.add(g, loss_scale=scale)
    d = guard.decide(loss_scale=scale, max_grad_norm=1.0)
    bad, sumsq = oracle.grad_stats(_bits(g), CODE[dtype], pre_mult=1.0 / scale)
    assert d.nonfinite == bad == 0 and not d.overflow
    assert abs(d.sumsq - sumsq) <= 2 * NORM_RTOL * sumsq  # sum of squares: twice the norm's relative bar
    assert abs(math.sqrt(d.sumsq) - math.sqrt(sumsq)) <= NORM_RTOL * math.sqrt(sumsq)
    # the device-side decision equals the closed form evaluated on the host from the same statistics
    clip = np.float32(min(1.0, 1.0 / (math.sqrt(d.sumsq) + 1e-6)))
    assert np.float32(d.clip_coef) == clip
    assert np.float32(d.grad_mult) == np.float32(clip * np.float32(1.0 / scale))
    assert np.float32(d.grad_norm) == np.float32(math.sqrt(d.sumsq))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_nonfinite_is_counted_exactly(cuda, oracle, dtype):
    from flextrain_amd.loss_scaler import GradientGuard
    n = 2_000_003
    gen = torch.Generator(device=cuda).manual_seed(5)
    g = torch.randn(n, device=cuda, generator=gen).to(dtype)
    rng = np.random.default_rng(5)
    pos = rng.choice(n, size=9, replace=False)
    pos[0], pos[1] = 0, n - 1  # first and last element: the scalar head / tail of the pass
    kinds = [float("inf"), float("-inf"), float("nan")]
    for i, k in enumerate(pos):
        g[int(k)] = kinds[i % 3]
    guard = GradientGuard(cuda)
    guard.begin()
    guard.add(g)
    d = guard.decide()
    bad, sumsq = oracle.grad_stats(_bits(g), CODE[dtype])
    assert d.overflow and d.nonfinite == bad == 9
    assert abs(d.sumsq - sumsq) <= 2 * NORM_RTOL * sumsq  # finite elements still summed
    ctl = guard.control.cpu()
    assert int(ctl.view(torch.int32)[0]) == 1  # skip flag


def test_accumulation_over_several_buffers(cuda, oracle):
    """A step whose gradients live in several buffers (param groups, units) shares one decision."""
    from flextrain_amd.loss_scaler import GradientGuard
    gen = torch.Generator(device=cuda).manual_seed(21)
    parts = [(torch.randn(n, device=cuda, generator=gen) * 0.1).to(dt)
             for n, dt in ((10_001, torch.bfloat16), (77, torch.float32), (500_000, torch.float16))]
    guard = GradientGuard(cuda)
    guard.begin()
    for part in parts:
        guard.add(part)
    d = guard.decide(max_grad_norm=0.5)
    want = sum(oracle.grad_stats(_bits(part), CODE[part.dtype])[1] for part in parts)
    assert abs(d.sumsq - want) <= 2 * NORM_RTOL * want
    assert d.clip_coef < 1.0
    guard.begin()  # a new step forgets the old sums
    guard.add(parts[1])
    d2 = guard.decide()
    assert abs(d2.sumsq - oracle.grad_stats(_bits(parts[1]), 0)[1]) <= 2 * NORM_RTOL * d2.sumsq


def _apply_oracle(oracle, pn, mn, vn, g, t, grad_mult, half_dtype):
    hn = np.zeros(pn.shape[0], dtype=np.uint16)
    oracle.adam_step(pn, _bits(g), mn, vn, step=t, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                     weight_decay=HP["weight_decay"], grad_mult=grad_mult, g_dtype=CODE[g.dtype],
                     half_out=hn, half_dtype=CODE[half_dtype])
    return hn


def _check_state(tag, p, m, v, h, pn, mn, vn, hn):
    hist = dict(p=ulp_histogram_gpu(p, pn), m=ulp_histogram_gpu(m, mn), v=ulp_histogram_gpu(v, vn), h=ulp_histogram_gpu(h, hn))
    worst = {k: x["max"] for k, x in hist.items()}
    print(f"[{tag}] ULP distance histograms (elements at 0 / 1 / 2 / more): "
          + "; ".join(f"{k}: {x['0']} / {x['1']} / {x['2']} / {x['>2']}" for k, x in hist.items()), flush=True)
    assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP, (tag, worst)


@pytest.mark.parametrize("path", ["host_decision", "device_decision"])
def test_config3_overflow_skips_and_scale_trace(cuda, oracle, path):
    """7B-layer partition, fp16 grads = N(0,1e-3) x loss scale, 8 steps, inf/nan injected at three
    seeded positions on steps 3 and 6: exactly those steps are skipped (state bit-identical), the
    scale goes 65536 -> 32768 -> 16384 (hysteresis 1), t advances only on applied steps, and every
    applied step equals AdamW on the unscaled gradients. Two ways through: the decision read back
    before the update is launched, and -- as bench.py and the optimizer front ends run it -- statistics
    and decision in one fused pass, the update launched blind under the device-side record, the
    record read afterwards."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import DynamicLossScaler, GradientGuard
    n = N_7B_LAYER
    eng = FlexTrainCPUAdam(**HP)
    scaler = DynamicLossScaler(init_scale=65536.0, delayed_shift=1)
    guard = GradientGuard(cuda)
    gen = torch.Generator(device=cuda).manual_seed(0)
    p = torch.randn(n, device=cuda, generator=gen) * 0.02
    m = torch.randn(n, device=cuda, generator=gen) * 1e-4
    v = torch.rand(n, device=cuda, generator=gen) * 1e-6
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
    hn = half_bits(h).copy()
    rng = np.random.default_rng(0)
    group = {"step": 0}
    seen_scales, skipped = [], []
    for it in range(1, 9):
        scale = float(scaler.loss_scale)
        seen_scales.append(scale)
        g = (torch.randn(n, device=cuda, generator=gen) * (1e-3 * scale)).to(torch.float16)
        if it in (3, 6):
            for k, kind in zip(rng.choice(n, size=3, replace=False), (float("inf"), float("-inf"), float("nan"))):
                g[int(k)] = kind
        guard.begin()
        if path == "device_decision":
            before = [t.clone() for t in (p, m, v, h)] if it in (3, 6) else None
            ctl = guard.add_and_decide(g, loss_scale=scale)
            eng._step({"step": group["step"] + 1}, h, p, g, m, v, control=ctl)  # launched without knowing the decision
            d = guard.read()
            scaler.update_scale(d.overflow)
            if d.overflow:
                skipped.append(it)
                for now, was in zip((p, m, v, h), before):
                    assert torch.equal(now, was)
                assert d.nonfinite == 3
                continue
            group["step"] += 1
            assert d.grad_mult == 1.0 / scale
        else:
            guard.add(g, loss_scale=scale)
            d = guard.decide(loss_scale=scale)
            scaler.update_scale(d.overflow)
            if d.overflow:
                skipped.append(it)
                before = [t.clone() for t in (p, m, v, h)]
                # even if a caller launches the update with the device-side decision, nothing moves
                eng._step({"step": group["step"] + 1}, h, p, g, m, v, control=guard.control)
                for now, was in zip((p, m, v, h), before):
                    assert torch.equal(now, was)
                assert d.nonfinite == 3
                continue
            group["step"] += 1
            assert d.grad_mult == 1.0 / scale  # power of two: exact
            eng._step(group, h, p, g, m, v, grad_mult=d.grad_mult)
        hn = _apply_oracle(oracle, pn, mn, vn, g, group["step"], d.grad_mult, torch.bfloat16)
        if it in (1, 4, 8):
            _check_state(f"cfg3 it={it} t={group['step']}", p, m, v, h, pn, mn, vn, hn)
    assert skipped == [3, 6]
    assert group["step"] == 6
    assert seen_scales == [65536.0] * 3 + [32768.0] * 3 + [16384.0] * 2
    assert seen_scales + [float(scaler.loss_scale)] == oracle.loss_scale_trace(
        [i in (3, 6) for i in range(1, 9)], 65536.0, delayed_shift=1)


def test_config4_clip_llama70b_layer(cuda, oracle):
    """855,654,400 elements, bf16 grads ~N(0, 5e-3): norm ~146, clipped to 1.0 with an
    fp32-accumulated norm, then AdamW at t = 1000."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import GradientGuard
    n = N_70B_LAYER
    assert n == 855_654_400
    eng = FlexTrainCPUAdam(**HP)
    gen = torch.Generator(device=cuda).manual_seed(4)
    p = torch.randn(n, device=cuda, generator=gen) * 0.02
    m = torch.randn(n, device=cuda, generator=gen) * 1e-4
    v = torch.rand(n, device=cuda, generator=gen) * 1e-6
    g = (torch.randn(n, device=cuda, generator=gen) * 5e-3).to(torch.bfloat16)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()

    guard = GradientGuard(cuda)
    guard.begin()
    guard.add(g)
    d = guard.decide(max_grad_norm=1.0)
    bad, sumsq = oracle.grad_stats(_bits(g), CODE[g.dtype])
    norm64 = math.sqrt(sumsq)
    print(f"[cfg4] norm gpu={d.grad_norm!r} fp64={norm64!r} rel={(math.sqrt(d.sumsq) - norm64) / norm64:.3e}", flush=True)
    assert bad == 0 and not d.overflow
    assert abs(math.sqrt(d.sumsq) - norm64) <= NORM_RTOL * norm64
    assert abs(d.grad_norm - norm64) <= NORM_RTOL * norm64
    assert 140.0 < d.grad_norm < 152.0
    assert np.float32(d.clip_coef) == np.float32(1.0 / (math.sqrt(d.sumsq) + 1e-6))
    assert abs(d.clip_coef - oracle.clip_coefficient(norm64, 1.0)) <= 2 * NORM_RTOL * d.clip_coef

    eng._step({"step": 1000}, h, p, g, m, v, control=guard.control)
    hn = _apply_oracle(oracle, pn, mn, vn, g, 1000, d.grad_mult, torch.bfloat16)
    _check_state("cfg4", p, m, v, h, pn, mn, vn, hn)


def test_step_keywords_check_overflow_and_clip(cuda, oracle):
    """`FlexTrainCPUOptimizer.step(contexts, loss_scale=, max_grad_norm=, check_overflow=)`: the
    statistics cover the gradients of all contexts together, an inf in one context stops every
    context, and an applied step equals the oracle with the returned multiplier."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.param_group import StepContext
    eng = FlexTrainCPUAdam(**HP)
    gen = torch.Generator(device=cuda).manual_seed(21)
    scale = 256.0
    sizes = (70_001, 0, 12_345)
    ctxs, host = [], []
    for n in sizes:
        p = torch.randn(n, device=cuda, generator=gen) * 0.02
        m = torch.randn(n, device=cuda, generator=gen) * 1e-4
        v = torch.rand(n, device=cuda, generator=gen) * 1e-6
        g = (torch.randn(n, device=cuda, generator=gen) * (5e-2 * scale)).to(torch.float16)
        h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
        ctxs.append(StepContext({"step": 1}, h, p, g, [m, v]))
        host.append([to_np(p).copy(), to_np(m).copy(), to_np(v).copy()])

    # plain reference behaviour: no keywords, nothing returned
    assert eng.step([]) is None

    # overflow in the LAST context: nothing moves anywhere
    ctxs[2].gradient[17] = float("inf")
    before = [[t.clone() for t in (c.full_parameter, *c.optimizer_states, c.half_parameter)] for c in ctxs]
    d = eng.step(ctxs, loss_scale=scale, check_overflow=True)
    assert d.overflow and d.nonfinite == 1
    for c, was in zip(ctxs, before):
        for now, old in zip((c.full_parameter, *c.optimizer_states, c.half_parameter), was):
            assert torch.equal(now, old)

    # repaired gradient: the step is applied with the clip of the joint norm
    ctxs[2].gradient[17] = 0.0
    d = eng.step(ctxs, loss_scale=scale, max_grad_norm=1.0, check_overflow=True)
    assert not d.overflow
    sumsq = sum(oracle.grad_stats(_bits(c.gradient), CODE[torch.float16], pre_mult=1.0 / scale)[1]
                for c in ctxs if c.gradient.numel())
    assert abs(d.grad_norm - math.sqrt(sumsq)) <= 2 * NORM_RTOL * math.sqrt(sumsq)
    assert d.clip_coef < 0.1  # norm ~ 0.05 * sqrt(82k) >> 1
    for c, (pn, mn, vn) in zip(ctxs, host):
        if not c.gradient.numel():
            continue
        hn = _apply_oracle(oracle, pn, mn, vn, c.gradient, 1, d.grad_mult, torch.bfloat16)
        _check_state("step keywords", c.full_parameter, c.optimizer_states[0], c.optimizer_states[1],
                     c.half_parameter, pn, mn, vn, hn)

    # loss_scale alone: a host-side multiplier, no statistics, nothing returned
    pn, mn, vn = host[0]
    assert eng.step(ctxs[0], loss_scale=scale) is None
    hn = _apply_oracle(oracle, pn, mn, vn, ctxs[0].gradient, 1, 1.0 / scale, torch.bfloat16)
    _check_state("loss_scale only", ctxs[0].full_parameter, *ctxs[0].optimizer_states, ctxs[0].half_parameter, pn, mn, vn, hn)

    with pytest.raises(ValueError):
        eng.step(ctxs, check_overflow=True, grad_mult=0.5)


def test_library_owned_scratch_is_per_stream(cuda, oracle):
    """ft_grad_stats and ft_grad_accumulate without a workspace (the library keeps one per device
    and stream): calls interleaved on two streams over different gradients, growing the scratch in
    between, must each report their own statistics."""
    from flextrain_amd import _C
    lib = _C.lib()
    streams = [torch.cuda.Stream(device=cuda) for _ in range(2)]
    sizes = [(3_000_001, 2_000_000), (5_000_003, 700_001)]
    gen = torch.Generator(device=cuda).manual_seed(21)
    grads = [[(torch.randn(n, device=cuda, generator=gen) * (k + 1)).to(torch.bfloat16) for n in sizes[k]] for k in range(2)]
    accs = [[torch.zeros(n, device=cuda) for n in sizes[k]] for k in range(2)]
    grads[1][0][12] = float("inf")
    records = [[torch.zeros(2, dtype=torch.float64, device=cuda) for _ in range(3)] for _ in range(2)]
    torch.cuda.synchronize()
    for round_ in range(2):
        for k, stream in enumerate(streams):
            g = grads[k][round_]
            _C.check("ft_grad_stats", lib.ft_grad_stats(g.data_ptr(), _C.BF16, g.numel(), 0.5, records[k][round_].data_ptr(), 0,
                                                        None, 0, stream.cuda_stream))
    for k, stream in enumerate(streams):  # the accumulation pass needs a larger scratch: the buffers grow
        g, acc = grads[k][0], accs[k][0]
        _C.check("ft_grad_accumulate", lib.ft_grad_accumulate(acc.data_ptr(), _C.F32, g.data_ptr(), _C.BF16, g.numel(), 1.0, 0, 0.5,
                                                              records[k][2].data_ptr(), 0, None, 0, stream.cuda_stream))
    torch.cuda.synchronize()
    for k in range(2):
        for round_ in range(2):
            bad, sumsq = oracle.grad_stats(_bits(grads[k][round_]), CODE[torch.bfloat16], pre_mult=0.5)
            got = records[k][round_].cpu()
            assert int(got[0:1].view(torch.int64).item()) == bad == (1 if (k, round_) == (1, 0) else 0)
            assert abs(float(got[1]) - sumsq) <= 2 * NORM_RTOL * sumsq
        bad, sumsq = oracle.grad_stats(_bits(grads[k][0]), CODE[torch.bfloat16], pre_mult=0.5)
        got = records[k][2].cpu()  # acc was zero: the accumulated values are the gradients, widened
        assert int(got[0:1].view(torch.int64).item()) == bad and abs(float(got[1]) - sumsq) <= 2 * NORM_RTOL * sumsq


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_fused_decision_equals_statistics_then_control(cuda, dtype):
    """ft_grad_decide / ft_grad_accumulate_decide against ft_grad_stats / ft_grad_accumulate followed
    by ft_grad_control: the same record and the same decision, bit for bit, also when the pass adds
    to an existing record and when an inf is present."""
    from flextrain_amd import _C
    from flextrain_amd.loss_scaler import GradientGuard
    lib = _C.lib()
    n = 1_234_567
    gen = torch.Generator(device=cuda).manual_seed(31)
    grads = [(torch.randn(n, device=cuda, generator=gen) * 37.0).to(dtype) for _ in range(3)]
    grads[2][n // 3] = float("inf")
    a, b = GradientGuard(cuda), GradientGuard(cuda)
    for g in grads:  # the record grows over the three buffers; decide after each
        a.add(g, loss_scale=64.0)
        a.decide_async(loss_scale=64.0, max_grad_norm=2.0)
        b.add_and_decide(g, loss_scale=64.0, max_grad_norm=2.0)
        torch.cuda.synchronize()
        assert a._buf.cpu().view(torch.int64).tolist() == b._buf.cpu().view(torch.int64).tolist()
    assert b.read().overflow and b.read().nonfinite == 1
    # the accumulation pass
    acc_a, acc_b = torch.zeros(n, device=cuda), torch.zeros(n, device=cuda)
    ws = torch.empty(int(lib.ft_grad_accumulate_workspace_bytes(n)), dtype=torch.uint8, device=cuda)
    rec_a, rec_b = torch.zeros(4, dtype=torch.float64, device=cuda), torch.zeros(4, dtype=torch.float64, device=cuda)
    stream = _C.current_stream_ptr(cuda)
    g = grads[0]
    code = _C.dtype_code(dtype)
    _C.check("ft_grad_accumulate", lib.ft_grad_accumulate(acc_a.data_ptr(), _C.F32, g.data_ptr(), code, n, 0.5, 0, 1 / 64.0,
                                                          rec_a.data_ptr(), 0, ws.data_ptr(), ws.numel(), stream))
    _C.check("ft_grad_control", lib.ft_grad_control(rec_a.data_ptr(), 1 / 64.0, 2.0, rec_a[2:].data_ptr(), stream))
    _C.check("ft_grad_accumulate_decide", lib.ft_grad_accumulate_decide(
        acc_b.data_ptr(), _C.F32, g.data_ptr(), code, n, 0.5, 0, 1 / 64.0, rec_b.data_ptr(), 0, 1 / 64.0, 2.0, rec_b[2:].data_ptr(),
        ws.data_ptr(), ws.numel(), stream))
    torch.cuda.synchronize()
    assert torch.equal(acc_a, acc_b) and rec_a.cpu().view(torch.int64).tolist() == rec_b.cpu().view(torch.int64).tolist()
    assert float(rec_b.cpu()[2:].view(torch.float32)[3]) < 1.0  # clipped: the decision really was taken
