"""The resident mixed-precision step (statistics -> decision -> update) allocates nothing and
clears nothing with memset, so it can be recorded into a HIP graph. The graph is replayed several
times with eager work and synchronisations in between; every replay is checked against the
oracle, including one whose gradients overflow (the device-side decision skips it). The same for
the gradient hand-off (fused accumulate / clear / statistics) in front of the step, checked against
the eager calls."""
import numpy as np
import pytest
import torch

from _util import CODE, HALF_ULP, MASTER_ULP, half_bits, max_ulp_gpu, to_np

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)


def test_resident_step_replays_in_a_hip_graph(cuda, oracle):
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import GradientGuard
    n, offset, scale, t = 3_000_001, 1, 1024.0, 5  # odd length at an odd offset: head, body and tail launches
    eng = FlexTrainCPUAdam(**HP)
    guard = GradientGuard(cuda)
    gen = torch.Generator(device=cuda).manual_seed(17)
    bufs = {k: torch.zeros(n + 8, device=cuda) for k in "pmv"}
    p, m, v = (bufs[k][offset:offset + n] for k in "pmv")
    p.copy_(torch.randn(n, device=cuda, generator=gen) * 0.02)
    m.copy_(torch.randn(n, device=cuda, generator=gen) * 1e-4)
    v.copy_(torch.rand(n, device=cuda, generator=gen) * 1e-6)
    g = torch.zeros(n + 8, dtype=torch.float16, device=cuda)[offset:offset + n]
    h = torch.zeros(n + 8, dtype=torch.bfloat16, device=cuda)[offset:offset + n]
    group = {"step": t}

    def fresh_gradient(overflow):
        g.copy_((torch.randn(n, device=cuda, generator=gen) * (1e-3 * scale)).to(torch.float16))
        if overflow:
            g[n // 2] = float("inf")

    def one_step():
        guard.begin()
        guard.add(g, loss_scale=scale)
        ctl = guard.decide_async(loss_scale=scale, max_grad_norm=1.0)
        eng._step(group, h, p, g, m, v, control=ctl)

    # warm up eagerly on a side stream (library buffers, lazy module loads), then capture there
    fresh_gradient(False)
    snapshot = [x.clone() for x in (p, m, v, h)]
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for dst, src in zip((p, m, v, h), snapshot):  # undo the warm-up step
        dst.copy_(src)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        one_step()
    torch.cuda.synchronize()
    for dst, src in zip((p, m, v, h), snapshot):  # capture runs nothing, but be independent of that
        dst.copy_(src)

    pn, mn, vn = (to_np(x).copy() for x in (p, m, v))
    hn = half_bits(h).copy()
    for replay, overflow in enumerate([False, False, True, False, False]):
        fresh_gradient(overflow)
        torch.cuda.synchronize()
        graph.replay()
        d = guard.read()  # reads the statistics and the decision the replay left
        assert d.overflow == overflow
        if not overflow:
            bad, sumsq = oracle.grad_stats(half_bits(g), CODE[torch.float16], pre_mult=1.0 / scale)
            assert bad == 0 and abs(d.sumsq - sumsq) <= 2e-6 * sumsq
            hn = np.zeros(n, np.uint16)
            oracle.adam_step(pn, half_bits(g), mn, vn, step=t, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                             weight_decay=HP["weight_decay"], grad_mult=d.grad_mult, g_dtype=CODE[torch.float16],
                             half_out=hn, half_dtype=CODE[torch.bfloat16])
        worst = dict(p=max_ulp_gpu(p, pn), m=max_ulp_gpu(m, mn), v=max_ulp_gpu(v, vn), h=max_ulp_gpu(h, hn))
        print(f"[graph replay {replay} overflow={overflow}] worst ULP distance: {worst}", flush=True)
        assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP
        # eager work between replays: an unrelated eager step on other buffers through the same library
        q = torch.randn(4099, device=cuda)
        eng._step({"step": 1}, None, q, torch.randn(4099, device=cuda), torch.zeros(4099, device=cuda), torch.zeros(4099, device=cuda))
        torch.cuda.synchronize()
    # the buffers around the slices were never touched
    for k in "pmv":
        assert not bufs[k][:offset].any() and not bufs[k][offset + n:].any()


def test_gradient_hand_off_and_step_replay_in_a_hip_graph(cuda):
    """Two micro-batches folded into an fp32 accumulator by the fused pass (the second one also
    gathers the statistics), the device-side decision, and the update consuming the accumulator:
    recorded once, replayed five times between eager work (one replay with an overflowing
    micro-batch). Every replay must leave exactly what the same calls leave when run eagerly on
    copies of the same state."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import GradientGuard
    n, scale, t = 2_500_003, 512.0, 7
    gen = torch.Generator(device=cuda).manual_seed(23)

    def make_state():
        return dict(p=torch.empty(n, device=cuda), m=torch.empty(n, device=cuda), v=torch.empty(n, device=cuda),
                    h=torch.zeros(n, dtype=torch.bfloat16, device=cuda), acc=torch.zeros(n, device=cuda),
                    g=[torch.zeros(n, dtype=torch.float16, device=cuda) for _ in range(2)])

    live, twin = make_state(), make_state()
    live["p"].copy_(torch.randn(n, device=cuda, generator=gen) * 0.02)
    live["m"].copy_(torch.randn(n, device=cuda, generator=gen) * 1e-4)
    live["v"].copy_(torch.rand(n, device=cuda, generator=gen) * 1e-6)
    eng = FlexTrainCPUAdam(**HP)
    guards = {id(live): GradientGuard(cuda), id(twin): GradientGuard(cuda)}
    group = {"step": t}

    def sequence(s):
        guard = guards[id(s)]
        guard.begin()
        guard.accumulate(s["acc"], s["g"][0], scale=0.5, zero_grads=True)
        guard.accumulate(s["acc"], s["g"][1], scale=0.5, zero_grads=True, with_stats=True, loss_scale=scale)
        ctl = guard.decide_async(loss_scale=scale, max_grad_norm=1.0)
        eng._step(group, s["h"], s["p"], s["acc"], s["m"], s["v"], control=ctl)

    def sync_twin():
        for k in "pmvh":
            twin[k].copy_(live[k])
        twin["acc"].copy_(live["acc"])
        for a, b in zip(twin["g"], live["g"]):
            a.copy_(b)

    def fresh_gradients(overflow):
        live["acc"].zero_()
        for k, g in enumerate(live["g"]):
            g.copy_((torch.randn(n, device=cuda, generator=gen) * (1e-3 * scale)).to(torch.float16))
        if overflow:
            live["g"][1][n - 5] = float("nan")

    # eager warm-up on a side stream (sizes the guard's workspace), undone afterwards, then capture
    fresh_gradients(False)
    snapshot = {k: live[k].clone() for k in "pmvh"}
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sequence(live)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sequence(live)
    torch.cuda.synchronize()
    for k in "pmvh":
        live[k].copy_(snapshot[k])

    for replay, overflow in enumerate([False, True, False, False, False]):
        fresh_gradients(overflow)
        sync_twin()
        torch.cuda.synchronize()
        graph.replay()
        sequence(twin)  # the same calls, eagerly, on the copies
        torch.cuda.synchronize()
        got, want = guards[id(live)].read(), guards[id(twin)].read()
        assert got.overflow == want.overflow == overflow
        assert got.nonfinite == want.nonfinite and got.sumsq == want.sumsq and got.grad_mult == want.grad_mult
        for k in "pmvh":
            assert torch.equal(live[k].view(torch.int32 if k != "h" else torch.int16),
                               twin[k].view(torch.int32 if k != "h" else torch.int16)), f"replay {replay}: {k} differs"
        assert torch.equal(live["acc"], twin["acc"]) or overflow  # NaN != NaN
        assert not live["g"][0].any() and not live["g"][1].any()  # sources cleared by the replay
        if not overflow:
            assert not torch.equal(live["p"], snapshot["p"])
            snapshot["p"] = live["p"].clone()
        print(f"[graph hand-off replay {replay} overflow={overflow}] norm {got.grad_norm:.6g} clip {got.clip_coef:.6g}: equal to eager", flush=True)
        eager_other = torch.randn(4099, device=cuda)  # unrelated eager work through the same library
        guards[id(twin)].begin(); guards[id(twin)].add(eager_other)
        torch.cuda.synchronize()


def test_non_layerwise_step_replays_in_a_hip_graph(cuda):
    """FlexTrainOptimizer.enqueue_step (statistics -> device-side decision -> update of every
    parameter group in one launch -> clearing the gradients) recorded once and replayed, against a
    twin optimizer stepped eagerly on the same gradients: same bits after every replay, also the
    one whose gradients overflow. Static loss scale and a fixed step count: both travel by value."""
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.loss_scaler import LossScaler

    def build():
        torch.manual_seed(3)
        a = torch.nn.Parameter((torch.randn(300, 257, device=cuda) * 0.02).to(torch.float16))
        b = torch.nn.Parameter((torch.randn(1001, device=cuda) * 0.02).to(torch.float16))
        c = torch.nn.Parameter((torch.randn(64, 64, device=cuda) * 0.02).to(torch.float16))
        opt = FlexTrainAdam([{"params": [a, c], "weight_decay": 0.1}, {"params": [b], "weight_decay": 0.0, "lr": 3e-4}],
                            lr=1e-3, loss_scaler=LossScaler(scale=1024.0), max_grad_norm=1.0)
        opt.update_states()
        return opt, (a, b, c)

    eager, eager_params = build()
    replayed, replay_params = build()
    gen = torch.Generator(device=cuda).manual_seed(4)

    def fresh_gradients(overflow):
        for pe, pr in zip(eager_params, replay_params):
            g = (torch.randn(pe.shape, device=cuda, generator=gen) * 0.3 * 1024.0).to(torch.float16)
            if overflow and pe.dim() == 1:
                g[17] = float("nan")
            pe.grad.copy_(g)
            pr.grad.copy_(g)

    fresh_gradients(False)
    assert eager.step() is True and replayed.step() is True  # warm-up: creates the guard and its scratch
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        replayed.enqueue_step()
    torch.cuda.synchronize()
    for replay, overflow in enumerate([False, True, False, False]):
        fresh_gradients(overflow)
        torch.cuda.synchronize()
        graph.replay()
        assert replayed.complete_step() is (not overflow)
        assert eager.step() is (not overflow)
        torch.cuda.synchronize()
        assert replayed.last_grad_norm == eager.last_grad_norm or overflow
        assert torch.equal(replayed._master_para, eager._master_para), replay
        assert torch.equal(replayed._device_para, eager._device_para), replay
        for se, sr in zip(eager.non_layerwise_step_contexts[0].optimizer_states, replayed.non_layerwise_step_contexts[0].optimizer_states):
            assert torch.equal(se, sr), replay
        assert not replayed._device_grad.any()


def test_capturable_step_follows_step_count_learning_rate_and_loss_scale_across_replays(cuda):
    """FlexTrainOptimizer(capturable=True): the groups' scalars and 1/loss_scale live in device
    memory, so ONE recorded enqueue_step() is replayed over real iterations -- the step count
    advances, the learning rate follows a schedule, the dynamic loss scale halves after an overflow --
    and stays bit-equal to a twin optimizer stepped eagerly with by-value scalars."""
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.loss_scaler import DynamicLossScaler

    def build(capturable):
        torch.manual_seed(8)
        a = torch.nn.Parameter((torch.randn(257, 300, device=cuda) * 0.02).to(torch.float16))
        b = torch.nn.Parameter((torch.randn(4099, device=cuda) * 0.02).to(torch.float16))
        groups = [{"params": [a], "weight_decay": 0.1}, {"params": [b], "weight_decay": 0.0, "lr": 3e-4}]
        opt = FlexTrainAdam(groups, lr=1e-3, loss_scaler=DynamicLossScaler(init_scale=2048.0, delayed_shift=1, scale_window=3),
                            max_grad_norm=1.0, capturable=capturable)
        return opt, groups, (a, b)

    eager, eager_groups, eager_params = build(False)
    replayed, replay_groups, replay_params = build(True)
    gen = torch.Generator(device=cuda).manual_seed(9)

    def fresh_gradients(overflow):
        scale = eager.loss_scaler.loss_scale
        assert replayed.loss_scaler.loss_scale == scale
        for pe, pr in zip(eager_params, replay_params):
            g = (torch.randn(pe.shape, device=cuda, generator=gen) * 0.3 * scale).to(torch.float16)
            if overflow and pe.dim() == 1:
                g[5] = float("inf")
            pe.grad.copy_(g)
            pr.grad.copy_(g)

    def advance(iteration):
        for groups, opt in ((eager_groups, eager), (replay_groups, replayed)):
            groups[0]["lr"] = 1e-3 * (0.9 ** iteration)  # a schedule, changed before update_states refreshes the records
            opt.update_states()

    advance(0)
    fresh_gradients(False)
    assert eager.step() is True and replayed.step() is True  # warm-up, eagerly
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    advance(1)
    fresh_gradients(False)
    with torch.cuda.graph(graph, stream=side):
        replayed.enqueue_step()
    torch.cuda.synchronize()
    seen_scales = []
    for iteration, overflow in enumerate([False, True, False, False, False, True, False], start=1):
        if iteration > 1:
            advance(iteration)
            fresh_gradients(overflow)
        seen_scales.append(eager.loss_scaler.loss_scale)
        torch.cuda.synchronize()
        graph.replay()
        assert replayed.complete_step() is (not overflow)
        assert eager.step() is (not overflow)
        torch.cuda.synchronize()
        assert torch.equal(replayed._master_para, eager._master_para), iteration
        assert torch.equal(replayed._device_para, eager._device_para), iteration
        for ce, cr in zip(eager.non_layerwise_step_contexts, replayed.non_layerwise_step_contexts):
            for se, sr in zip(ce.optimizer_states, cr.optimizer_states):
                assert torch.equal(se, sr), iteration
        assert replayed.loss_scaler.loss_scale == eager.loss_scaler.loss_scale
    moves = [b - a for a, b in zip(seen_scales, seen_scales[1:]) if b != a]
    assert any(d < 0 for d in moves) and any(d > 0 for d in moves)  # the scale fell and rose between replays
    assert replay_groups[0]["step"] == 8
