"""The resident mixed-precision step (statistics -> decision -> update) allocates nothing and
clears nothing with memset, so it can be recorded into a HIP graph. The graph is replayed several
times with eager work and synchronisations in between; every replay is checked against the
oracle, including one whose gradients overflow (the device-side decision skips it)."""
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
