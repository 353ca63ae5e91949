"""Several host threads drive the library at once, each with its own optimizer object, stream,
statistics buffers and tensors (ctypes releases the GIL inside every call). Registry, per-thread
error strings and launch bookkeeping must hold up; every thread's results are checked against the
oracle."""
import threading

import numpy as np
import pytest
import torch

from _util import CODE, half_bits, to_np

pytestmark = pytest.mark.gpu


def test_four_threads_step_concurrently(cuda, oracle):
    from flextrain_amd import FlexTrainCPUAdam, _C
    from flextrain_amd.loss_scaler import GradientGuard
    n, steps, scale = 300_007, 12, 256.0
    results, errors = {}, []

    def worker(k):
        try:
            torch.cuda.set_device(cuda)
            stream = torch.cuda.Stream(device=cuda)
            hp = dict(lr=1e-4 * (k + 1), weight_decay=0.01 * k, betas=(0.9, 0.999), eps=1e-8)
            eng = FlexTrainCPUAdam(**hp)
            guard = GradientGuard(cuda)
            gen = torch.Generator(device=cuda).manual_seed(100 + k)
            with torch.cuda.stream(stream):
                p = torch.randn(n, device=cuda, generator=gen) * 0.02
                m = torch.zeros(n, device=cuda)
                v = torch.zeros(n, device=cuda)
                h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
                pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
                hn = np.zeros(n, np.uint16)
                for t in range(1, steps + 1):
                    g = (torch.randn(n, device=cuda, generator=gen) * (1e-3 * scale)).to(torch.float16)
                    guard.begin()
                    guard.add(g, loss_scale=scale)
                    ctl = guard.decide_async(loss_scale=scale, max_grad_norm=0.5)
                    eng._step({"step": t}, h, p, g, m, v, control=ctl)
                    d = guard.read()
                    oracle.adam_step(pn, half_bits(g), mn, vn, step=t, grad_mult=d.grad_mult, g_dtype=CODE[torch.float16],
                                     half_out=hn, half_dtype=CODE[torch.bfloat16], **hp)
                    # an error raised in this thread must carry this thread's message
                    if t == 3:
                        try:
                            eng._step({"step": t}, h, p, g[: n - k - 1], m, v)
                        except ValueError as e:
                            assert str(n - k - 1) in str(e), str(e)
                        else:
                            raise AssertionError("length mismatch was accepted")
                stream.synchronize()
                results[k] = all(np.array_equal(to_np(a).view(np.uint32), b.view(np.uint32)) for a, b in ((p, pn), (m, mn), (v, vn))) \
                    and np.array_equal(half_bits(h), hn)
        except BaseException as e:  # noqa: BLE001 - reported to the main thread
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert results == {0: True, 1: True, 2: True, 3: True}
