"""Several host threads driving the library at once, each on a stream of its own: update steps
through their own optimizer objects and statistics passes with the library's per-(device, stream)
scratch. Every thread's results must equal the oracle's, as if it had run alone."""
import threading

import numpy as np
import pytest
import torch

from _util import CODE, MASTER_ULP, NORM_RTOL, HALF_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu


def test_threads_on_their_own_streams(cuda, oracle):
    from flextrain_amd import FlexTrainCPUAdam, _C
    lib = _C.lib()
    workers, rounds = 4, 25
    results, errors = [None] * workers, []

    def work(k):
        try:
            torch.cuda.set_device(cuda)
            stream = torch.cuda.Stream(device=cuda)
            gen = torch.Generator(device=cuda).manual_seed(100 + k)
            n = 100_003 + 4099 * k
            with torch.cuda.stream(stream):
                p = torch.randn(n, device=cuda, generator=gen) * 0.02
                m = torch.zeros(n, device=cuda)
                v = torch.zeros(n, device=cuda)
                h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
                grads = [(torch.randn(n, device=cuda, generator=gen) * 1e-2).to(torch.float16) for _ in range(rounds)]
                record = torch.zeros(2, dtype=torch.float64, device=cuda)
                pn, mn, vn = to_np(p).copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
                eng = FlexTrainCPUAdam(lr=1e-3 * (k + 1), weight_decay=0.01 * k)
                stats = []
                for t, g in enumerate(grads, 1):
                    # workspace NULL: the library's own scratch for this (device, stream)
                    _C.check("ft_grad_stats", lib.ft_grad_stats(g.data_ptr(), CODE[g.dtype], n, 1.0, record.data_ptr(), 0, None, 0,
                                                                _C.current_stream_ptr(cuda)))
                    stats.append(record.clone())
                    eng._step({"step": t}, h, p, g, m, v)
                stream.synchronize()
            hn = np.zeros(n, np.uint16)
            for t, g in enumerate(grads, 1):
                gn = half_bits(g)
                bad, sumsq = oracle.grad_stats(gn, CODE[g.dtype])
                got = stats[t - 1].cpu()
                assert int(got[0:1].view(torch.int64).item()) == bad == 0
                assert abs(float(got[1]) - sumsq) <= NORM_RTOL * sumsq
                oracle.adam_step(pn, gn, mn, vn, step=t, lr=1e-3 * (k + 1), weight_decay=0.01 * k, g_dtype=CODE[g.dtype],
                                 half_out=hn, half_dtype=CODE[torch.bfloat16])
            results[k] = dict(p=max_ulp(to_np(p), pn), m=max_ulp(to_np(m), mn), v=max_ulp(to_np(v), vn),
                              h=max_ulp(half_bits(h), hn, bf16=True))
        except BaseException as exc:  # surfaces in the main thread
            errors.append((k, repr(exc)))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(workers)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for k, worst in enumerate(results):
        assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP, (k, worst)
