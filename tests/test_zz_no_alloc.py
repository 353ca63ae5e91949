"""The entry point that allocates nothing: ft_grad_accumulate_static against ft_grad_accumulate and
against the CPU checker.

Called through the C ABI (ctypes on libftadam.so). Same kernels behind both entry points, so
everything is compared bit for bit: the accumulator, the cleared gradients and the statistics
record, on two calls in a row on one GPU, the second with a smaller input (the static scratch still
holds the first call's partials then), plus the size limit and the allocation-free property. The
accumulator is also compared bit for bit with the checker's, and the statistics with its fp64 sum
(count exact, sum of squares within 1e-9 relative), so that the two entry points cannot be wrong
together.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(cuda, n, acc_dtype, g_dtype, seed, bad):
    gen = torch.Generator(device=cuda).manual_seed(seed)
    acc = (torch.randn(n, device=cuda, generator=gen) * 0.01).to(acc_dtype)
    g = (torch.randn(n, device=cuda, generator=gen) * 1e-3 * 64).to(g_dtype)
    for i in bad:
        g[i] = float("inf")
    return acc, g


def _record(cuda):
    return torch.full((2,), -1.0, dtype=torch.float64, device=cuda)  # ft_grad_stats_t, 16 bytes


def _bits(t):
    return t.view(torch.int32 if t.element_size() == 4 else torch.int16)


@pytest.mark.parametrize("acc_dtype,g_dtype", [(torch.float32, torch.bfloat16), (torch.float16, torch.float16)])
def test_static_scratch_entry_point_equals_the_workspace_one(cuda, oracle, acc_dtype, g_dtype):
    from flextrain_amd import _C
    lib = _C.lib()

    def host(t):  # numpy view the checker takes: fp32 as it is, 16-bit types as bit patterns
        c = t.detach().cpu().contiguous()
        return c.numpy().copy() if c.dtype == torch.float32 else c.view(torch.int16).numpy().view(np.uint16).copy()
    stream = _C.current_stream_ptr(cuda)
    code = _C.dtype_code
    # the second call is smaller and starts at an odd element: edge elements on both sides
    calls = [(3_000_003, 0, (5, 1_500_000, 3_000_002)), (700_001, 1, ())]
    for k, (n, off, bad) in enumerate(calls):
        acc, g = _inputs(cuda, n + off, acc_dtype, g_dtype, seed=40 + k, bad=[b + off for b in bad])
        acc2, g2 = acc.clone(), g.clone()
        a, b, a2, b2 = acc[off:], g[off:], acc2[off:], g2[off:]
        acc_host, g_host = host(a), host(b)
        oracle.grad_accumulate(acc_host, code(acc_dtype), g_host, code(g_dtype), scale=0.25, zero_g=True)
        bad_host, sumsq_host = oracle.grad_stats(acc_host, code(acc_dtype), pre_mult=1.0 / 64)
        want, got = _record(cuda), _record(cuda)
        ws_bytes = int(lib.ft_grad_accumulate_workspace_bytes(n))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
        _C.check("ft_grad_accumulate", lib.ft_grad_accumulate(
            a.data_ptr(), code(acc_dtype), b.data_ptr(), code(g_dtype), n, 0.25, 1, 1.0 / 64, want.data_ptr(), 0,
            ws.data_ptr(), ws_bytes, stream))
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(cuda), torch.cuda.mem_get_info(cuda)[0]
        _C.check("ft_grad_accumulate_static", lib.ft_grad_accumulate_static(
            a2.data_ptr(), code(acc_dtype), b2.data_ptr(), code(g_dtype), n, 0.25, 1, 1.0 / 64, got.data_ptr(), 0, stream))
        torch.cuda.synchronize()
        if k > 0:  # the first call on a device may make the runtime load the code object; later ones change nothing
            assert (torch.cuda.memory_allocated(cuda), torch.cuda.mem_get_info(cuda)[0]) == before
        assert torch.equal(_bits(acc), _bits(acc2)), f"call {k}: accumulators differ"
        assert torch.equal(_bits(g), _bits(g2)) and not bool(g2[off:].view(torch.int16).any()), f"call {k}: gradients not cleared alike"
        hw, hg = want.cpu(), got.cpu()
        assert hw.view(torch.int64).tolist() == hg.view(torch.int64).tolist(), f"call {k}: statistics differ: {hw} / {hg}"
        assert int(hg[0:1].view(torch.int64).item()) == len(bad) and float(hg[1]) > 0.0
        # against the CPU checker: the accumulator bit for bit, the statistics of the new accumulator
        assert np.array_equal(host(a2), acc_host), f"call {k}: accumulator differs from the checker's"
        assert int(hg[0:1].view(torch.int64).item()) == bad_host
        assert abs(float(hg[1]) - sumsq_host) <= 1e-9 * sumsq_host, (float(hg[1]), sumsq_host)
    # adding to an existing record, and no statistics at all (no scratch used)
    acc, g = _inputs(cuda, 100_000, acc_dtype, g_dtype, seed=50, bad=())
    acc2, g2 = acc.clone(), g.clone()
    want, got = _record(cuda), _record(cuda)
    want.copy_(hg)
    got.copy_(hg)
    ws = torch.empty(int(lib.ft_grad_accumulate_workspace_bytes(100_000)), dtype=torch.uint8, device=cuda)
    _C.check("ft_grad_accumulate", lib.ft_grad_accumulate(acc.data_ptr(), code(acc_dtype), g.data_ptr(), code(g_dtype), 100_000, 1.0, 0,
                                                          1.0, want.data_ptr(), 1, ws.data_ptr(), ws.numel(), stream))
    _C.check("ft_grad_accumulate_static", lib.ft_grad_accumulate_static(acc2.data_ptr(), code(acc_dtype), g2.data_ptr(), code(g_dtype),
                                                                        100_000, 1.0, 0, 1.0, got.data_ptr(), 1, stream))
    _C.check("ft_grad_accumulate_static", lib.ft_grad_accumulate_static(acc2.data_ptr(), code(acc_dtype), g2.data_ptr(), code(g_dtype),
                                                                        100_000, 0.0, 0, 1.0, None, 0, stream))
    torch.cuda.synchronize()
    assert torch.equal(_bits(acc), _bits(acc2)) and torch.equal(_bits(g), _bits(g2))
    assert want.cpu().view(torch.int64).tolist() == got.cpu().view(torch.int64).tolist()


def test_static_scratch_entry_point_refuses_more_than_its_maximum(cuda):
    from flextrain_amd import _C
    lib = _C.lib()
    t = torch.zeros(16, device=cuda)
    rec = _record(cuda)
    rc = lib.ft_grad_accumulate_static(t.data_ptr(), _C.F32, t.data_ptr(), _C.F32, (1 << 28) + 1, 1.0, 0, 1.0, rec.data_ptr(), 0,
                                       _C.current_stream_ptr(cuda))
    assert rc == -1 and b"at most" in lib.ft_last_error()
    torch.cuda.synchronize()
    assert float(rec[1]) == -1.0  # nothing ran
