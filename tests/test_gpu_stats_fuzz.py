"""Random calls of the statistics and accumulation passes against the CPU oracle: any length around
the tile and alignment boundaries, any start element, every pair of types, with and without clearing,
statistics written or added to a record, the decision taken in the same pass or afterwards, the
caller's workspace, the library's own, or the static one. Accumulators and cleared sources bit for
bit, inf/nan counts exact, sums of squares within 1e-6, decisions as the oracle's formulas give them."""
import ctypes
import os

import numpy as np
import pytest
import torch

from _util import CODE, NORM_RTOL, max_ulp_gpu, to_np

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
SPECIALS = [float("inf"), float("-inf"), float("nan")]


def _bits(t):
    n = to_np(t)
    return n.view(np.uint16) if n.dtype == np.float16 else n


def _raw(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a


def _length(rng):
    kind = int(rng.integers(0, 4))
    if kind == 0:
        return int(rng.integers(1, 40))
    if kind == 1:  # around the point where the vector body moves to a tile boundary
        return int(rng.integers(4096 - 300, 4096 + 600))
    if kind == 2:
        return int(rng.integers(1, 20_000))
    return int(rng.integers(100_000, 600_000))


@pytest.mark.parametrize("seed", range(int(os.environ.get("FT_FUZZ_SEEDS", "24"))))
def test_random_statistics_and_accumulation(cuda, oracle, seed):
    from flextrain_amd import _C
    lib = _C.lib()
    rng = np.random.default_rng(30_000 + seed)
    gen = torch.Generator(device=cuda).manual_seed(seed)
    stream = _C.current_stream_ptr(cuda)
    record = torch.zeros(4, dtype=torch.float64, device=cuda)  # ft_grad_stats_t, then ft_step_control_t
    ws_bytes = int(lib.ft_grad_accumulate_workspace_bytes(700_000))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    bad_total, sumsq_total, started = 0, 0.0, False
    loss_scale = float(rng.choice([1.0, 256.0, 3000.0]))
    inv = float(np.float32(1.0 / loss_scale))
    for call in range(int(rng.integers(2, 7))):
        n, offset = _length(rng), int(rng.integers(0, 300))
        acc_dtype, g_dtype = DTYPES[int(rng.integers(0, 3))], DTYPES[int(rng.integers(0, 3))]
        kind = ["stats", "accumulate", "accumulate_stats"][int(rng.integers(0, 3))]
        workspace = ["caller", "library", "static"][int(rng.integers(0, 3))]
        decide = bool(rng.integers(0, 2)) and kind != "accumulate" and workspace != "static"
        max_norm = float(rng.choice([0.0, 0.5]))
        # fp16 gradients are kept small enough that an accumulator of any type stays finite unless a special value is planted
        G = (torch.randn(n + offset + 8, device=cuda, generator=gen) * 0.05 * min(loss_scale, 256.0)).to(g_dtype)
        A = (torch.randn(n + offset + 8, device=cuda, generator=gen) * 0.5).to(acc_dtype)
        g_offset = offset if rng.integers(0, 3) else int(rng.integers(0, 8))  # now and then g is cut elsewhere than acc
        g, a = G[g_offset:g_offset + n], A[offset:offset + n]
        if rng.integers(0, 4) == 0:
            for _ in range(int(rng.integers(1, 4))):
                g[int(rng.integers(0, n))] = SPECIALS[int(rng.integers(0, 3))]
        gn, an = _bits(g).copy(), _bits(a).copy()
        outside = (A[:offset].clone(), A[offset + n:].clone(), G[:g_offset].clone(), G[g_offset + n:].clone())
        ws_ptr, ws_len = (ws.data_ptr(), ws_bytes) if workspace == "caller" else (None, 0)
        accumulate_flag = 1 if started else 0
        ctl_ptr = record.data_ptr() + 16
        if kind == "stats":
            if decide:
                rc = lib.ft_grad_decide(g.data_ptr(), CODE[g_dtype], n, inv, record.data_ptr(), accumulate_flag, inv, max_norm, ctl_ptr,
                                        ws_ptr, ws_len, stream)
            else:
                rc = lib.ft_grad_stats(g.data_ptr(), CODE[g_dtype], n, inv, record.data_ptr(), accumulate_flag, ws_ptr, ws_len, stream)
            _C.check("statistics", rc)
            bad, sumsq = oracle.grad_stats(gn, CODE[g_dtype], pre_mult=inv)
        else:
            scale, zero = float(rng.choice([1.0, 0.25, 0.3])), bool(rng.integers(0, 2))
            with_stats = kind == "accumulate_stats"
            stats_ptr = record.data_ptr() if with_stats else None
            if workspace == "static":
                rc = lib.ft_grad_accumulate_static(a.data_ptr(), CODE[acc_dtype], g.data_ptr(), CODE[g_dtype], n, scale, int(zero), inv,
                                                   stats_ptr, accumulate_flag, stream)
            elif decide:
                rc = lib.ft_grad_accumulate_decide(a.data_ptr(), CODE[acc_dtype], g.data_ptr(), CODE[g_dtype], n, scale, int(zero), inv,
                                                   stats_ptr, accumulate_flag, inv, max_norm, ctl_ptr, ws_ptr, ws_len, stream)
            else:
                rc = lib.ft_grad_accumulate(a.data_ptr(), CODE[acc_dtype], g.data_ptr(), CODE[g_dtype], n, scale, int(zero), inv,
                                            stats_ptr, accumulate_flag, ws_ptr, ws_len, stream)
            _C.check("accumulation", rc)
            oracle.grad_accumulate(an, CODE[acc_dtype], gn, CODE[g_dtype], scale=scale, zero_g=zero)
            assert max_ulp_gpu(a, an) == 0, (seed, call, n, offset, acc_dtype, g_dtype)
            assert np.array_equal(_raw(_bits(g)), _raw(gn)), (seed, call, "source")  # raw bits: a planted nan equals itself
            if not with_stats:
                assert torch.equal(A[:offset], outside[0]) and torch.equal(A[offset + n:], outside[1])
                continue
            bad, sumsq = oracle.grad_stats(an, CODE[acc_dtype], pre_mult=inv)
        assert torch.equal(A[:offset], outside[0]) and torch.equal(A[offset + n:], outside[1]), (seed, call, "outside acc")
        assert torch.equal(G[:g_offset], outside[2]) and torch.equal(G[g_offset + n:], outside[3]), (seed, call, "outside g")
        bad_total, sumsq_total, started = bad_total + bad, sumsq_total + sumsq, True
        host = record.cpu()
        assert int(host[0:1].view(torch.int64).item()) == bad_total, (seed, call, kind, workspace)
        assert abs(float(host[1]) - sumsq_total) <= 2 * NORM_RTOL * max(sumsq_total, 1e-30), (seed, call, kind, float(host[1]), sumsq_total)
        if decide:
            ctl = host[2:4].view(torch.float32)
            skip = int(host[2:3].view(torch.int32)[0].item())
            assert skip == int(bad_total != 0)
            norm = float(host[1]) ** 0.5
            assert abs(float(ctl[2]) - norm) <= 1e-6 * max(norm, 1e-30)
            clip = oracle.clip_coefficient(norm, max_norm if max_norm > 0 else None)
            assert abs(float(ctl[3]) - clip) <= 1e-6 * clip
            assert np.float32(ctl[1].item()) == np.float32(np.float32(ctl[3].item()) * np.float32(inv))
