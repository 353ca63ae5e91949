"""The statistics pass as one launch (the block that delivers the last partial sum takes the final
sum and the decision) against the same pass as two launches: bit-identical records, whatever the
size, on several streams at once, after the per-stream state has been released, and under HIP graph
capture (where the library falls back to two launches by itself)."""
import numpy as np
import pytest
import torch

from _util import CODE

pytestmark = pytest.mark.gpu


def _raw(buf: torch.Tensor) -> bytes:
    return buf.cpu().numpy().tobytes()


def _decide(lib, g, stats, ctl, ws, accumulate=0, inv_scale=1.0 / 128, max_norm=1.0, stream=None):
    from flextrain_amd import _C
    _C.check("ft_grad_decide", lib.ft_grad_decide(
        g.data_ptr(), CODE[g.dtype], g.numel(), inv_scale, stats.data_ptr(), accumulate, inv_scale, max_norm,
        ctl.data_ptr(), ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
        stream if stream is not None else _C.current_stream_ptr(g.device)))


@pytest.fixture
def lib():
    from flextrain_amd import _C
    L = _C.lib()
    yield L
    L.ft_set_stats_launches(1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_one_launch_equals_two_launches(cuda, lib, dtype):
    """Sizes from nothing but edge elements to thousands of tiles per block, offsets that move the
    vector body, an inf now and then: the 32 bytes of statistics and decision are the same bits."""
    rng = np.random.default_rng(3)
    ws = torch.empty(int(lib.ft_grad_stats_workspace_bytes()), dtype=torch.uint8, device=cuda)
    for k, n in enumerate((1, 5, 8, 9, 1023, 1024, 4096, 4097, 262_144, 1_000_003, 8_388_608 + 11, 50_000_017)):
        offset = int(rng.integers(0, 8))
        buf = (torch.randn(n + offset + 8, device=cuda) * 3).to(dtype)
        g = buf[offset:offset + n]
        if k % 4 == 3:
            g[int(rng.integers(0, n))] = float("inf")
        got = []
        for launches in (1, 2, 1):
            lib.ft_set_stats_launches(launches)
            rec = torch.full((4,), -1.0, dtype=torch.float64, device=cuda)
            _decide(lib, g, rec[0:2], rec[2:4], ws)
            _decide(lib, g, rec[0:2], rec[2:4], ws, accumulate=1)  # the record is added to, not replaced
            got.append(_raw(rec))
        assert got[0] == got[1] == got[2], (dtype, n, offset)


def test_streams_have_their_own_counters(cuda, lib):
    """Passes enqueued on four streams at once, each with the library's own scratch: every stream's
    result equals the one of a pass that ran alone."""
    from flextrain_amd import _C
    n = 30_000_001
    gs = [(torch.randn(n, device=cuda) * (k + 1)).to(torch.bfloat16) for k in range(4)]
    alone = []
    for g in gs:
        rec = torch.zeros(4, dtype=torch.float64, device=cuda)
        _decide(lib, g, rec[0:2], rec[2:4], None)
        alone.append(_raw(rec))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=cuda) for _ in range(4)]
    recs = [torch.zeros(4, dtype=torch.float64, device=cuda) for _ in range(4)]
    torch.cuda.synchronize()
    for _ in range(5):
        for s, g, rec in zip(streams, gs, recs):
            _decide(lib, g, rec[0:2], rec[2:4], None, stream=s.cuda_stream)
    torch.cuda.synchronize()
    for k in range(4):
        assert _raw(recs[k]) == alone[k], k
    # giving the per-stream state back, then using the streams again
    for s in streams:
        _C.check("ft_release_stream_scratch", lib.ft_release_stream_scratch(s.cuda_stream))
    for s, g, rec in zip(streams, gs, recs):
        rec.zero_()
    torch.cuda.synchronize()
    for s, g, rec in zip(streams, gs, recs):
        _decide(lib, g, rec[0:2], rec[2:4], None, stream=s.cuda_stream)
    torch.cuda.synchronize()
    for k in range(4):
        assert _raw(recs[k]) == alone[k], k
    for s in streams:
        _C.check("ft_release_stream_scratch", lib.ft_release_stream_scratch(s.cuda_stream))


def test_capture_takes_the_two_launch_form_and_replays(cuda, lib):
    """A pass recorded into a HIP graph must not share a counter with eager passes: the library
    records the two-launch form. Replays between eager passes on other data give the eager result."""
    n = 3_000_017
    g = (torch.randn(n, device=cuda) * 2).to(torch.float16)
    other = (torch.randn(n // 3, device=cuda) * 5).to(torch.float16)
    ws = torch.empty(int(lib.ft_grad_stats_workspace_bytes()), dtype=torch.uint8, device=cuda)
    ws2 = torch.empty_like(ws)
    eager = torch.zeros(4, dtype=torch.float64, device=cuda)
    _decide(lib, g, eager[0:2], eager[2:4], ws)
    torch.cuda.synchronize()
    rec = torch.zeros(4, dtype=torch.float64, device=cuda)
    side = torch.cuda.Stream(device=cuda)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _decide(lib, g, rec[0:2], rec[2:4], ws)
    scratch = torch.zeros(4, dtype=torch.float64, device=cuda)
    for _ in range(4):
        rec.fill_(-7.0)
        graph.replay()
        _decide(lib, other, scratch[0:2], scratch[2:4], ws2)  # eager work between the replays
        torch.cuda.synchronize()
        assert _raw(rec) == _raw(eager)
