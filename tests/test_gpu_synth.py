"""The seeded input generator on the GPU: the kernel must produce exactly the bits the host loop
produces (same functions compiled for both), for every dtype, both distributions, ragged sizes,
element offsets beyond 2^32, and into pinned host memory."""
import pytest
import torch

from flextrain_amd import synth

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.view(torch.int32 if t.dtype == torch.float32 else torch.int16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind,scale", [(synth.NORMAL, 1.0), (synth.NORMAL, 1e-3), (synth.NORMAL, 65.536), (synth.UNIFORM, 1e-6)])
def test_device_fill_equals_host_fill(cuda, dtype, kind, scale):
    for n, first in ((1, 0), (257, 5), (1_000_003, 0), (300_001, (1 << 33) + 7)):
        dev = synth.fill_(torch.empty(n, dtype=dtype, device=cuda), 0, 3, kind=kind, scale=scale, first_index=first)
        host = synth.fill_(torch.empty(n, dtype=dtype), 0, 3, kind=kind, scale=scale, first_index=first)
        assert torch.equal(_bits(dev).cpu(), _bits(host)), (n, first)


def test_large_fill_and_pinned_target(cuda):
    from flextrain_amd.memory import pinned_empty
    n = (1 << 25) + 11
    dev = synth.fill_(torch.empty(n, device=cuda), 5, 1, scale=0.02)
    host = synth.fill_(torch.empty(n), 5, 1, scale=0.02)  # threaded on the host
    assert torch.equal(_bits(dev).cpu(), _bits(host))
    # a kernel can fill pinned host memory directly (this is how offloaded state can be seeded)
    pinned = pinned_empty(1 << 20, torch.float32)
    lib_view = pinned  # host tensor: filled by the host path ...
    synth.fill_(lib_view, 5, 1, scale=0.02)
    assert torch.equal(_bits(pinned), _bits(host[:1 << 20]))
    # ... and a slice of a GPU tensor at an element offset is filled in place without touching its neighbours
    buf = torch.zeros(1000, dtype=torch.bfloat16, device=cuda)
    synth.fill_(buf[3:997], 5, 2, scale=1e-3)
    want = synth.fill_(torch.empty(994, dtype=torch.bfloat16), 5, 2, scale=1e-3)
    assert torch.equal(_bits(buf[3:997]).cpu(), _bits(want)) and not buf[:3].any() and not buf[997:].any()


def _digests(bits, block):
    """[(sum, weighted sum)] per block, modulo 2^64 (the fixture's definition, in torch int64)."""
    mask = (1 << 64) - 1
    weights = (torch.arange(block, device=bits.device, dtype=torch.int64) % 65521) + 1
    out = []
    for lo in range(0, bits.numel(), block):
        b = bits[lo:lo + block].to(torch.int64)
        if bits.dtype == torch.int32:
            b = b & 0xFFFFFFFF
        else:
            b = b & 0xFFFF
        out.append([int(b.sum().item()) & mask, int((b * weights[:b.numel()]).sum().item()) & mask])
    return out


def test_full_size_partition_against_committed_digests(cuda):
    """The 7B-layer partition at full size, inputs from the seeded generator: the GPU's inputs and
    the GPU's results must have the digests that the CPU oracle produced on another machine
    (tests/golden/fullsize_digests.json, written by tests/golden/make_fullsize_digests.py)."""
    import json
    import os
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.memory import allocate_device_arrays
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fullsize_digests.json")) as f:
        want = json.load(f)
    n, block = want["elements"], want["block"]
    p, m, v, g, h = allocate_device_arrays([(n, torch.float32)] * 3 + [(n, torch.bfloat16)] * 2, cuda)
    synth.fill_(p, 0, 0, scale=0.02)
    synth.fill_(m, 0, 1, scale=1e-4)
    synth.fill_(v, 0, 2, kind=synth.UNIFORM, scale=1e-6)
    synth.fill_(g, 0, 3, scale=1e-3)
    for name, t in (("p", p), ("m", m), ("v", v), ("g", g)):
        assert _digests(_bits(t), block) == want["inputs"][name], f"input {name} differs from the generator on the host"
    hyper = dict(want["hyper"])
    hyper["betas"] = tuple(hyper["betas"])
    eng = FlexTrainCPUAdam(**hyper)
    eng._step({"step": want["step"]}, h, p, g, m, v)
    for name, t in (("p", p), ("m", m), ("v", v), ("h", h)):
        got = _digests(_bits(t), block)
        bad = [k for k, (a, b) in enumerate(zip(got, want["outputs"][name])) if a != b]
        assert not bad, f"output {name}: blocks {bad[:8]} of {len(got)} differ from the oracle's digests"
