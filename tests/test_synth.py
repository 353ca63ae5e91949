"""The seeded input generator on the host (no GPU needed): pinned known answers, chunk invariance,
an independent float64 evaluation of the same transform, distribution checks, 16-bit rounding."""
import numpy as np
import pytest
import torch

from flextrain_amd import synth

MASK = (1 << 64) - 1


def _mix64(z):
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9 & MASK
    z = (z ^ (z >> 27)) * 0x94D049BB133111EB & MASK
    return z ^ (z >> 31)


def _float64_twin(seed, substream, first_index, n, kind, scale):
    """The same hash with Python integers, the transform with numpy's float64 log / cos."""
    key = _mix64(seed ^ (0x9E3779B97F4A7C15 * (substream + 1) & MASK))
    bits = [_mix64((key + 0xD1342543DE82EF95 * (first_index + i)) & MASK) for i in range(n)]
    k1 = np.array([b >> 40 for b in bits], dtype=np.float64)
    k2 = np.array([(b >> 8) & 0xFFFFFF for b in bits], dtype=np.float64)
    u1 = (k1 + 1.0) / 2.0 ** 24
    if kind == synth.UNIFORM:
        return u1 * scale
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * (k2 + 1.0) / 2.0 ** 24) * scale


def test_known_answers_never_change():
    """Bits pinned at the time the generator was written: inputs made with it stay reproducible."""
    x = synth.fill_(torch.empty(8), 0, 0)
    assert [v & 0xFFFFFFFF for v in x.view(torch.int32).tolist()] == [
        0x3FCBB279, 0x3F7B8C3B, 0xBD8C8887, 0x3ECE797B, 0xBF8024E1, 0x3ECB252C, 0xBED52BA0, 0xBF50C5F7]
    u = synth.fill_(torch.empty(4), 0, 2, kind=synth.UNIFORM, scale=1e-6)
    assert [v & 0xFFFFFFFF for v in u.view(torch.int32).tolist()] == [0x35014475, 0x33948C69, 0x34C1D558, 0x34AD07E4]
    g = synth.fill_(torch.empty(4, dtype=torch.bfloat16), 0, 3, scale=1e-3, first_index=1 << 33)
    assert [v & 0xFFFF for v in g.view(torch.int16).tolist()] == [0x3A7E, 0xB963, 0xBA62, 0x3995]


@pytest.mark.parametrize("kind", [synth.NORMAL, synth.UNIFORM])
@pytest.mark.parametrize("seed,substream,first_index", [(0, 0, 0), (7, 3, 12345), (2 ** 40 + 5, 9, 2 ** 35)])
def test_matches_an_independent_float64_evaluation(kind, seed, substream, first_index):
    """A dropped polynomial term, a wrong octant or a wrong bit field would show here: the fp32
    transform must agree with numpy's float64 log / sqrt / cos on the same hash bits."""
    n = 20000
    got = synth.fill_(torch.empty(n), seed, substream, kind=kind, scale=1.0, first_index=first_index).double().numpy()
    want = _float64_twin(seed, substream, first_index, n, kind, 1.0)
    assert np.max(np.abs(got - want)) < 1e-6
    if kind == synth.UNIFORM:
        assert got.min() > 0.0 and got.max() <= 1.0


def test_chunks_substreams_and_seeds():
    whole = synth.fill_(torch.empty(100_003), 11, 4, scale=0.02)
    pieces = torch.empty(100_003)
    for lo, hi in ((0, 1), (1, 4097), (4097, 70_000), (70_000, 100_003)):
        synth.fill_(pieces[lo:hi], 11, 4, scale=0.02, first_index=lo)
    assert torch.equal(whole, pieces)
    big = synth.fill_(torch.empty((1 << 21) + 3), 11, 4, scale=0.02)  # large fills are cut over threads
    assert torch.equal(big[:100_003], whole)
    assert not torch.equal(whole, synth.fill_(torch.empty(100_003), 11, 5, scale=0.02))
    assert not torch.equal(whole, synth.fill_(torch.empty(100_003), 12, 4, scale=0.02))


def test_distribution():
    from scipy import stats
    x = synth.fill_(torch.empty(1 << 21), 0, 0).double().numpy()
    assert abs(x.mean()) < 3e-3 and abs(x.std() - 1.0) < 3e-3
    assert abs(stats.kurtosis(x)) < 0.02 and abs(stats.skew(x)) < 0.01
    assert stats.kstest(x[:200_000], "norm").pvalue > 1e-3
    assert abs(np.corrcoef(x[:-1], x[1:])[0, 1]) < 3e-3  # neighbours are independent
    u = synth.fill_(torch.empty(1 << 21), 0, 1, kind=synth.UNIFORM).double().numpy()
    assert abs(u.mean() - 0.5) < 1e-3 and stats.kstest(u[:200_000], "uniform").pvalue > 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale", [1.0, 1e-3, 3e-6, 65536.0 * 30])
def test_sixteen_bit_outputs_are_the_fp32_values_rounded_to_nearest_even(dtype, scale):
    """Down to fp16 subnormals and up to overflow (scale 2e6): the same bits as torch's cast."""
    lo = synth.fill_(torch.empty(1 << 16, dtype=dtype), 3, 2, scale=scale)
    ref = synth.fill_(torch.empty(1 << 16), 3, 2, scale=scale).to(dtype)
    assert torch.equal(lo.view(torch.int16), ref.view(torch.int16))


def test_argument_errors():
    with pytest.raises(ValueError):
        synth.fill_(torch.empty(4, dtype=torch.float64), 0, 0)
    with pytest.raises(ValueError):
        synth.fill_(torch.empty(4, 4), 0, 0)
    with pytest.raises(ValueError):
        synth.fill_(torch.empty(4), 0, 0, kind=7)
    assert synth.fill_(torch.empty(0), 0, 0).numel() == 0


def test_committed_full_size_digests_match_the_generator_and_the_oracle_on_the_first_block(oracle):
    """The fixture for the full-size GPU test, re-derived here for its first block of 2^24 elements
    (the update is elementwise, so a prefix of the inputs gives a prefix of the outputs)."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fullsize_digests.json")) as f:
        want = json.load(f)
    n = want["block"]
    weights = (np.arange(n, dtype=np.uint64) % np.uint64(65521)) + np.uint64(1)

    def digest(bits):
        b = bits.astype(np.uint64)
        return [int(b.sum(dtype=np.uint64)), int((b * weights).sum(dtype=np.uint64))]

    p = synth.fill_(torch.empty(n), 0, 0, scale=0.02).numpy()
    m = synth.fill_(torch.empty(n), 0, 1, scale=1e-4).numpy()
    v = synth.fill_(torch.empty(n), 0, 2, kind=synth.UNIFORM, scale=1e-6).numpy()
    g = synth.fill_(torch.empty(n, dtype=torch.bfloat16), 0, 3, scale=1e-3).view(torch.int16).numpy().view(np.uint16)
    for name, bits in (("p", p.view(np.uint32)), ("m", m.view(np.uint32)), ("v", v.view(np.uint32)), ("g", g)):
        assert digest(bits) == want["inputs"][name][0], name
    h = np.zeros(n, np.uint16)
    hyper = dict(want["hyper"])
    hyper["betas"] = tuple(hyper["betas"])
    oracle.adam_step(p, g, m, v, step=want["step"], g_dtype=oracle.BF16, half_out=h, half_dtype=oracle.BF16, **hyper)
    for name, bits in (("p", p.view(np.uint32)), ("m", m.view(np.uint32)), ("v", v.view(np.uint32)), ("h", h)):
        assert digest(bits) == want["outputs"][name][0], name
