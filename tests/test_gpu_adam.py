"""GPU parity of the fused Adam/AdamW kernel against the CPU oracle (through the C ABI).

Bars: fp32 p/m/v within 2 ULP of the oracle, 16-bit recast within 1 ULP of its format, on
identical seeded inputs. The kernels are written to be bit-exact; the tests print the worst
distance they saw so that a drift from 0 is visible even while inside the tolerance.
"""
import numpy as np
import pytest
import torch

from _util import BF16, CODE, F16, F32, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np, ulp_histogram_gpu

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)


def _engine(**kw):
    from flextrain_amd import FlexTrainCPUAdam
    return FlexTrainCPUAdam(**kw)


def _gen(n, device, seed, g_dtype=torch.float32, g_std=1e-3, zero_state=False):
    gen = torch.Generator(device=device).manual_seed(seed)
    p = torch.randn(n, device=device, generator=gen) * 0.02
    g = (torch.randn(n, device=device, generator=gen) * g_std).to(g_dtype)
    if zero_state:
        m = torch.zeros(n, device=device)
        v = torch.zeros(n, device=device)
    else:
        m = torch.randn(n, device=device, generator=gen) * 1e-4
        v = torch.rand(n, device=device, generator=gen) * 1e-6
    return p, g, m, v


def _oracle_step(oracle, p, g, m, v, *, step, half_dtype=None, adamw_mode=True, grad_mult=1.0, hp=HP):
    """Runs the oracle on host copies; returns numpy (p, m, v, half-bits-or-None)."""
    pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
    gn = to_np(g)
    if g.dtype == torch.float16:
        gn = gn.view(np.uint16)
    hn = np.zeros(pn.shape[0], dtype=np.uint16) if half_dtype is not None else None
    oracle.adam_step(pn, gn, mn, vn, step=step, lr=hp["lr"], betas=hp["betas"], eps=hp["eps"],
                     weight_decay=hp["weight_decay"], bias_correction=hp["bias_correction"],
                     adamw_mode=adamw_mode, grad_mult=grad_mult, g_dtype=CODE[g.dtype], half_out=hn,
                     half_dtype=CODE[half_dtype] if half_dtype is not None else F16)
    return pn, mn, vn, hn


def _compare(tag, got, want, half_dtype=None):
    p, m, v, h = got
    pn, mn, vn, hn = want
    worst = {k: max_ulp(to_np(a), b) for k, a, b in (("p", p, pn), ("m", m, mn), ("v", v, vn))}
    if h is not None:
        worst["h"] = max_ulp(half_bits(h), hn, bf16=True) if half_dtype == torch.bfloat16 \
            else max_ulp(half_bits(h).view(np.float16), hn.view(np.float16))
    print(f"[{tag}] worst ULP distance: {worst}", flush=True)
    assert worst["p"] <= MASTER_ULP and worst["m"] <= MASTER_ULP and worst["v"] <= MASTER_ULP, (tag, worst)
    if h is not None:
        assert worst["h"] <= HALF_ULP, (tag, worst)
    return worst


def test_config1_ten_steps_fp32(cuda, oracle):
    """N = 2^20, fp32 grads fresh each step, m = v = 0 at t = 1, ten AdamW steps, no copy-out."""
    n = 1 << 20
    eng = _engine(**HP)
    p, _, m, v = _gen(n, cuda, seed=0, zero_state=True)
    pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
    gen = torch.Generator(device=cuda).manual_seed(1234)
    group = {}
    for t in range(1, 11):
        g = torch.randn(n, device=cuda, generator=gen) * 1e-3
        group["step"] = t
        eng._step(group, None, p, g, m, v)
        oracle.adam_step(pn, to_np(g), mn, vn, step=t, **{k: HP[k] for k in ("lr", "betas", "eps", "weight_decay")})
        _compare(f"cfg1 t={t}", (p, m, v, None), (pn, mn, vn, None))


@pytest.mark.parametrize("g_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("half_dtype", [None, torch.float16, torch.bfloat16])
def test_dtype_matrix(cuda, oracle, g_dtype, half_dtype):
    n = 300_000 + 3
    eng = _engine(**HP)
    p, g, m, v = _gen(n, cuda, seed=7, g_dtype=g_dtype)
    want = _oracle_step(oracle, p, g, m, v, step=17, half_dtype=half_dtype)
    h = torch.zeros(n, dtype=half_dtype, device=cuda) if half_dtype is not None else None
    eng._step({"step": 17}, h, p, g, m, v)
    _compare(f"g={g_dtype} h={half_dtype}", (p, m, v, h), want, half_dtype)


@pytest.mark.parametrize("adamw_mode,wd,bias_correction", [
    (True, 0.0, True), (True, 0.01, False), (False, 0.01, True), (False, 0.0, False), (False, 0.1, False),
])
def test_modes(cuda, oracle, adamw_mode, wd, bias_correction):
    n = 65_536 + 5
    hp = dict(HP, weight_decay=wd, bias_correction=bias_correction)
    eng = _engine(adamw_mode=adamw_mode, **hp)
    p, g, m, v = _gen(n, cuda, seed=3)
    for t in (1, 2, 1000):
        want = _oracle_step(oracle, p, g, m, v, step=t, half_dtype=torch.float16, adamw_mode=adamw_mode, hp=hp)
        h = torch.zeros(n, dtype=torch.float16, device=cuda)
        eng._step({"step": t}, h, p, g, m, v)
        _compare(f"adamw={adamw_mode} wd={wd} bc={bias_correction} t={t}", (p, m, v, h), want, torch.float16)


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 15, 16, 17, 63, 64, 65, 127, 128, 129, 1000, 2047, 2048, 2049, 4099])
@pytest.mark.parametrize("offset", [0, 1, 2, 3])
def test_tails_and_offsets(cuda, oracle, n, offset):
    """Ragged sizes, and segments that start at any element offset of larger flat buffers (the way
    StepContext views are cut): head / vector body / tail must give the same values."""
    eng = _engine(**HP)
    pad = 8
    total = offset + n + pad
    P, G, M, V = _gen(total, cuda, seed=100 + n, g_dtype=torch.bfloat16)
    H = torch.full((total,), 7.0, dtype=torch.bfloat16, device=cuda)
    before = [t.clone() for t in (P, M, V, H)]
    sl = slice(offset, offset + n)
    want = _oracle_step(oracle, P[sl], G[sl], M[sl], V[sl], step=5, half_dtype=torch.bfloat16)
    eng._step({"step": 5}, H[sl], P[sl], G[sl], M[sl], V[sl])
    _compare(f"n={n} off={offset}", (P[sl], M[sl], V[sl], H[sl]), want, torch.bfloat16)
    # nothing outside the segment was touched
    for now, was in zip((P, M, V, H), before):
        assert torch.equal(now[:offset], was[:offset]) and torch.equal(now[offset + n:], was[offset + n:])


def test_mismatched_alignment_keeps_the_results(cuda, oracle):
    """Arrays whose element offsets differ cannot share the aligned vector body (they go through the
    tile kernel that assumes element alignment only, and its element-per-lane edges); results must
    not change."""
    eng = _engine(**HP)
    n = 10_001
    P, G, M, V = _gen(n + 8, cuda, seed=9, g_dtype=torch.float16)
    H = torch.zeros(n + 8, dtype=torch.float16, device=cuda)
    p, g, m, v, h = P[0:n], G[1:n + 1], M[2:n + 2], V[3:n + 3], H[1:n + 1]
    want = _oracle_step(oracle, p, g, m, v, step=3, half_dtype=torch.float16)
    eng._step({"step": 3}, h, p, g, m, v)
    _compare("misaligned", (p, m, v, h), want, torch.float16)


@pytest.mark.parametrize("odd_one,g_dtype,half_dtype", [
    (odd, g, h) for g, h in ((torch.bfloat16, torch.bfloat16), (torch.float32, torch.float16), (torch.float16, None))
    for odd in "pgmvh" if not (odd == "h" and h is None)])
@pytest.mark.parametrize("control", [None, "scale", "skip"])
def test_one_array_off_the_others(cuda, oracle, odd_one, g_dtype, half_dtype, control):
    """One array starts 1, 2, 3, 4 or 16 elements into its buffer, the others at the start of theirs (a
    16-bit copy cut at an odd element, a state array one element off; with 4 and 16 the arrays agree
    as vectors and disagree on cache lines, which takes the same kernel): many tiles, bits as the
    oracle's, nothing written outside the views, a skipped step leaves everything alone."""
    eng = _engine(**HP)
    n, pad = 300_003, 24
    for shift in (1, 2, 3, 4, 16):
        P, G, M, V = _gen(n + pad, cuda, seed=40 + shift, g_dtype=g_dtype)
        H = torch.full((n + pad,), 7.0, dtype=half_dtype, device=cuda) if half_dtype is not None else None
        offs = {k: (shift if k == odd_one else 0) for k in "pgmvh"}
        p, g, m, v = (t[offs[k]:offs[k] + n] for k, t in (("p", P), ("g", G), ("m", M), ("v", V)))
        h = H[offs["h"]:offs["h"] + n] if H is not None else None
        before = {k: t.clone() for k, t in (("p", P), ("g", G), ("m", M), ("v", V), ("h", H)) if t is not None}
        mult = 0.25 if control else 1.0
        want = _oracle_step(oracle, p, g, m, v, step=9, half_dtype=half_dtype, grad_mult=mult)
        kwargs = {}
        if control:
            rec = torch.zeros(4, dtype=torch.float32, device=cuda)
            rec[1], rec[3] = mult, 1.0
            rec.view(torch.int32)[0] = 1 if control == "skip" else 0
            kwargs["control"] = rec
        eng._step({"step": 9}, h, p, g, m, v, **kwargs)
        if control == "skip":
            for k, t in (("p", P), ("m", M), ("v", V), ("h", H)):
                assert t is None or torch.equal(t, before[k]), (odd_one, shift, k)
            continue
        _compare(f"{odd_one} off by {shift}", (p, m, v, h), want, half_dtype)
        for k, t in (("p", P), ("g", G), ("m", M), ("v", V), ("h", H)):
            if t is not None:
                o = offs[k]
                assert torch.equal(t[:o], before[k][:o]) and torch.equal(t[o + n:], before[k][o + n:]), (odd_one, shift, k)
        assert torch.equal(G, before["g"])


@pytest.mark.parametrize("odd_one", ["m", "g", "h", "pv"])
def test_relaxed_tiles_over_several_steps(cuda, oracle, odd_one):
    """The relaxed-alignment tiles read the array that is off the cache lines through the caches, and
    neighbouring tiles on different dies share a line of it: five steps in a row on the same arrays
    (each reading what the one before wrote, other arrays updated in between) stay bit for bit with
    the oracle."""
    eng = _engine(**HP)
    n, pad = 1_000_003, 8
    P, G, M, V = _gen(n + pad, cuda, seed=77, g_dtype=torch.bfloat16)
    H = torch.zeros(n + pad, dtype=torch.bfloat16, device=cuda)
    offs = {k: (1 if k in odd_one else 0) for k in "pgmvh"}
    p, g, m, v, h = (t[offs[k]:offs[k] + n] for k, t in (("p", P), ("g", G), ("m", M), ("v", V), ("h", H)))
    pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
    hn = np.zeros(n, np.uint16)
    for step in range(1, 6):
        g.copy_((torch.randn(n, device=cuda, generator=torch.Generator(device=cuda).manual_seed(step)) * 1e-3).to(torch.bfloat16))
        oracle.adam_step(pn, to_np(g), mn, vn, step=step, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                         weight_decay=HP["weight_decay"], bias_correction=HP["bias_correction"], adamw_mode=True,
                         g_dtype=CODE[torch.bfloat16], half_out=hn, half_dtype=CODE[torch.bfloat16])
        eng._step({"step": step}, h, p, g, m, v)
    _compare(f"{odd_one} off, five steps", (p, m, v, h), (pn, mn, vn, hn), torch.bfloat16)


def test_special_values(cuda, oracle):
    """Zeros, denormals, huge and tiny magnitudes, negative zero; g = m = v = 0 leaves m = v = 0 and
    p' = fma(p, -lr*wd, p) exactly (what happens to the zero padding at the end of a unit)."""
    eng = _engine(**HP)
    vals = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-40, 1e-38, 1.17549435e-38, 1e-30, 1e-20, 1e-10, 1e-5, 1.0,
                     -1.0, 3.0, 1e5, 1e10, 1e18, 3e38, -3e38, 65504.0, 65520.0, 2.0 ** -24, 2.0 ** -25], dtype=np.float32)
    grid = np.array(np.meshgrid(vals, vals, np.abs(vals[:12]), indexing="ij")).reshape(3, -1)
    n = grid.shape[1]
    p = torch.from_numpy(np.ascontiguousarray(grid[0])).to(cuda)
    g = torch.from_numpy(np.ascontiguousarray(grid[1])).to(cuda)
    v = torch.from_numpy(np.ascontiguousarray(grid[2])).to(cuda)
    m = torch.from_numpy(np.ascontiguousarray(grid[1][::-1])).to(cuda) * 0.5
    want = _oracle_step(oracle, p, g, m, v, step=2, half_dtype=torch.float16)
    h = torch.zeros(n, dtype=torch.float16, device=cuda)
    eng._step({"step": 2}, h, p, g, m, v)
    _compare("special", (p, m, v, h), want, torch.float16)

    n = 4096
    p0 = torch.randn(n, device=cuda)
    z = [torch.zeros(n, device=cuda) for _ in range(3)]
    p = p0.clone()
    eng._step({"step": 1}, None, p, z[0], z[1], z[2])
    assert not z[1].any() and not z[2].any()
    wdec = np.float32(np.float32(-1.0 * np.float32(HP["lr"])) * np.float32(HP["weight_decay"]))
    expect = np.array([np.float32(np.float64(x) * np.float64(wdec) + np.float64(x)) for x in to_np(p0)], dtype=np.float32)
    assert np.array_equal(to_np(p).view(np.uint32), expect.view(np.uint32))


def test_grad_mult_and_device_control(cuda, oracle):
    """grad_mult as a host scalar and as a device-side decision give the same bits; skip leaves all
    four arrays untouched."""
    from flextrain_amd.loss_scaler import GradientGuard
    eng = _engine(**HP)
    n = 123_457
    scale = 65536.0
    p, g, m, v = _gen(n, cuda, seed=11, g_dtype=torch.float16, g_std=1e-3 * 64)
    mult = float(np.float32(1.0 / scale))
    want = _oracle_step(oracle, p, g, m, v, step=4, half_dtype=torch.bfloat16, grad_mult=mult)

    p1, m1, v1 = p.clone(), m.clone(), v.clone()
    h1 = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    eng._step({"step": 4}, h1, p1, g, m1, v1, grad_mult=mult)
    _compare("host mult", (p1, m1, v1, h1), want, torch.bfloat16)

    guard = GradientGuard(cuda)
    guard.begin()
    guard.add(g, loss_scale=scale)
    ctl = guard.decide_async(loss_scale=scale, max_grad_norm=None)
    p2, m2, v2 = p.clone(), m.clone(), v.clone()
    h2 = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    eng._step({"step": 4}, h2, p2, g, m2, v2, control=ctl)
    _compare("device control", (p2, m2, v2, h2), want, torch.bfloat16)

    g_bad = g.clone()
    g_bad[n // 2] = float("nan")
    guard.begin()
    guard.add(g_bad, loss_scale=scale)
    ctl = guard.decide_async(loss_scale=scale)
    p3, m3, v3 = p.clone(), m.clone(), v.clone()
    h3 = torch.full((n,), 3.0, dtype=torch.bfloat16, device=cuda)
    eng._step({"step": 4}, h3, p3, g_bad, m3, v3, control=ctl)
    assert torch.equal(p3, p) and torch.equal(m3, m) and torch.equal(v3, v)
    assert torch.equal(h3, torch.full((n,), 3.0, dtype=torch.bfloat16, device=cuda))


def test_config2_llama7b_layer(cuda, oracle):
    """The 7B decoder-layer partition at full size: 202,383,360 elements, bf16 grads, AdamW at
    t = 100, bf16 copy-out."""
    n = 4 * 4096 ** 2 + 3 * 4096 * 11008 + 2 * 4096
    assert n == 202_383_360
    eng = _engine(**HP)
    p, g, m, v = _gen(n, cuda, seed=0, g_dtype=torch.bfloat16)
    want = _oracle_step(oracle, p, g, m, v, step=100, half_dtype=torch.bfloat16)
    h = torch.zeros(n, dtype=torch.bfloat16, device=cuda)
    eng._step({"step": 100}, h, p, g, m, v)
    hist = {k: ulp_histogram_gpu(t, w) for k, t, w in (("p", p, want[0]), ("m", m, want[1]), ("v", v, want[2]), ("h", h, want[3]))}
    print("[cfg2] ULP distance histograms (elements at 0 / 1 / 2 / more): "
          + "; ".join(f"{k}: {x['0']} / {x['1']} / {x['2']} / {x['>2']}" for k, x in hist.items()), flush=True)
    assert max(hist[k]["max"] for k in "pmv") <= MASTER_ULP and hist["h"]["max"] <= HALF_ULP, hist


def test_errors_are_reported_not_undefined(cuda):
    eng = _engine(**HP)
    n = 64
    p, g, m, v = _gen(n, cuda, seed=1)
    with pytest.raises(AssertionError):
        eng._step({}, None, p, g, m, v)  # no "step"
    with pytest.raises(ValueError):
        eng._step({"step": 1}, None, p, g[:-1], m, v)  # length mismatch
    with pytest.raises(ValueError):
        eng._step({"step": 1}, None, p.double(), g, m, v)  # master dtype
    with pytest.raises(ValueError):
        eng._step({"step": 1}, None, torch.zeros(2 * n, device=cuda)[::2], g, m, v)  # non-contiguous
    with pytest.raises(ValueError):
        eng._step({"step": 1}, p.clone(), p, g, m, v)  # fp32 "half" parameter
    from flextrain_amd import _C
    with pytest.raises(_C.FtError):
        _C.check("ft_adam_step", _C.lib().ft_adam_step(987654, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, p.data_ptr(),
                                                       g.data_ptr(), 0, m.data_ptr(), v.data_ptr(), None, 1, n, None, None))
