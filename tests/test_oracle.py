"""Pins the CPU oracle before anything is compared against it.

1. against golden vectors produced by the reference's own C++ (tests/golden/adam_reference.npz),
2. against what the mathematics fixes: exact rational arithmetic with one rounding per operation,
   closed forms at t = 1, invariants, torch.optim.AdamW, numpy/torch dtype casts, float64 sums.
No test here re-types the oracle's formula in floating point and calls that a check.
"""
import hashlib
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "adam_reference.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


def _isas(oracle):
    return list(range(oracle.best_isa() + 1))


# ------------------------------------------------------------------------------------------------
# 1. the reference's own outputs
# ------------------------------------------------------------------------------------------------
def test_golden_hyperparameter_cases(oracle, golden):
    cases = json.loads(bytes(golden["cases"]).decode())
    assert len(cases) == 43
    ins = [golden[k].view(np.float32) for k in ("in_p", "in_g", "in_m", "in_v")]
    for k, case in enumerate(cases):
        for isa in _isas(oracle):
            p, g, m, v = (x.copy() for x in ins)
            h = np.zeros(p.shape[0], dtype=np.uint16)
            oracle.adam_step(p, g, m, v, step=case["step"], lr=case["lr"], betas=tuple(case["betas"]), eps=case["eps"],
                             weight_decay=case["wd"], bias_correction=case["bias_correction"],
                             adamw_mode=case["adamw_mode"], half_out=h, half_dtype=oracle.F16, isa=isa)
            for name, got in (("p", p.view(np.uint32)), ("m", m.view(np.uint32)), ("v", v.view(np.uint32)), ("h", h)):
                want = golden[f"case_{k}_{name}"]
                if name == "h":  # NaN payloads of the fp16 copy are not compared, NaN-ness is
                    nan_g, nan_w = (got & 0x7fff) > 0x7c00, (want & 0x7fff) > 0x7c00
                    assert np.array_equal(nan_g, nan_w)
                    got, want = np.where(nan_g, 0, got), np.where(nan_w, 0, want)
                assert np.array_equal(got, want), (case, name, isa, np.flatnonzero(got != want)[:5])


def test_golden_tails(oracle, golden):
    """Ragged sizes: the reference steps tails through a padded vector; per-element results must
    be those of the plain formula."""
    ins = [golden[k].view(np.float32) for k in ("in_p", "in_g", "in_m", "in_v")]
    for n in (1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 500):
        p, g, m, v = (x[:n].copy() for x in ins)
        h = np.zeros(n, dtype=np.uint16)
        oracle.adam_step(p, g, m, v, step=7, lr=1e-4, weight_decay=0.01, half_out=h, half_dtype=oracle.F16)
        assert np.array_equal(p.view(np.uint32), golden[f"tail_{n}_p"])
        assert np.array_equal(m.view(np.uint32), golden[f"tail_{n}_m"])
        assert np.array_equal(v.view(np.uint32), golden[f"tail_{n}_v"])
        assert np.array_equal(h, golden[f"tail_{n}_h"])


def test_golden_config1_trajectory(oracle, golden):
    """The CPU-runnable configuration at its real size: 2^20 elements, 10 AdamW steps, digests of p|m|v."""
    want = json.loads(bytes(golden["cfg1_digest"]).decode())
    n = 1 << 20
    rng = np.random.default_rng(0)
    p = rng.normal(0, 0.02, n).astype(np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t in range(1, 11):
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        oracle.adam_step(p, g, m, v, step=t, lr=1e-4, weight_decay=0.01)
        hsh = hashlib.sha256()
        for x in (p, m, v):
            hsh.update(x.tobytes())
        assert hsh.hexdigest() == want[t - 1], f"step {t}"
    assert int(golden["repeat_same_step_equal"][0]) == 1


def test_bias_correction_sqrt_is_evaluated_in_float(oracle, golden):
    """1/sqrt(1-beta2^t): the unqualified sqrt() of the reference resolves to the float overload.
    For the steps where the float and the double reading give different scalars, the golden
    vectors agree with the float one only."""
    cases = json.loads(bytes(golden["cases"]).decode())
    ins = [golden[k].view(np.float32) for k in ("in_p", "in_g", "in_m", "in_v")]
    told_apart = 0
    for k, case in enumerate(cases):
        if not case["bias_correction"]:
            continue
        kw = dict(step=case["step"], lr=case["lr"], betas=tuple(case["betas"]), eps=case["eps"], weight_decay=case["wd"])
        if oracle.scalars(**kw).bias2 == oracle.scalars(double_sqrt=True, **kw).bias2:
            continue
        p, g, m, v = (x.copy() for x in ins)
        oracle.adam_step(p, g, m, v, adamw_mode=case["adamw_mode"], double_sqrt=True, **kw)
        assert not np.array_equal(p.view(np.uint32), golden[f"case_{k}_p"])
        told_apart += 1
    assert told_apart >= 1


def test_compiled_reference_agrees_on_fresh_inputs(oracle):
    """Where oracle/_ref is built, compare on inputs that are not in the fixture."""
    ref = oracle.reference_module()
    if ref is None:
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(99)
    oid = 7000
    for n in (1, 33, 1000, 70_001):
        for t in (1, 5, 333):
            p = rng.normal(0, 0.02, n).astype(np.float32)
            g = rng.normal(0, 1e-3, n).astype(np.float32)
            m = rng.normal(0, 1e-4, n).astype(np.float32)
            v = rng.uniform(0, 1e-6, n).astype(np.float32)
            tp, tg, tm, tv = (torch.from_numpy(x.copy()) for x in (p, g, m, v))
            th = torch.zeros(n, dtype=torch.float16)
            ref.create_adam(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, False)
            ref.adam_update_copy(oid, t, 2e-4, 0.9, 0.999, 1e-8, 0.05, True, tp, tg, tm, tv, th)
            ref.destroy_adam(oid)
            h = np.zeros(n, np.uint16)
            oracle.adam_step(p, g, m, v, step=t, lr=2e-4, weight_decay=0.05, half_out=h, half_dtype=oracle.F16)
            assert np.array_equal(p.view(np.uint32), tp.numpy().view(np.uint32))
            assert np.array_equal(m.view(np.uint32), tm.numpy().view(np.uint32))
            assert np.array_equal(v.view(np.uint32), tv.numpy().view(np.uint32))
            assert np.array_equal(h, th.numpy().view(np.uint16))


# ------------------------------------------------------------------------------------------------
# 2. exact arithmetic: one rounding per operation, in the reference's order
# ------------------------------------------------------------------------------------------------
def fl32(x: Fraction) -> Fraction:
    """Round a rational to the nearest binary32 value (ties to even), exactly."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    a = abs(x)
    e = math.floor(math.log2(a)) if a.denominator.bit_length() < 900 else 0
    while Fraction(2) ** e > a:
        e -= 1
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    q_exp = max(e - 23, -149)            # weight of the last mantissa bit
    scaled = a / Fraction(2) ** q_exp
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return sign * n * Fraction(2) ** q_exp


def fl32_sqrt(x: Fraction) -> Fraction:
    """Correctly rounded binary32 square root of a non-negative rational."""
    if x == 0:
        return Fraction(0)
    guess = fl32(Fraction(math.sqrt(float(x))))
    # walk to the binary32 value whose rounding interval contains sqrt(x)
    for _ in range(4):
        f = np.float32(float(guess))
        lo = Fraction(float(np.nextafter(f, np.float32(0))))
        hi = Fraction(float(np.nextafter(f, np.float32(np.inf))))
        lower, upper = (guess + lo) / 2, (guess + hi) / 2
        if lower * lower > x:
            guess = lo
        elif upper * upper < x:
            guess = hi
        else:
            break
    return guess


def F(x) -> Fraction:
    return Fraction(float(x))


def exact_step(s, p, g, m, v, grad_mult=1.0):
    """The reference's op sequence (cpu_adam.h:188-205) in exact rationals, rounding once per op."""
    g = fl32(F(g) * F(grad_mult))
    if s.wd_mode == 2:
        g = fl32(F(p) * F(s.wd_coef) + g)
    m1 = fl32(F(m) * F(s.beta1))
    mn = fl32(g * F(s.omb1) + m1)
    v1 = fl32(F(v) * F(s.beta2))
    g2 = fl32(g * g)
    vn = fl32(g2 * F(s.omb2) + v1)
    sq = fl32_sqrt(vn)
    d = fl32(sq * F(s.bias2) + F(s.eps))
    u = fl32(mn / d)
    p1 = fl32(F(p) * F(s.wd_coef) + F(p)) if s.wd_mode == 1 else F(p)
    pn = fl32(u * F(s.step_size) + p1)
    return pn, mn, vn


@pytest.mark.parametrize("adamw_mode,wd", [(True, 0.01), (True, 0.0), (False, 0.01)])
def test_every_operation_rounds_once_in_the_reference_order(oracle, adamw_mode, wd):
    """Catches a dropped term, a swapped operand, a product that was not fused (or one that was):
    each would change the last bit of some element here."""
    rng = np.random.default_rng(1)
    n = 400
    p = rng.normal(0, 0.02, n).astype(np.float32)
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    m = rng.normal(0, 1e-4, n).astype(np.float32)
    v = rng.uniform(0, 1e-6, n).astype(np.float32)
    mult = float(np.float32(0.37))
    s = oracle.scalars(step=9, lr=3e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd, adamw_mode=adamw_mode)
    want = [exact_step(s, p[i], g[i], m[i], v[i], mult) for i in range(n)]
    oracle.adam_step(p, g, m, v, step=9, lr=3e-4, weight_decay=wd, adamw_mode=adamw_mode, grad_mult=mult)
    for i in range(n):
        assert (F(p[i]), F(m[i]), F(v[i])) == want[i], i


def exact_trace(s, p, g, m, v, grad_mult=1.0):
    """All eleven intermediates of exact_step, in the order of oracle.TRACE_NAMES."""
    g = fl32(F(g) * F(grad_mult))
    if s.wd_mode == 2:
        g = fl32(F(p) * F(s.wd_coef) + g)
    m1 = fl32(F(m) * F(s.beta1))
    mn = fl32(g * F(s.omb1) + m1)
    v1 = fl32(F(v) * F(s.beta2))
    g2 = fl32(g * g)
    vn = fl32(g2 * F(s.omb2) + v1)
    sq = fl32_sqrt(vn)
    d = fl32(sq * F(s.bias2) + F(s.eps))
    u = fl32(mn / d)
    p1 = fl32(F(p) * F(s.wd_coef) + F(p)) if s.wd_mode == 1 else F(p)
    pn = fl32(u * F(s.step_size) + p1)
    return dict(zip(("g32", "m1", "m_new", "v1", "g2", "v_new", "sqrt", "denom", "update", "p1", "p_new"),
                    (g, m1, mn, v1, g2, vn, sq, d, u, p1, pn)))


@pytest.mark.parametrize("adamw_mode,wd", [(True, 0.01), (True, 0.0), (False, 0.01)])
def test_trace_exposes_the_same_intermediates(oracle, adamw_mode, wd):
    """adam_trace (one element, every intermediate) against exact rationals rounded once per
    operation, for the three weight-decay modes; its p', m', v' are those of adam_step. A trace
    that skipped the L2 term, decayed after the update or reported a value from the wrong line
    would differ in some named entry."""
    rng = np.random.default_rng(21)
    n = 200
    p = rng.normal(0, 0.02, n).astype(np.float32)
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    m = rng.normal(0, 1e-4, n).astype(np.float32)
    v = rng.uniform(0, 1e-6, n).astype(np.float32)
    mult = float(np.float32(0.61))
    s = oracle.scalars(step=7, lr=2e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd, adamw_mode=adamw_mode)
    assert s.wd_mode == (0 if wd == 0.0 else (1 if adamw_mode else 2))
    traces = [oracle.adam_trace(s, float(p[i]), float(g[i]), float(m[i]), float(v[i]), grad_mult=mult) for i in range(n)]
    for i in range(n):
        want = exact_trace(s, p[i], g[i], m[i], v[i], mult)
        assert set(traces[i]) == set(want)
        for name, value in want.items():
            assert F(traces[i][name]) == value, (i, name)
    ps, ms, vs = p.copy(), m.copy(), v.copy()
    oracle.adam_step(ps, g, ms, vs, step=7, lr=2e-4, weight_decay=wd, adamw_mode=adamw_mode, grad_mult=mult)
    assert np.array_equal(ps, np.array([t["p_new"] for t in traces], np.float32))
    assert np.array_equal(ms, np.array([t["m_new"] for t in traces], np.float32))
    assert np.array_equal(vs, np.array([t["v_new"] for t in traces], np.float32))


def test_host_scalars_follow_the_reference_types(oracle):
    """beta^t in double then float; everything after in float (cpu_adam.h:67-102,148-166)."""
    for t in (1, 2, 10, 100, 1000, 12345):
        s = oracle.scalars(step=t, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
        b1, b2 = np.float32(0.9), np.float32(0.999)
        b1t = np.float32(np.float64(b1) ** np.float64(t))
        b2t = np.float32(np.float64(b2) ** np.float64(t))
        assert np.float32(s.beta1_t) == b1t and np.float32(s.beta2_t) == b2t
        assert np.float32(s.bias1) == np.float32(1) - b1t
        assert np.float32(s.bias2) == np.float32(1) / np.sqrt(np.float32(1) - b2t, dtype=np.float32)
        assert np.float32(s.step_size) == (np.float32(-1) * np.float32(1e-4)) / np.float32(s.bias1)
        assert np.float32(s.wd_coef) == (np.float32(-1) * np.float32(1e-4)) * np.float32(0.01)
        assert np.float32(s.omb1) == np.float32(1) - b1 and np.float32(s.omb2) == np.float32(1) - b2
    s = oracle.scalars(step=5, lr=1e-4, weight_decay=0.01, bias_correction=False)
    assert s.bias1 == 1.0 and s.bias2 == 1.0
    assert oracle.scalars(step=5, lr=1e-4, weight_decay=0.0).wd_mode == 0
    assert oracle.scalars(step=5, lr=1e-4, weight_decay=-1.0).wd_mode == 0  # reference tests `> 0`
    assert oracle.scalars(step=5, lr=1e-4, weight_decay=0.1, adamw_mode=False).wd_mode == 2


def test_closed_form_first_step(oracle):
    """t = 1, m = v = 0: m' = fl(g*fl(1-b1)), v' = fl(fl(g^2)*fl(1-b2)) exactly, and
    p' ~ p*(1 - lr*wd) - lr*g/(|g| + eps), i.e. a step of -lr*sign(g) for |g| >> eps."""
    rng = np.random.default_rng(2)
    n = 10_000
    p0 = rng.normal(0, 0.02, n).astype(np.float32)
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    p, m, v = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    lr, wd, eps = 1e-4, 0.01, 1e-8
    oracle.adam_step(p, g, m, v, step=1, lr=lr, weight_decay=wd, eps=eps)
    omb1 = np.float32(1) - np.float32(0.9)
    omb2 = np.float32(1) - np.float32(0.999)
    assert np.array_equal(m, g * omb1)                 # numpy float32 multiply is one IEEE rounding
    assert np.array_equal(v, (g * g) * omb2)
    want = p0.astype(np.float64) * (1 - lr * wd) - lr * g.astype(np.float64) / (np.abs(g.astype(np.float64)) + eps)
    assert np.max(np.abs(p - want)) < 2e-8              # within ~2 ULP of the largest |p| (ulp(0.08) = 7.5e-9)
    big = np.abs(g) > 1e-5
    assert np.allclose((p - p0 * np.float32(1 - lr * wd))[big], -lr * np.sign(g[big]), rtol=2e-3)


def test_invariants(oracle):
    n = 1000
    rng = np.random.default_rng(3)
    # zero gradient and state: state stays zero, p decays by exactly one fma (unit padding case)
    p0 = rng.normal(0, 1, n).astype(np.float32)
    p, z1, z2, z3 = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32)
    s = oracle.adam_step(p, z1, z2, z3, step=3, lr=1e-3, weight_decay=0.1)
    assert not z2.any() and not z3.any()
    for i in range(0, n, 37):
        assert F(p[i]) == fl32(F(p0[i]) * F(s.wd_coef) + F(p0[i]))
    # v stays non-negative; results do not depend on position, length or thread count
    p = rng.normal(0, 0.02, n).astype(np.float32)
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    m = rng.normal(0, 1e-4, n).astype(np.float32)
    v = rng.uniform(0, 1e-6, n).astype(np.float32)
    a = [x.copy() for x in (p, g, m, v)]
    oracle.adam_step(a[0], a[1], a[2], a[3], step=4, lr=1e-4, weight_decay=0.01, threads=1)
    assert (a[3] >= 0).all()
    big = [np.concatenate([np.zeros(5000, np.float32), x, np.zeros(77, np.float32)]) for x in (p, g, m, v)]
    oracle.adam_step(big[0], big[1], big[2], big[3], step=4, lr=1e-4, weight_decay=0.01)
    for k in (0, 2, 3):
        assert np.array_equal(big[k][5000:5000 + n].view(np.uint32), a[k].view(np.uint32))


def test_against_torch_adamw(oracle):
    """Same algebra, different rounding order: agreement to ~1e-6 relative over 10 steps."""
    torch.manual_seed(0)
    n = 5000
    p0 = (torch.randn(n) * 0.02)
    tp = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([tp], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, foreach=False)
    p, m, v = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t in range(1, 11):
        g = torch.randn(n) * 1e-2
        tp.grad = g.clone()
        opt.step()
        oracle.adam_step(p, g.numpy().copy(), m, v, step=t, lr=1e-3, weight_decay=0.01)
    st = opt.state[tp]
    assert np.allclose(p, tp.detach().numpy(), rtol=2e-6, atol=2e-8)  # atol: a few ULP of |p| ~ 0.05
    assert np.allclose(m, st["exp_avg"].numpy(), rtol=2e-6, atol=2e-9)     # |m| ~ 3e-3: a few ULP
    # The reference forms 1-beta2 in float (1 - 0.999f = 0.00099998713), torch in double (0.001):
    # a relative offset of 1.3e-5 in every increment of v, which the golden vectors confirm.
    assert np.allclose(v, st["exp_avg_sq"].numpy(), rtol=3e-5, atol=1e-12)


def test_adam_l2_mode_against_torch_adam(oracle):
    torch.manual_seed(1)
    n = 3000
    p0 = torch.randn(n) * 0.02
    tp = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Adam([tp], lr=1e-3, weight_decay=0.1, foreach=False)
    p, m, v = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t in range(1, 6):
        g = torch.randn(n) * 1e-2
        tp.grad = g.clone()
        opt.step()
        oracle.adam_step(p, g.numpy().copy(), m, v, step=t, lr=1e-3, weight_decay=0.1, adamw_mode=False)
    assert np.allclose(p, tp.detach().numpy(), rtol=5e-6, atol=2e-8)


def test_isa_variants_agree(oracle):
    rng = np.random.default_rng(5)
    n = 100_003
    base = [rng.normal(0, 0.02, n).astype(np.float32), rng.normal(0, 1e-3, n).astype(np.float32),
            rng.normal(0, 1e-4, n).astype(np.float32), rng.uniform(0, 1e-6, n).astype(np.float32)]
    outs = []
    for isa in _isas(oracle):
        p, g, m, v = (x.copy() for x in base)
        h = np.zeros(n, np.uint16)
        oracle.adam_step(p, g, m, v, step=11, lr=1e-4, weight_decay=0.01, half_out=h, half_dtype=oracle.BF16, isa=isa)
        outs.append((p, m, v, h))
    for o in outs[1:]:
        for a, b in zip(o, outs[0]):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


# ------------------------------------------------------------------------------------------------
# conversions and 16-bit inputs
# ------------------------------------------------------------------------------------------------
def _float_sample():
    """All 65536 upper halves crossed with lower-half patterns that sit on and around every
    rounding boundary of both 16-bit formats."""
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x0fff, 0x1000, 0x1001, 0x1fff, 0x2000, 0x2fff, 0x3000, 0x3001, 0x7fff,
                     0x8000, 0x8001, 0xbfff, 0xc000, 0xffff], dtype=np.uint32)
    return (hi[:, None] | lows[None, :]).reshape(-1)


def test_f32_to_f16_matches_numpy_and_torch(oracle):
    bits = _float_sample()
    x = bits.view(np.float32)
    got = oracle.convert(x, oracle.F32, oracle.F16)
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7c00) == 0x7c00).all() and ((got[nan] & 0x03ff) != 0).all()
    want_t = torch.from_numpy(x.copy()).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[~nan], want_t[~nan])
    # ties to even, enumerated: halfway between neighbouring halves
    for lo16, expect in ((0x3c00, 0x3c00), (0x3c01, 0x3c02)):
        a = np.array([lo16], np.uint16).view(np.float16).astype(np.float32)
        b = np.array([lo16 + 1], np.uint16).view(np.float16).astype(np.float32)
        mid = ((a.astype(np.float64) + b.astype(np.float64)) / 2).astype(np.float32)
        assert oracle.convert(mid, oracle.F32, oracle.F16)[0] == expect


def test_f32_to_bf16_matches_torch(oracle):
    bits = _float_sample()
    x = bits.view(np.float32)
    got = oracle.convert(x, oracle.F32, oracle.BF16)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7f80) == 0x7f80).all() and ((got[nan] & 0x007f) != 0).all()
    # closed form on the non-NaN part: round half to even on bit 16
    b = bits[~nan].astype(np.uint64)
    assert np.array_equal(got[~nan], ((b + 0x7fff + ((b >> 16) & 1)) >> 16).astype(np.uint16))


def test_16bit_to_f32_is_exact(oracle):
    h = np.arange(1 << 16, dtype=np.uint16)
    got = oracle.convert(h, oracle.F16, oracle.F32)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan]) and np.isnan(got[nan]).all()
    got = oracle.convert(h, oracle.BF16, oracle.F32)
    assert np.array_equal(got.view(np.uint32), h.astype(np.uint32) << 16)


@pytest.mark.parametrize("code,tdtype", [(1, torch.float16), (2, torch.bfloat16)])
def test_16bit_gradients_equal_upconverted_fp32_gradients(oracle, code, tdtype):
    """g16 -> f32 is exact, so stepping with 16-bit gradients must equal stepping with their fp32 image."""
    torch.manual_seed(2)
    n = 4097
    g16 = (torch.randn(n) * 1e-3).to(tdtype)
    g32 = g16.to(torch.float32).numpy().copy()
    rng = np.random.default_rng(2)
    base = [rng.normal(0, 0.02, n).astype(np.float32), rng.normal(0, 1e-4, n).astype(np.float32),
            rng.uniform(0, 1e-6, n).astype(np.float32)]
    a = [x.copy() for x in base]
    b = [x.copy() for x in base]
    oracle.adam_step(a[0], g16.view(torch.int16).numpy().view(np.uint16), a[1], a[2], step=3, lr=1e-4,
                     weight_decay=0.01, g_dtype=code, grad_mult=0.5)
    oracle.adam_step(b[0], g32, b[1], b[2], step=3, lr=1e-4, weight_decay=0.01, grad_mult=0.5)
    for x, y in zip(a, b):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))


# ------------------------------------------------------------------------------------------------
# extensions: statistics, clip coefficient, scale trace
# ------------------------------------------------------------------------------------------------
def test_grad_stats_against_float64(oracle):
    rng = np.random.default_rng(7)
    n = 300_001
    g = rng.normal(0, 3.0, n).astype(np.float32)
    bad, sumsq = oracle.grad_stats(g, oracle.F32, pre_mult=0.25)
    assert bad == 0
    want = float(np.sum((g * np.float32(0.25)).astype(np.float64) ** 2))
    assert abs(sumsq - want) <= 1e-12 * want
    g[[0, 17, n - 1]] = [np.inf, -np.inf, np.nan]
    bad, sumsq2 = oracle.grad_stats(g, oracle.F32, pre_mult=0.25)
    assert bad == 3 and sumsq2 < sumsq
    for code, dt in ((oracle.F16, torch.float16), (oracle.BF16, torch.bfloat16)):
        t = (torch.randn(10_001) * 2).to(dt)
        t[5] = float("nan")
        t[6] = float("-inf")
        bits = t.view(torch.int16).numpy().view(np.uint16)
        bad, sumsq = oracle.grad_stats(bits, code)
        finite = t.to(torch.float64)[torch.isfinite(t.to(torch.float32))]
        assert bad == 2 and abs(sumsq - float((finite ** 2).sum())) <= 1e-12 * sumsq


@pytest.mark.parametrize("code", [0, 2])
def test_grad_stats_keeps_huge_and_tiny_finite_gradients(oracle, code):
    """Finite gradients whose squares leave the fp32 range (|g| above 1.8e19 or below 1e-23) must
    neither overflow the sum nor vanish from it: the sum is checked against exact rational
    arithmetic, rounded to fp64 once, alone and mixed with ordinary values."""
    from fractions import Fraction
    for mags in ((1e-25,), (1e-20,), (1e19,), (1e20,), (3e38,), (1e-25, 3e-3, 1e-20), (1e19, -2.5, 3e38, 1e20, 1e-3)):
        g32 = np.array(mags * 5, dtype=np.float32)
        if code == 2:  # bf16 bit patterns of the same magnitudes (rounded to bf16)
            t = torch.from_numpy(g32).to(torch.bfloat16)
            g = t.view(torch.int16).numpy().view(np.uint16)
            vals = t.to(torch.float32).numpy()
        else:
            g, vals = g32, g32
        bad, sumsq = oracle.grad_stats(g, code)
        exact = sum(Fraction(float(x)) ** 2 for x in vals)
        assert bad == 0 and math.isfinite(sumsq) and sumsq > 0
        assert abs(Fraction(sumsq) - exact) <= exact * Fraction(1, 10 ** 14), mags


def test_clip_coefficient_and_multiplier(oracle):
    assert oracle.clip_coefficient(0.5, 1.0) == 1.0
    assert oracle.clip_coefficient(146.0, 1.0) == pytest.approx(1 / 146.000001)
    assert oracle.clip_coefficient(10.0, None) == 1.0
    # torch's own clip_grad_norm_ applies the same coefficient
    t = torch.nn.Parameter(torch.zeros(1000))
    t.grad = torch.randn(1000) * 5
    g0 = t.grad.clone()
    norm = torch.nn.utils.clip_grad_norm_([t], max_norm=1.0)
    assert torch.allclose(t.grad, g0 * oracle.clip_coefficient(float(norm), 1.0), rtol=1e-6)
    assert oracle.combined_multiplier(65536.0, 1.0) == np.float32(2.0 ** -16)
    # Scales that are no power of two with a clip below 1: the multiplier is the fp32 product of the
    # two separately rounded factors, fl(fl(clip) * fl(1/scale)). The cases are chosen (and checked)
    # so that the other plausible readings -- fl(clip/scale), or the product formed in double and
    # rounded once -- give a different float.
    for scale, clip in ((3.0, 0.839667), (65535.0, 0.543673), (1000.0, 0.014088), (48000.0, 0.915513), (100.0, 0.301756)):
        a, b = fl32(Fraction(clip)), fl32(Fraction(1.0 / scale))
        want = fl32(a * b)
        assert fl32(Fraction(clip) / Fraction(scale)) != want and fl32(Fraction(clip) * Fraction(1.0 / scale)) != want
        assert F(oracle.combined_multiplier(scale, clip)) == want, (scale, clip)


def test_loss_scale_traces(oracle):
    """The two hand-derived 8-step traces (overflow on steps 3 and 6, initial scale 65536)."""
    ov = [i in (3, 6) for i in range(1, 9)]
    assert oracle.loss_scale_trace(ov, 65536.0, delayed_shift=1) == \
        [65536.0] * 3 + [32768.0] * 3 + [16384.0] * 2 + [16384.0]
    assert oracle.loss_scale_trace(ov, 65536.0, delayed_shift=2) == [65536.0] * 6 + [32768.0] * 2 + [32768.0]
    # growth: first doubling when cur_iter = window - 1 (last_overflow_iter starts at -1)
    tr = oracle.loss_scale_trace([False] * 8, 4.0, scale_window=4)
    assert tr == [4.0, 4.0, 4.0, 4.0, 8.0, 8.0, 8.0, 8.0, 16.0]
    assert oracle.loss_scale_trace([True] * 4, 4.0, min_scale=1.0) == [4.0, 2.0, 1.0, 1.0, 1.0]


def test_grad_accumulate_closed_forms(oracle):
    """scale = 1: one add of the exactly widened gradient (numpy / torch); scale != 1: one fma,
    checked in exact rationals; 16-bit accumulators: round-to-nearest-even of that fp32 value."""
    rng = np.random.default_rng(11)
    n = 5001
    acc0 = rng.normal(0, 1, n).astype(np.float32)
    g16 = (torch.randn(n) * 0.1).to(torch.bfloat16)
    acc = acc0.copy()
    gbits = g16.view(torch.int16).numpy().view(np.uint16).copy()
    oracle.grad_accumulate(acc, oracle.F32, gbits, oracle.BF16)
    assert np.array_equal(acc, acc0 + g16.float().numpy())
    acc = acc0.copy()
    scale = np.float32(0.3)
    oracle.grad_accumulate(acc, oracle.F32, gbits, oracle.BF16, scale=float(scale), zero_g=True)
    assert not gbits.any()
    gf = g16.float().numpy()
    for i in range(0, n, 50):
        assert F(acc[i]) == fl32(F(gf[i]) * F(scale) + F(acc0[i]))
    for code, dt in ((oracle.F16, torch.float16), (oracle.BF16, torch.bfloat16)):
        a = (torch.randn(n) * 2).to(dt)
        g = (torch.randn(n) * 0.5).to(torch.float16)
        abits = a.view(torch.int16).numpy().view(np.uint16).copy()
        oracle.grad_accumulate(abits, code, g.view(torch.int16).numpy().view(np.uint16).copy(), oracle.F16)
        want = (a.float() + g.float()).to(dt).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(abits, want)
