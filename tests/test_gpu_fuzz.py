"""Seeded random cases of the resident update against the oracle: random lengths, random element
offsets per array (equal offsets take the vector path with head and tail launches, unequal ones the
all-scalar path), every gradient / copy-out type, both decay modes, bias correction on and off,
host-side multipliers, device-side control records, the step's scalars by value or in a device record,
special values sprinkled in. Bit-exact bar
(the documented tolerance is 2 ULP / 1 ULP; the kernels are written to hit 0)."""
import os

import numpy as np
import pytest
import torch

from _util import CODE, F16, half_bits, to_np

pytestmark = pytest.mark.gpu

G_DTYPES = [torch.float32, torch.float16, torch.bfloat16]
H_DTYPES = [None, torch.float16, torch.bfloat16]
SPECIALS = [0.0, -0.0, 1e-45, -1e-45, 1e-38, 3e38, -3e38, float("inf"), float("-inf"), float("nan"), 1.0, -1.0]


def _bits32(t):
    return to_np(t).view(np.uint32)


@pytest.mark.parametrize("seed", range(int(os.environ.get("FT_FUZZ_SEEDS", "6"))))
def test_random_cases_bit_exact(cuda, oracle, seed):
    from flextrain_amd import FlexTrainCPUAdam
    rng = np.random.default_rng(1000 + seed)
    gen = torch.Generator(device=cuda).manual_seed(2000 + seed)
    worst_cases = 0
    for case in range(40):
        n = int(rng.choice([rng.integers(1, 40), rng.integers(40, 2000), rng.integers(2000, 300_000)]))
        same_offsets = rng.random() < 0.7
        base_off = int(rng.integers(0, 8))
        offs = {k: base_off if same_offsets else int(rng.integers(0, 8)) for k in "pgmvh"}
        g_dtype = G_DTYPES[int(rng.integers(0, 3))]
        h_dtype = H_DTYPES[int(rng.integers(0, 3))]
        adamw = bool(rng.integers(0, 2))
        hp = dict(lr=float(10 ** rng.uniform(-5, -2)), betas=(float(rng.choice([0.9, 0.8, 0.95])), float(rng.choice([0.999, 0.99, 0.95]))),
                  eps=float(rng.choice([1e-8, 1e-6, 1e-5])), weight_decay=float(rng.choice([0.0, 0.01, 0.1])),
                  bias_correction=bool(rng.integers(0, 2)))
        step = int(rng.choice([1, 2, 7, 100, 1000, 123456]))
        mode = rng.choice(["plain", "mult", "ctl", "skip"])

        def arr(k, dtype, fill):
            buf = torch.zeros(n + 16, dtype=dtype, device=cuda)
            view = buf[offs[k]:offs[k] + n]
            view.copy_(fill)
            return buf, view

        pb, p = arr("p", torch.float32, torch.randn(n, device=cuda, generator=gen) * 0.02)
        mb, m = arr("m", torch.float32, torch.randn(n, device=cuda, generator=gen) * 1e-4)
        vb, v = arr("v", torch.float32, torch.rand(n, device=cuda, generator=gen) * 1e-6)
        gb, g = arr("g", g_dtype, (torch.randn(n, device=cuda, generator=gen) * 1e-2).to(g_dtype))
        hb, h = (None, None) if h_dtype is None else arr("h", h_dtype, torch.zeros(n, device=cuda).to(h_dtype))
        if rng.random() < 0.3:  # special values in gradients and parameters (never a negative v: sqrt)
            for _ in range(min(n, 6)):
                g[int(rng.integers(0, n))] = SPECIALS[int(rng.integers(0, len(SPECIALS)))]
                p[int(rng.integers(0, n))] = SPECIALS[int(rng.integers(0, 7))]

        grad_mult, control = 1.0, None
        if mode == "mult":
            grad_mult = float(np.float32(rng.choice([0.5, 1.0 / 1024, 0.3, 1.7])))
        elif mode in ("ctl", "skip"):
            grad_mult = float(np.float32(rng.choice([0.25, 0.0123])))
            control = torch.zeros(4, dtype=torch.float32, device=cuda)
            control[1] = grad_mult
            control.view(torch.int32)[0] = 1 if mode == "skip" else 0

        pn, mn, vn = to_np(p).copy(), to_np(m).copy(), to_np(v).copy()
        gn = half_bits(g) if g_dtype != torch.float32 else to_np(g)
        hn = None if h is None else half_bits(h).copy()
        if mode != "skip":
            hn = None if h is None else np.zeros(n, np.uint16)
            oracle.adam_step(pn, gn, mn, vn, step=step, lr=hp["lr"], betas=hp["betas"], eps=hp["eps"],
                             weight_decay=hp["weight_decay"], bias_correction=hp["bias_correction"], adamw_mode=adamw,
                             grad_mult=grad_mult, g_dtype=CODE[g_dtype], half_out=hn,
                             half_dtype=CODE[h_dtype] if h_dtype is not None else F16)

        eng = FlexTrainCPUAdam(adamw_mode=adamw, **hp)
        kw, group = {}, {"step": step}
        in_record = rng.random() < 0.35  # the step's scalars read from device memory instead of passed by value
        if in_record:
            eng.make_capturable(group, cuda)
            group["hyper_record"].fill(group, grad_mult=grad_mult if mode == "mult" else 1.0).sync()
        elif mode == "mult":
            kw["grad_mult"] = grad_mult
        if control is not None:
            kw["control"] = control
        eng._step(group, h, p, g, m, v, **kw)

        tag = (seed, case, n, offs, str(g_dtype), str(h_dtype), adamw, hp, step, mode, in_record)
        # NaN payloads: compare bits where finite, NaN-ness where not
        for name, got, want in (("p", p, pn), ("m", m, mn), ("v", v, vn)):
            gbits, wbits = _bits32(got), want.view(np.uint32)
            nan_g, nan_w = np.isnan(to_np(got)), np.isnan(want)
            assert np.array_equal(nan_g, nan_w), (name, tag)
            assert np.array_equal(gbits[~nan_g], wbits[~nan_w]), (name, tag)
        if h is not None:
            hg = half_bits(h)
            fl = (lambda b: b.view(np.float16).astype(np.float32)) if h_dtype == torch.float16 else \
                (lambda b: (b.astype(np.uint32) << 16).view(np.float32))
            nan_g, nan_w = np.isnan(fl(hg)), np.isnan(fl(hn))
            assert np.array_equal(nan_g, nan_w), ("h", tag)
            assert np.array_equal(hg[~nan_g], hn[~nan_w]), ("h", tag)
        # nothing outside the views was written
        for k, buf in (("p", pb), ("m", mb), ("v", vb), ("g", gb), ("h", hb)):
            if buf is not None:
                assert not buf[:offs[k]].any() and not buf[offs[k] + n:].any(), (k, tag)
        worst_cases += 1
    assert worst_cases == 40


@pytest.mark.parametrize("seed", range(int(os.environ.get("FT_FUZZ_SEEDS", "4"))))
def test_random_many_context_calls_bit_exact(cuda, oracle, seed):
    """Seeded random calls of the many-contexts launch: 1 to 40 contexts of random length (a few
    elements to a few hundred thousand), random gaps between them in the flat buffers (so every
    head/tail combination occurs), random gradient / copy types, some contexts without a copy, up to
    five parameter groups with random hyper-parameters, host multiplier or device control record,
    special values sprinkled in. Every context against the oracle, bit for bit; nothing outside."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.param_group import StepContext
    rng = np.random.default_rng(3000 + seed)
    gen = torch.Generator(device=cuda).manual_seed(4000 + seed)
    for case in range(12):
        count = int(rng.integers(1, 41))
        lengths = [int(rng.choice([rng.integers(0, 6), rng.integers(1, 600), rng.integers(600, 20_000), rng.integers(20_000, 300_000)]))
                   for _ in range(count)]
        gaps = [int(rng.integers(0, 6)) for _ in range(count)]
        total = sum(lengths) + sum(gaps) + 16
        g_dtype = G_DTYPES[int(rng.integers(0, 3))]
        h_dtype = H_DTYPES[int(rng.integers(1, 3))]
        adamw = bool(rng.integers(0, 2))
        groups = [dict(lr=float(10 ** rng.uniform(-5, -2)), betas=(float(rng.choice([0.9, 0.8])), float(rng.choice([0.999, 0.95]))),
                       eps=float(rng.choice([1e-8, 1e-6])), weight_decay=float(rng.choice([0.0, 0.01, 0.1])),
                       bias_correction=bool(rng.integers(0, 2)), step=int(rng.choice([1, 3, 100, 54321])))
                  for _ in range(int(rng.integers(1, 6)))]
        P = torch.randn(total, device=cuda, generator=gen) * 0.02
        G = (torch.randn(total, device=cuda, generator=gen) * 1e-2).to(g_dtype)
        M = torch.randn(total, device=cuda, generator=gen) * 1e-4
        V = torch.rand(total, device=cuda, generator=gen) * 1e-6
        H = torch.full((total,), 3.0, dtype=h_dtype, device=cuda)
        if rng.random() < 0.4:
            for _ in range(8):
                G[int(rng.integers(0, total))] = SPECIALS[int(rng.integers(0, len(SPECIALS)))]
                P[int(rng.integers(0, total))] = SPECIALS[int(rng.integers(0, 7))]
        mode = rng.choice(["plain", "mult", "ctl", "skip"])
        grad_mult, control = 1.0, None
        if mode == "mult":
            grad_mult = float(np.float32(rng.choice([0.5, 1.0 / 1024, 0.3])))
        elif mode in ("ctl", "skip"):
            grad_mult = float(np.float32(rng.choice([0.25, 0.0123])))
            control = torch.zeros(4, dtype=torch.float32, device=cuda)
            control[1] = grad_mult
            control.view(torch.int32)[0] = 1 if mode == "skip" else 0

        ctxs, spans, lo = [], [], int(rng.integers(0, 8))
        for n, gap in zip(lengths, gaps):
            sl = slice(lo, lo + n)
            with_copy = rng.random() < 0.8
            ctxs.append(StepContext(groups[int(rng.integers(0, len(groups)))], H[sl] if with_copy else None, P[sl], G[sl], [M[sl], V[sl]]))
            spans.append(sl)
            lo += n + gap
        before = [t.clone() for t in (P, M, V, H)]
        wants = []
        for c in ctxs:
            n = c.full_parameter.numel()
            pn, mn, vn = to_np(c.full_parameter).copy(), to_np(c.optimizer_states[0]).copy(), to_np(c.optimizer_states[1]).copy()
            gn = half_bits(c.gradient) if g_dtype != torch.float32 else to_np(c.gradient)
            hn = None if c.half_parameter is None else half_bits(c.half_parameter).copy()
            if mode != "skip" and n:
                hn = None if c.half_parameter is None else np.zeros(n, np.uint16)
                hp = c.param_group
                oracle.adam_step(pn, gn, mn, vn, step=hp["step"], lr=hp["lr"], betas=hp["betas"], eps=hp["eps"],
                                 weight_decay=hp["weight_decay"], bias_correction=hp["bias_correction"], adamw_mode=adamw,
                                 grad_mult=grad_mult, g_dtype=CODE[g_dtype], half_out=hn, half_dtype=CODE[h_dtype])
            wants.append((pn, mn, vn, hn))

        eng = FlexTrainCPUAdam(adamw_mode=adamw)
        kw = {"grad_mult": grad_mult} if mode == "mult" else ({"control": control} if control is not None else {})
        eng._step_many(ctxs, **kw)
        torch.cuda.synchronize()

        tag = (seed, case, count, str(g_dtype), str(h_dtype), adamw, mode)
        fl = (lambda b: b.view(np.float16).astype(np.float32)) if h_dtype == torch.float16 else \
            (lambda b: (b.astype(np.uint32) << 16).view(np.float32))
        for k, (c, (pn, mn, vn, hn)) in enumerate(zip(ctxs, wants)):
            for name, got, want in (("p", c.full_parameter, pn), ("m", c.optimizer_states[0], mn), ("v", c.optimizer_states[1], vn)):
                gbits, wbits = _bits32(got), want.view(np.uint32)
                nan_g, nan_w = np.isnan(to_np(got)), np.isnan(want)
                assert np.array_equal(nan_g, nan_w) and np.array_equal(gbits[~nan_g], wbits[~nan_w]), (name, k, tag)
            if c.half_parameter is not None:
                hg = half_bits(c.half_parameter)
                nan_g, nan_w = np.isnan(fl(hg)), np.isnan(fl(hn))
                assert np.array_equal(nan_g, nan_w) and np.array_equal(hg[~nan_g], hn[~nan_w]), ("h", k, tag)
        keep = torch.ones(total, dtype=torch.bool, device=cuda)
        for sl in spans:
            keep[sl] = False
        for now, old in zip((P, M, V, H), before):
            a, b = now[keep], old[keep]
            assert torch.equal(a.view(torch.int32 if a.dtype == torch.float32 else torch.int16),
                               b.view(torch.int32 if b.dtype == torch.float32 else torch.int16)), ("outside", tag)
        for c, sl in zip(ctxs, spans):  # a context without a copy leaves the copy buffer alone
            if c.half_parameter is None:
                assert bool((H[sl] == 3.0).all()), ("copy written for a context without one", tag)
