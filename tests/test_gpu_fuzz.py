"""Seeded random cases of the resident update against the oracle: random lengths, random element
offsets per array (equal offsets take the vector path with head and tail launches, unequal ones the
all-scalar path), every gradient / copy-out type, both decay modes, bias correction on and off,
host-side multipliers, device-side control records, special values sprinkled in. Bit-exact bar
(the documented tolerance is 2 ULP / 1 ULP; the kernels are written to hit 0)."""
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


@pytest.mark.parametrize("seed", range(6))
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
        kw = {}
        if mode == "mult":
            kw["grad_mult"] = grad_mult
        elif control is not None:
            kw["control"] = control
        eng._step({"step": step}, h, p, g, m, v, **kw)

        tag = (seed, case, n, offs, str(g_dtype), str(h_dtype), adamw, hp, step, mode)
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
