#!/usr/bin/env python3
"""Writes tests/golden/adam_reference.npz from the reference's own C++ CPU Adam.

The vectors come from the pybind module that `make -f oracle/Makefile ref` compiles from the
reference's two source files where they lie (flextrain/ops/csrc/adam/cpu_adam.cpp and
cpu_adam_impl.cpp), i.e. from the reference implementation itself, not from this repository's
restatement. Run it where the reference checkout is available:

    make -f oracle/Makefile ref && python tests/golden/make_adam_golden.py

Everything is stored as raw bit patterns (uint32 / uint16) so that a comparison is exact.
Inputs are drawn with numpy's PCG64 (seed 0), which is reproducible across platforms.

Contents
  in_p, in_g, in_m, in_v          shared inputs, 512 elements: 448 random + 64 special values
  case_<k>_{p,m,v,h}              outputs of adam_update_copy for hyper-parameter case k
  cases                           JSON list describing every case (step, mode, wd, bias_correction, lr ...)
  tail_<n>_{p,m,v,h}              outputs for n in TAIL_SIZES on the first n shared inputs (AdamW, t=7)
  cfg1_digest                     sha256 of p|m|v after each of 10 AdamW steps on 2^20 elements
                                  (the CPU-runnable configuration: p~N(0,0.02), fresh g~N(0,1e-3) per step, m=v=0 at t=1)
  repeat_same_step_equal          1 if calling the same step twice from identical state copies gave
                                  identical outputs (the cached-power branch of IncrementStep)
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

N = 512
TAIL_SIZES = (1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 500)
SPECIAL = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-40, -1e-40, 1e-38, 1.17549435e-38, 1e-30, -1e-30, 1e-20,
                    1e-10, 1e-5, 1.0, -1.0, 3.0, 1e5, 1e10, -1e10, 1e18, 3e38, -3e38, 65504.0, 65520.0,
                    2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -14, 1.0009765625, 1.00048828125,
                    1.00146484375, 0.1], dtype=np.float32)


def shared_inputs():
    rng = np.random.default_rng(0)
    k = N - 2 * len(SPECIAL)
    p = np.concatenate([rng.normal(0, 0.02, k), SPECIAL, SPECIAL[::-1]]).astype(np.float32)
    g = np.concatenate([rng.normal(0, 1e-3, k), SPECIAL[::-1], SPECIAL]).astype(np.float32)
    m = np.concatenate([rng.normal(0, 1e-4, k), 0.5 * SPECIAL, -0.25 * SPECIAL]).astype(np.float32)
    v = np.concatenate([rng.uniform(0, 1e-6, k), np.abs(SPECIAL), np.abs(SPECIAL[::-1])]).astype(np.float32)
    return p, g, m, v


def run_ref(ref, oid, p, g, m, v, *, step, lr, betas, eps, wd, bias_correction, copy=True):
    tp, tg, tm, tv = (torch.from_numpy(x.copy()) for x in (p, g, m, v))
    th = torch.zeros(p.shape[0], dtype=torch.float16)
    if copy:
        ref.adam_update_copy(oid, step, lr, betas[0], betas[1], eps, wd, bias_correction, tp, tg, tm, tv, th)
    else:
        ref.adam_update(oid, step, lr, betas[0], betas[1], eps, wd, bias_correction, tp, tg, tm, tv)
    return (tp.numpy().view(np.uint32).copy(), tm.numpy().view(np.uint32).copy(),
            tv.numpy().view(np.uint32).copy(), th.numpy().view(np.uint16).copy())


def main():
    ref = oracle.reference_module()
    if ref is None:
        sys.exit("oracle/_ref is not built (make -f oracle/Makefile ref) or this CPU cannot run it")
    out = {}
    p, g, m, v = shared_inputs()
    out.update(in_p=p.view(np.uint32), in_g=g.view(np.uint32), in_m=m.view(np.uint32), in_v=v.view(np.uint32))

    cases, oid = [], 100
    for adamw in (True, False):
        for wd in (0.0, 0.01):
            for bias_correction in (True, False):
                for step in (1, 2, 10, 100, 1000):
                    case = dict(step=step, adamw_mode=adamw, wd=wd, bias_correction=bias_correction,
                                lr=1e-4, betas=(0.9, 0.999), eps=1e-8)
                    ref.create_adam(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, adamw, False)
                    rp, rm, rv, rh = run_ref(ref, oid, p, g, m, v, step=step, lr=1e-4, betas=(0.9, 0.999), eps=1e-8,
                                             wd=wd, bias_correction=bias_correction)
                    ref.destroy_adam(oid)
                    oid += 1
                    k = len(cases)
                    out[f"case_{k}_p"], out[f"case_{k}_m"], out[f"case_{k}_v"], out[f"case_{k}_h"] = rp, rm, rv, rh
                    cases.append(case)
    # other betas / eps / lr, so that every scalar is exercised away from its default
    for step, lr, betas, eps, wd in ((3, 3e-3, (0.8, 0.95), 1e-6, 0.1), (50, 1.0, (0.0, 0.5), 1e-3, 1.0),
                                     (12345, 6e-5, (0.95, 0.9999), 1e-12, 1e-4)):
        case = dict(step=step, adamw_mode=True, wd=wd, bias_correction=True, lr=lr, betas=betas, eps=eps)
        ref.create_adam(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, False)
        rp, rm, rv, rh = run_ref(ref, oid, p, g, m, v, step=step, lr=lr, betas=betas, eps=eps, wd=wd, bias_correction=True)
        ref.destroy_adam(oid)
        oid += 1
        k = len(cases)
        out[f"case_{k}_p"], out[f"case_{k}_m"], out[f"case_{k}_v"], out[f"case_{k}_h"] = rp, rm, rv, rh
        cases.append(case)
    out["cases"] = np.frombuffer(json.dumps(cases).encode(), dtype=np.uint8)

    for n in TAIL_SIZES:
        ref.create_adam(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, False)
        rp, rm, rv, rh = run_ref(ref, oid, p[:n], g[:n], m[:n], v[:n], step=7, lr=1e-4, betas=(0.9, 0.999), eps=1e-8,
                                 wd=0.01, bias_correction=True)
        ref.destroy_adam(oid)
        oid += 1
        out[f"tail_{n}_p"], out[f"tail_{n}_m"], out[f"tail_{n}_v"], out[f"tail_{n}_h"] = rp, rm, rv, rh

    # the CPU-runnable configuration at its real size, kept as digests
    n1 = 1 << 20
    rng = np.random.default_rng(0)
    tp = torch.from_numpy(rng.normal(0, 0.02, n1).astype(np.float32))
    tm, tv = torch.zeros(n1), torch.zeros(n1)
    ref.create_adam(oid, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, False)
    digests = []
    for t in range(1, 11):
        tg = torch.from_numpy(rng.normal(0, 1e-3, n1).astype(np.float32))
        ref.adam_update(oid, t, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, tp, tg, tm, tv)
        hsh = hashlib.sha256()
        for x in (tp, tm, tv):
            hsh.update(x.numpy().tobytes())
        digests.append(hsh.hexdigest())
    out["cfg1_digest"] = np.frombuffer(json.dumps(digests).encode(), dtype=np.uint8)

    # same step twice from identical state: the cached beta^t branch (cpu_adam.h:75-83)
    a = run_ref(ref, oid, p, g, m, v, step=10, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, wd=0.01, bias_correction=True)
    b = run_ref(ref, oid, p, g, m, v, step=10, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, wd=0.01, bias_correction=True)
    out["repeat_same_step_equal"] = np.array([int(all(np.array_equal(x, y) for x, y in zip(a, b)))], dtype=np.uint8)
    ref.destroy_adam(oid)

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "adam_reference.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {os.path.getsize(path)} bytes, {len(cases)} cases, flavour {ref.flavour}")


if __name__ == "__main__":
    main()
