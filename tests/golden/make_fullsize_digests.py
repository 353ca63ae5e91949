#!/usr/bin/env python3
"""Writes tests/golden/fullsize_digests.json: what the CPU oracle makes of the full-size 7B-layer
partition (202,383,360 elements, bf16 gradients, AdamW at t = 100, bf16 copy-out) when the inputs
come from the seeded generator (seed 0; substreams 0..3 = p ~ N(0, 0.02), m ~ N(0, 1e-4),
v ~ U(0, 1e-6], g ~ N(0, 1e-3) rounded to bf16).

The generator gives the same input bits on every machine, on the host and on the GPU, so a GPU
run can be checked against these digests without the oracle running beside it, and a digest made
on one CPU pins the oracle on another. Per array and per block of 2^24 elements the file holds
the sum of the raw bit patterns and a position-weighted sum (weight (i mod 65521) + 1), both
modulo 2^64: any changed, dropped, swapped or shifted element changes them.

    python -m flextrain_amd.build && make -f oracle/Makefile oracle && python tests/golden/make_fullsize_digests.py
"""
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
from flextrain_amd import synth  # noqa: E402

BLOCK = 1 << 24
HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)
N_7B_LAYER = 4 * 4096 ** 2 + 3 * 4096 * 11008 + 2 * 4096


def digests(bits: np.ndarray):
    """[(sum, weighted sum)] per block of BLOCK elements, modulo 2^64."""
    out = []
    weights = (np.arange(BLOCK, dtype=np.uint64) % np.uint64(65521)) + np.uint64(1)
    for lo in range(0, bits.shape[0], BLOCK):
        b = bits[lo:lo + BLOCK].astype(np.uint64)
        out.append((int(b.sum(dtype=np.uint64)), int((b * weights[:b.shape[0]]).sum(dtype=np.uint64))))
    return out


def main():
    n = N_7B_LAYER
    p, m, v = (torch.empty(n) for _ in range(3))
    g = torch.empty(n, dtype=torch.bfloat16)
    synth.fill_(p, 0, 0, scale=0.02)
    synth.fill_(m, 0, 1, scale=1e-4)
    synth.fill_(v, 0, 2, kind=synth.UNIFORM, scale=1e-6)
    synth.fill_(g, 0, 3, scale=1e-3)
    pn, mn, vn = p.numpy(), m.numpy(), v.numpy()
    gn = g.view(torch.int16).numpy().view(np.uint16)
    record = {"elements": n, "block": BLOCK, "step": 100, "hyper": {k: (list(x) if isinstance(x, tuple) else x) for k, x in HP.items()},
              "inputs": {"p": digests(pn.view(np.uint32)), "m": digests(mn.view(np.uint32)), "v": digests(vn.view(np.uint32)),
                         "g": digests(gn)}}
    hn = np.zeros(n, np.uint16)
    oracle.adam_step(pn, gn, mn, vn, step=100, g_dtype=oracle.BF16, half_out=hn, half_dtype=oracle.BF16, **HP)
    record["outputs"] = {"p": digests(pn.view(np.uint32)), "m": digests(mn.view(np.uint32)), "v": digests(vn.view(np.uint32)),
                         "h": digests(hn)}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fullsize_digests.json")
    with open(path, "w") as f:
        json.dump(record, f)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
