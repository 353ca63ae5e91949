"""Random sequences of offloaded steps against the CPU oracle.

Each seed draws an engine (chunk size, number of slots, transfer mode) and a sequence of steps on
slices of one pinned state: any start element and length, gradients of any type on the GPU or in
pinned host memory, the 16-bit copy nowhere, on the GPU or in pinned host memory, a control record
that skips or scales, blocking or not, some of the steps inside a window of either kind. Overlapping
slices stepped back to back exercise the ordering between a step's write-back and the next step's
reads. After the last step the whole state and both copies must equal the oracle's."""
import os

import numpy as np
import pytest
import torch

from _util import CODE, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu

HP = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
G_DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _control(cuda, skip, mult):
    rec = torch.zeros(4, dtype=torch.float32, device=cuda)
    rec[1], rec[3] = mult, 1.0
    rec.view(torch.int32)[0] = skip
    return rec


@pytest.mark.parametrize("seed", range(int(os.environ.get("FT_FUZZ_SEEDS", "12"))))
def test_random_offloaded_steps(cuda, oracle, seed):
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.memory import pinned_empty
    rng = np.random.default_rng(10_000 + seed)
    piece = int(rng.choice([0, 1 << 20]))  # windows in one piece, or in pieces of about 1 Mi elements
    total = int(rng.integers(50_000, 3_200_000 if piece else 1_200_000))
    chunk = 1 << int(rng.integers(14, 19))
    slots, mode = int(rng.integers(2, 5)), int(rng.integers(0, 5))
    half_dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
    print(f"[offload fuzz] seed={seed} total={total} chunk={chunk} slots={slots} mode={mode} piece={piece} half={half_dtype}", flush=True)
    eng = FlexTrainCPUAdam(offload_chunk_elems=chunk, offload_slots=slots, offload_mode=mode, offload_window_piece_elems=piece, **HP)
    P, M, V = (pinned_empty(total, torch.float32) for _ in range(3))
    P.copy_(torch.from_numpy(rng.normal(0, 0.02, total).astype(np.float32)))
    M.copy_(torch.from_numpy(rng.normal(0, 1e-4, total).astype(np.float32)))
    V.copy_(torch.from_numpy(rng.uniform(0, 1e-6, total).astype(np.float32)))
    H_dev = torch.full((total,), 3.0, dtype=half_dtype, device=cuda)
    H_host = pinned_empty(total, half_dtype)
    H_host.fill_(5.0)
    pn, mn, vn = P.numpy().copy(), M.numpy().copy(), V.numpy().copy()
    hn = {"dev": half_bits(H_dev).copy(), "host": half_bits(H_host).copy()}
    keep = []  # pinned gradients must outlive the non-blocking steps that read them (GPU tensors, the control
    # record included, are covered by the step's own guard on the caller's stream)

    def one_step(lo, hi, step, blocking):
        n = hi - lo
        g_dtype = G_DTYPES[int(rng.integers(0, 3))]
        g = (torch.randn(n, device=cuda) * 1e-3 * 64).to(g_dtype)
        if rng.integers(0, 3) == 0:
            g_host = pinned_empty(n, g_dtype)
            g_host.copy_(g)
            torch.cuda.synchronize()
            g = g_host
        keep.append(g)
        where = ["none", "dev", "host"][int(rng.integers(0, 3))]
        h = None if where == "none" else (H_dev if where == "dev" else H_host)[lo:hi]
        kind = int(rng.integers(0, 4))  # 0, 1: plain multiplier; 2: control record that scales; 3: control record that skips
        mult = 1.0 / 64
        kwargs = dict(grad_mult=mult) if kind < 2 else dict(grad_mult=99.0, control=_control(cuda, int(kind == 3), mult))
        eng._step({"step": step}, h, P[lo:hi], g, M[lo:hi], V[lo:hi], blocking=blocking, **kwargs)
        if kind == 3:
            return
        gn = to_np(g)
        if g_dtype == torch.float16:
            gn = gn.view(np.uint16)
        ps, ms, vs = pn[lo:hi].copy(), mn[lo:hi].copy(), vn[lo:hi].copy()
        hs = np.zeros(n, np.uint16)
        oracle.adam_step(ps, gn, ms, vs, step=step, grad_mult=mult, g_dtype=CODE[g_dtype], half_out=hs, half_dtype=CODE[half_dtype], **HP)
        pn[lo:hi], mn[lo:hi], vn[lo:hi] = ps, ms, vs
        if where != "none":
            hn[where][lo:hi] = hs

    def random_slice(lo_bound, hi_bound):
        lo = int(rng.integers(lo_bound, hi_bound))
        hi = int(rng.integers(lo + 1, hi_bound + 1))
        return lo, hi

    step = 0
    for _ in range(int(rng.integers(3, 8))):
        step += 1
        if rng.integers(0, 3) == 0:  # a window over part of the state, stepped in shares that tile it exactly once
            wlo, whi = random_slice(0, total - 1)
            write_through = bool(rng.integers(0, 2))
            token = eng.open_window(P[wlo:whi], M[wlo:whi], V[wlo:whi], write_through=write_through)
            cuts = sorted(set([wlo, whi] + [int(c) for c in rng.integers(wlo, whi, int(rng.integers(0, 4)))]))
            order = list(zip(cuts[:-1], cuts[1:]))
            rng.shuffle(order)
            for lo, hi in order:
                if hi > lo:
                    one_step(lo, hi, step, blocking=False)
            if whi < total and rng.integers(0, 2):  # and one outside it while it is open
                one_step(*random_slice(whi, total), step, blocking=bool(rng.integers(0, 2)))
            eng.close_window(token)
        else:
            one_step(*random_slice(0, total), step, blocking=bool(rng.integers(0, 2)))
    eng.stream_wait(write_back=True)
    eng.synchronize()
    torch.cuda.synchronize()
    worst = dict(p=max_ulp(P.numpy(), pn), m=max_ulp(M.numpy(), mn), v=max_ulp(V.numpy(), vn))
    for where, t in (("dev", H_dev), ("host", H_host)):
        bits = half_bits(t)
        worst["h_" + where] = max_ulp(bits, hn[where], bf16=True) if half_dtype == torch.bfloat16 \
            else max_ulp(bits.view(np.float16), hn[where].view(np.float16))
    print(f"[offload fuzz] seed={seed} worst ULP distance: {worst}", flush=True)
    assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and max(worst["h_dev"], worst["h_host"]) <= HALF_ULP, worst
