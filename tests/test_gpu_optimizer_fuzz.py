"""Random models through FlexTrainAdam's own step (the parameters that belong to no layer unit),
every parameter checked against the CPU oracle.

Each seed draws parameter shapes and their grouping (a group's parameters need not be neighbours in
the flat buffer), hyper-parameters per group, the parameter type, where the master state lives, the
accumulation type, loss scaling with an inf/nan planted in some iteration, clipping, and whether the
per-step scalars travel by value or live in device memory. Four iterations each; bars as everywhere
(fp32 state within 2 ULP, 16-bit parameters within 1; 0 is what comes out)."""
import math
import os

import numpy as np
import pytest
import torch

from _util import CODE, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(int(os.environ.get("FT_FUZZ_SEEDS", "16"))))
def test_random_model(cuda, oracle, seed):
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.loss_scaler import DynamicLossScaler
    rng = np.random.default_rng(20_000 + seed)
    torch.manual_seed(seed)
    dtype = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(0, 3))]
    n_groups = int(rng.integers(1, 4))
    groups = [dict(params=[], lr=float(rng.choice([1e-4, 1e-3, 3e-3])), weight_decay=float(rng.choice([0.0, 0.01, 0.1])),
                   betas=[(0.9, 0.999), (0.8, 0.99)][int(rng.integers(0, 2))]) for _ in range(n_groups)]
    params, owner = [], []
    for _ in range(int(rng.integers(1, 7))):
        shape = [(int(rng.integers(1, 300)),), (int(rng.integers(1, 200)), int(rng.integers(1, 200)))][int(rng.integers(0, 2))]
        p = torch.nn.Parameter((torch.randn(shape, device=cuda) * 0.02).to(dtype))
        k = int(rng.integers(0, n_groups))
        groups[k]["params"].append(p)
        params.append(p)
        owner.append(k)
    groups = [g for g in groups if g["params"]]
    # the optimizer lays parameters out in the caller's order: group by group
    order = [p for g in groups for p in g["params"]]
    group_of = {id(p): g for g in groups for p in g["params"]}
    offload = bool(rng.integers(0, 2))
    gradacc = torch.float32 if (dtype != torch.float32 and rng.integers(0, 2)) else None
    scaled = dtype == torch.float16 or bool(rng.integers(0, 2))
    max_norm = [None, 0.5][int(rng.integers(0, 2))]
    capturable = (not offload) and bool(rng.integers(0, 2))
    planted_iteration = int(rng.integers(1, 5)) if scaled and rng.integers(0, 2) else None
    print(f"[optimizer fuzz] seed={seed} dtype={dtype} params={[tuple(p.shape) for p in order]} groups={len(groups)} offload={offload} "
          f"gradacc={gradacc} scaled={scaled} max_norm={max_norm} capturable={capturable} planted={planted_iteration}", flush=True)
    scaler = DynamicLossScaler(init_scale=256.0, delayed_shift=1, scale_window=1000) if scaled else None
    state = [(to_np(p.detach().float().flatten()).copy(), np.zeros(p.numel(), np.float32), np.zeros(p.numel(), np.float32)) for p in order]
    opt = FlexTrainAdam(groups, lr=1e-4, offload=offload, gradacc_dtype=gradacc, loss_scaler=scaler, max_grad_norm=max_norm,
                        capturable=capturable)
    overflows = []
    for iteration in range(1, 5):
        opt.update_states()
        scale = float(scaler.loss_scale) if scaler is not None else 1.0
        grads, sumsq = [], 0.0
        for p in order:
            g = (torch.randn(p.shape, device=cuda) * 0.05 * scale).to(dtype)
            if iteration == planted_iteration and p is order[-1]:
                g.view(-1)[int(rng.integers(0, p.numel()))] = [float("inf"), float("nan")][int(rng.integers(0, 2))]
            grads.append(g)
            unscaled = g.double() / scale
            sumsq += float((unscaled[torch.isfinite(unscaled)] ** 2).sum())
        if gradacc is None:
            for p, g in zip(order, grads):
                p.grad.copy_(g)
        else:  # the wider accumulator is fed by hooks: backward of an identity hands each hook exactly g
            for p, g in zip(order, grads):
                (p * 1).backward(g)
        applied = opt.step()
        overflow = iteration == planted_iteration
        overflows.append(overflow)
        assert applied == (not overflow)
        grad_mult = 1.0
        if scaler is not None or max_norm is not None:
            decision = opt._guard.read()
            assert decision.overflow == overflow
            if not overflow:
                norm = math.sqrt(sumsq)
                assert abs(decision.grad_norm - norm) <= 1e-6 * norm
                grad_mult = decision.grad_mult
                assert np.float32(grad_mult) == oracle.combined_multiplier(scale, decision.clip_coef if max_norm is not None else 1.0)
        if overflow:
            continue
        for (pn, mn, vn), p, g in zip(state, order, grads):
            group = group_of[id(p)]
            g_used = g.float() if gradacc is not None else g
            gn = to_np(g_used.flatten())
            if g_used.dtype == torch.float16:
                gn = gn.view(np.uint16)
            oracle.adam_step(pn, gn, mn, vn, step=iteration, lr=group["lr"], betas=group["betas"], weight_decay=group["weight_decay"],
                             grad_mult=grad_mult, g_dtype=CODE[g_used.dtype])
    torch.cuda.synchronize()
    offset = 0
    for (pn, mn, vn), p in zip(state, order):
        n = p.numel()
        master = opt._master_para[offset:offset + n]
        worst = max_ulp(to_np(master), pn)
        assert worst <= MASTER_ULP, (seed, tuple(p.shape), worst)
        got = p.detach().flatten()
        if dtype == torch.float32:
            assert max_ulp(to_np(got), pn) <= MASTER_ULP
        else:
            want = torch.from_numpy(pn).to(dtype)  # round to nearest even, as the kernel's copy-out does
            wb, gb = half_bits(want), half_bits(got)
            worst_h = max_ulp(gb, wb, bf16=True) if dtype == torch.bfloat16 else max_ulp(gb.view(np.float16), wb.view(np.float16))
            assert worst_h <= HALF_ULP, (seed, tuple(p.shape), worst_h)
        offset += n
    assert all(g["step"] == 4 for g in groups)
    if scaler is not None:
        assert scaler.loss_scale == oracle.loss_scale_trace(overflows, 256.0, delayed_shift=1)[-1]
