"""Random schedules through the per-unit optimizer pipeline, every unit checked against the CPU oracle.

Each seed draws a schedule the other coordinator tests do not combine: number of units and of
micro-batches, ragged share and group boundaries (shares that start at any element offset), where
the state lives (HBM, pinned host memory, some of each), windows of either kind, how resident units
are cut and on which stream they run, the accumulation type, loss scaling with an inf/nan planted
somewhere, stepping during backward, split between backward and the next forward pass (alpha), or
deferred to the next forward pass with or without clipping.
Bars as everywhere: fp32 state within 2 ULP, the 16-bit parameters within 1 (0 is what comes out)."""
import math
import os

import numpy as np
import pytest
import torch

from _util import CODE, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu


class _Unit:
    def __init__(self, paras):
        self.paras = paras


def _draw(seed):
    rng = np.random.default_rng(seed)
    cfg = dict(seed=seed)
    cfg["num_units"] = int(rng.integers(1, 5))
    cfg["micro_batches"] = int(rng.choice([1, 2, 3, 4, 6]))
    cfg["unit_numel"] = cfg["micro_batches"] * int(rng.integers(2_000, 20_000))
    cfg["padding"] = int(rng.integers(0, 100))
    n_groups = int(rng.integers(1, 4))
    real = cfg["unit_numel"] - cfg["padding"]
    cuts = sorted(set(int(c) for c in rng.integers(1, real - 1, n_groups - 1)))
    cfg["bounds"] = [0] + cuts + [real]
    cfg["group_args"] = [dict(lr=float(rng.choice([1e-4, 3e-4, 1e-3])), weight_decay=float(rng.choice([0.0, 0.01, 0.1])))
                         for _ in range(len(cfg["bounds"]) - 1)]
    cfg["offload"] = bool(rng.integers(0, 2))
    cfg["resident_units"] = int(rng.integers(0, cfg["num_units"] + 1)) if cfg["offload"] else 0
    cfg["unit_windows"] = [None, True, False][int(rng.integers(0, 3))]
    cfg["window_write_through"] = bool(rng.integers(0, 2))
    divisors = [d for d in range(1, cfg["micro_batches"] + 1) if cfg["micro_batches"] % d == 0]
    cfg["resident_shares"] = int(rng.choice(divisors))
    cfg["step_stream"] = bool(rng.integers(0, 2))
    cfg["gradacc"] = [None, torch.float32][int(rng.integers(0, 2))]
    cfg["scaled"] = bool(rng.integers(0, 2))
    cfg["defer"] = bool(rng.integers(0, 2))
    cfg["max_grad_norm"] = 0.05 if (cfg["defer"] and rng.integers(0, 2)) else None
    # the share of every unit's step that runs during the next forward pass (0: all during backward)
    cfg["alpha"] = 0.0 if cfg["defer"] or rng.integers(0, 2) else float(rng.uniform(0.02, 0.98))
    cfg["iterations"] = 3
    # (iteration, unit, micro-batch, element) of a planted inf/nan; checked only where gradients are scaled
    cfg["planted"] = (int(rng.integers(1, 4)), int(rng.integers(0, cfg["num_units"])), int(rng.integers(0, cfg["micro_batches"])),
                      int(rng.integers(0, real)), [float("inf"), float("-inf"), float("nan")][int(rng.integers(0, 3))]) \
        if cfg["scaled"] and rng.integers(0, 3) else None
    return cfg


@pytest.mark.parametrize("seed", range(int(os.environ.get("FT_FUZZ_SEEDS", "16"))))
def test_random_schedule(cuda, oracle, seed):
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    from flextrain_amd.loss_scaler import DynamicLossScaler
    cfg = _draw(seed)
    print(f"[coordinator fuzz] {cfg}", flush=True)
    torch.manual_seed(seed)
    num_units, mbs, n, bounds = cfg["num_units"], cfg["micro_batches"], cfg["unit_numel"], cfg["bounds"]
    dtype = torch.float16 if cfg["scaled"] else torch.bfloat16
    real = bounds[-1]
    flat, per_group = [], [[] for _ in cfg["group_args"]]
    for u in range(num_units):
        f = torch.zeros(n, dtype=dtype, device=cuda)
        f[:real] = (torch.randn(real, device=cuda) * 0.02).to(dtype)
        flat.append(f)
        for k in range(len(per_group)):
            per_group[k].append(torch.nn.Parameter(f[bounds[k]:bounds[k + 1]]))
    groups = [dict(params=per_group[k], **cfg["group_args"][k]) for k in range(len(per_group))]
    opt = FlexTrainAdam(groups, lr=1e-4, unit_parameter_map={u: _Unit([g[u] for g in per_group]) for u in range(num_units)},
                        aligned_unit_numel=n, offload=cfg["offload"])
    scaler = DynamicLossScaler(init_scale=1024.0, delayed_shift=1, scale_window=1000) if cfg["scaled"] else None
    coord = FlexTrainOptsCoordinator()
    coord.initialize(opt, flat, mbs, offload=cfg["offload"], device=cuda, resident_units=cfg["resident_units"],
                     unit_windows=cfg["unit_windows"], window_write_through=cfg["window_write_through"],
                     resident_shares=cfg["resident_shares"], step_stream=cfg["step_stream"], gradacc_dtype=cfg["gradacc"],
                     loss_scaler=scaler, max_grad_norm=cfg["max_grad_norm"], defer_to_forward=cfg["defer"], alpha=cfg["alpha"])
    segments = [(bounds[k], bounds[k + 1] if k + 1 < len(bounds) - 1 else n, groups[k]) for k in range(len(groups))]
    state = [(to_np(f.float()).copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)) for f in flat]
    expected_half = [half_bits(f).copy() for f in flat]
    gen = torch.Generator(device=cuda).manual_seed(1000 + seed)

    def forward_pass():
        coord.warmup_forward_pipeline()
        for u in range(num_units):
            coord.pre_unit_forward(u)
            for mb in range(mbs):
                coord.post_micro_batch_forward(u, mb)

    def apply(units, step, grad_mult, accumulated):
        for u in units:
            pn, mn, vn = state[u]
            gn = accumulated[u]
            hn = expected_half[u].copy()
            for lo, hi, group in segments:
                hs = np.zeros(hi - lo, np.uint16)
                ps, ms, vs = pn[lo:hi].copy(), mn[lo:hi].copy(), vn[lo:hi].copy()
                oracle.adam_step(ps, np.ascontiguousarray(gn[lo:hi]), ms, vs, step=step, lr=group["lr"], weight_decay=group["weight_decay"],
                                 grad_mult=grad_mult, g_dtype=CODE[torch.float32] if cfg["gradacc"] is not None else CODE[dtype],
                                 half_out=hs, half_dtype=CODE[dtype])
                pn[lo:hi], mn[lo:hi], vn[lo:hi], hn[lo:hi] = ps, ms, vs, hs
            expected_half[u] = hn

    def check(tag):
        for u, (pn, mn, vn) in enumerate(state):
            m, v = coord.unit_optimizer_states(u)
            worst = dict(p=max_ulp(to_np(coord.unit_master_parameter(u)), pn), m=max_ulp(to_np(m), mn), v=max_ulp(to_np(v), vn),
                         h=max_ulp(half_bits(flat[u]), expected_half[u], bf16=True) if dtype == torch.bfloat16
                         else max_ulp(half_bits(flat[u]).view(np.float16), expected_half[u].view(np.float16)))
            assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP, (tag, u, worst, cfg)

    applied, overflows = 0, []
    for iteration in range(1, cfg["iterations"] + 1):
        if cfg["defer"] or cfg["alpha"] > 0:
            forward_pass()
            coord.synchronize()
            check(f"before iteration {iteration}")
        if not cfg["defer"]:
            opt.update_states()
        scale = coord.loss_scale
        accumulated, bad_units, sumsq = {}, set(), 0.0
        for u in reversed(range(num_units)):
            buf = coord.pre_unit_backward(u)
            acc = np.zeros(n, np.float32) if cfg["gradacc"] is not None else None
            for mb in range(mbs):
                g = (torch.randn(n, device=cuda, generator=gen) * 1e-3 * scale).to(dtype)
                g[real:] = 0  # padding never receives gradient
                if cfg["planted"] is not None and cfg["planted"][:3] == (iteration, u, mb):
                    g[cfg["planted"][3]] = cfg["planted"][4]
                    bad_units.add(u)
                if cfg["gradacc"] is None:
                    buf += g
                else:
                    buf.copy_(g)
                    oracle.grad_accumulate(acc, CODE[torch.float32], half_bits(g).copy(), CODE[dtype])
                if mb == mbs - 1:
                    accumulated[u] = acc if cfg["gradacc"] is not None else (half_bits(buf) if dtype == torch.float16 else to_np(buf)).copy()
                coord.post_micro_batch_backward(u, mb)
            values = torch.from_numpy(acc).double() if cfg["gradacc"] is not None else buf.double().cpu()
            values = values / scale
            sumsq += float((values[torch.isfinite(values)] ** 2).sum())
        decision = coord.clear_backward_pipeline()
        overflow = bool(bad_units)
        overflows.append(overflow)
        if scaler is None and cfg["max_grad_norm"] is None:
            assert decision is None
        else:
            assert decision.overflow == overflow, cfg
        if cfg["defer"]:
            if overflow:
                assert coord.last_skipped_units == list(range(num_units))
                continue
            grad_mult = float(np.float32(1.0 / scale)) if scaler is not None else 1.0
            if cfg["max_grad_norm"] is not None:
                norm = math.sqrt(sumsq)
                assert abs(decision.grad_norm - norm) <= 1e-6 * norm, cfg
                assert np.float32(decision.grad_mult) == oracle.combined_multiplier(scale, decision.clip_coef)
                grad_mult = decision.grad_mult
            applied += 1
            opt.update_states()
            apply(range(num_units), applied, grad_mult, accumulated)
        else:
            first_bad = max(bad_units) if bad_units else -1  # that unit and every unit stepped after it are skipped
            if bad_units and coord._defer:  # alpha rounded up to the whole slice: nothing is stepped before the global decision
                first_bad = num_units - 1
            if scaler is not None:
                assert coord.last_skipped_units == list(range(first_bad + 1)), cfg
            apply([u for u in range(num_units) if u > first_bad], iteration,
                  float(np.float32(1.0 / scale)) if scaler is not None else 1.0, accumulated)
            if cfg["alpha"] == 0:
                check(f"after iteration {iteration}")
    if cfg["defer"] or cfg["alpha"] > 0:
        forward_pass()
        coord.synchronize()
        check("final")
    if scaler is not None:
        assert coord.loss_scale == oracle.loss_scale_trace(overflows, 1024.0, delayed_shift=1)[-1]
