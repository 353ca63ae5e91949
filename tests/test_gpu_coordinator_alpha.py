"""The forward / backward split of a unit's step (the reference's alpha split,
``flextrain/memory/coordinator/optimizer.py:144-175,352-492,605-696``) in the per-unit pipeline, driven the
way the reference's engine drives it (``flextrain/engine.py:353-399``: forward pass with the
forward-side hooks, ``update_states()``, backward pass with the backward-side hooks, hooks handed a
task object with ``.unit`` and ``.micro_batch``).

Whatever alpha is, every element of every unit is stepped exactly once per iteration with that
iteration's step count, so the state must equal the oracle's AdamW trajectory bit for bit; only WHEN a
share is stepped (during backward, or during the next forward pass) changes.
"""
import os
from collections import namedtuple

import numpy as np
import pytest
import torch

from _util import CODE, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu

LLMTask = namedtuple("LLMTask", ["unit", "micro_batch"])  # flextrain/scheduler.py:5-13


class _Unit:
    def __init__(self, paras):
        self.paras = paras


def _build(cuda, *, num_units, unit_numel, micro_batches, offload, dtype=torch.bfloat16, capturable=False, **kwargs):
    """Units of a weight (decay) and a bias (no decay, other lr) whose boundary falls inside a slice."""
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    w_numel = unit_numel - 7001
    flat = [(torch.randn(unit_numel, device=cuda) * 0.02).to(dtype) for _ in range(num_units)]
    weights = [torch.nn.Parameter(f[:w_numel]) for f in flat]
    biases = [torch.nn.Parameter(f[w_numel:]) for f in flat]
    decay = {"params": weights, "weight_decay": 0.1}
    plain = {"params": biases, "weight_decay": 0.0, "lr": 3e-4}
    opt = FlexTrainAdam([decay, plain], lr=1e-4, unit_parameter_map={u: _Unit([weights[u], biases[u]]) for u in range(num_units)},
                        aligned_unit_numel=unit_numel, offload=offload, capturable=capturable)
    coord = FlexTrainOptsCoordinator()
    coord.initialize(opt, flat, micro_batches, offload=offload, device=cuda, **kwargs)
    state = [(to_np(f.float()).copy(), np.zeros(unit_numel, np.float32), np.zeros(unit_numel, np.float32)) for f in flat]
    return flat, (decay, plain), w_numel, opt, coord, state


def _forward_pass(coord, num_units, micro_batches, as_tasks=True):
    coord.warmup_forward_pipeline()
    for u in range(num_units):
        coord.pre_unit_forward(u)
        for mb in range(micro_batches):
            if as_tasks:
                coord.pre_micro_batch_forward(LLMTask(u, mb))
                coord.post_micro_batch_forward(LLMTask(u, mb))
            else:
                coord.post_micro_batch_forward(u, mb)


def _backward_pass(coord, num_units, micro_batches, unit_numel, gen, cuda, dtype=torch.bfloat16, scale=1.0, plant=None):
    accumulated = {}
    coord.warmup_backward_pipeline()
    for u in reversed(range(num_units)):
        buf = coord.pre_unit_backward(u)
        for mb in range(micro_batches):
            coord.pre_micro_batch_backward(LLMTask(u, mb))
            g = (torch.randn(unit_numel, device=cuda, generator=gen) * 1e-3 * scale).to(dtype)
            if plant is not None and plant == (u, mb):
                g[unit_numel // 2 + 3] = float("inf")
            buf += g
            if mb == micro_batches - 1:
                accumulated[u] = buf.clone()
            coord.post_micro_batch_backward(LLMTask(u, mb))
    return accumulated, coord.clear_backward_pipeline()


def _oracle_unit(oracle, state_u, grad, groups, w_numel, unit_numel, step, g_dtype, half_dtype, grad_mult=1.0):
    pn, mn, vn = state_u
    gn = to_np(grad)
    if gn.dtype == np.float16:
        gn = gn.view(np.uint16)
    hn = np.zeros(unit_numel, np.uint16)
    for lo, hi, group in ((0, w_numel, groups[0]), (w_numel, unit_numel, groups[1])):
        hs = np.zeros(hi - lo, np.uint16)
        ps, ms, vs = pn[lo:hi].copy(), mn[lo:hi].copy(), vn[lo:hi].copy()
        oracle.adam_step(ps, np.ascontiguousarray(gn[lo:hi]), ms, vs, step=step, lr=group.get("lr", 1e-4),
                         weight_decay=group["weight_decay"], grad_mult=grad_mult, g_dtype=CODE[g_dtype], half_out=hs,
                         half_dtype=CODE[half_dtype])
        pn[lo:hi], mn[lo:hi], vn[lo:hi], hn[lo:hi] = ps, ms, vs, hs
    return hn


def _check(tag, coord, flat, state, expected_half, bf16=True):
    for u, (pn, mn, vn) in enumerate(state):
        m, v = coord.unit_optimizer_states(u)
        got_h, want_h = half_bits(flat[u]), expected_half[u]
        worst = dict(p=max_ulp(to_np(coord.unit_master_parameter(u)), pn), m=max_ulp(to_np(m), mn), v=max_ulp(to_np(v), vn),
                     h=max_ulp(got_h, want_h, bf16=True) if bf16 else max_ulp(got_h.view(np.float16), want_h.view(np.float16)))
        print(f"[{tag} unit={u}] worst ULP distance: {worst}", flush=True)
        assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP, (tag, u, worst)


@pytest.mark.parametrize("alpha", [0.0, 0.25, 0.6, 1.0])
@pytest.mark.parametrize("offload,windows,resident_units", [(False, False, 0), (True, True, 0), (True, False, 0), (True, True, 1)])
def test_alpha_split_matches_oracle(cuda, oracle, alpha, offload, windows, resident_units):
    torch.manual_seed(3)
    num_units, micro_batches, unit_numel = 3, 4, 1 << 18
    flat, groups, w_numel, opt, coord, state = _build(
        cuda, num_units=num_units, unit_numel=unit_numel, micro_batches=micro_batches, offload=offload, alpha=alpha,
        unit_windows=windows, resident_units=resident_units)
    slice_numel = unit_numel // micro_batches
    want_fwd = 0 if alpha == 0 else slice_numel if alpha == 1 else -(-int(np.ceil(alpha * slice_numel)) // 256) * 256
    assert (coord._mb_fwd_numel, coord._mb_bwd_numel) == (want_fwd, slice_numel - want_fwd)
    assert len(coord.unit_share_blocks(0, forward=True)) == (3 if alpha > 0 else 0)
    assert len(coord.unit_share_blocks(0, forward=False)) == (3 if alpha < 1 else 0)
    if 0 < alpha < 1:
        assert coord.unit_share_blocks(0, True)[0].numel() == want_fwd * micro_batches
        assert coord.unit_share_blocks(0, False)[0].numel() == unit_numel - want_fwd * micro_batches
    gen = torch.Generator(device=cuda).manual_seed(4)
    expected_half = [half_bits(f).copy() for f in flat]
    pending = None  # gradients whose forward shares are still to be stepped
    for iteration in (1, 2, 3):
        _forward_pass(coord, num_units, micro_batches, as_tasks=iteration != 2)
        coord.synchronize()
        if pending is not None:
            # every share of the previous iteration has now been stepped
            for u in range(num_units):
                expected_half[u] = _oracle_unit(oracle, state[u], pending[u], groups, w_numel, unit_numel, iteration - 1,
                                                torch.bfloat16, torch.bfloat16)
            _check(f"alpha={alpha} offload={offload} windows={windows} after forward of it={iteration}", coord, flat, state, expected_half)
        opt.update_states()  # the reference's order: between the forward and the backward pass
        pending, decision = _backward_pass(coord, num_units, micro_batches, unit_numel, gen, cuda)
        assert decision is None
        if alpha > 0:  # backward may not start again before the forward shares have been stepped
            with pytest.raises(RuntimeError, match="have not been applied"):
                coord.pre_unit_backward(num_units - 1)
    _forward_pass(coord, num_units, micro_batches)
    coord.synchronize()
    for u in range(num_units):
        expected_half[u] = _oracle_unit(oracle, state[u], pending[u], groups, w_numel, unit_numel, 3, torch.bfloat16, torch.bfloat16)
    _check(f"alpha={alpha} offload={offload} windows={windows} final", coord, flat, state, expected_half)
    assert groups[0]["step"] == groups[1]["step"] == 3


def test_backward_share_runs_during_backward_and_forward_share_during_forward(cuda, oracle):
    """Which elements move when: after the backward pass of an iteration exactly the backward-share
    elements (behind the first ceil(alpha * slice) elements of every micro-batch's slice) have new
    values, the forward-share elements follow in the next forward pass."""
    torch.manual_seed(8)
    num_units, micro_batches, unit_numel = 2, 4, 1 << 16
    flat, groups, w_numel, opt, coord, state = _build(
        cuda, num_units=num_units, unit_numel=unit_numel, micro_batches=micro_batches, offload=False, alpha=0.25)
    before = [coord.unit_master_parameter(u).clone() for u in range(num_units)]
    gen = torch.Generator(device=cuda).manual_seed(5)
    _forward_pass(coord, num_units, micro_batches)
    opt.update_states()
    _backward_pass(coord, num_units, micro_batches, unit_numel, gen, cuda)
    slice_numel, fwd = unit_numel // micro_batches, coord._mb_fwd_numel
    assert fwd == 4096
    in_fwd = (torch.arange(unit_numel, device=cuda) % slice_numel) < fwd
    for u in range(num_units):
        changed = coord.unit_master_parameter(u) != before[u]
        assert not changed[in_fwd].any() and changed[~in_fwd].float().mean() > 0.99
    _forward_pass(coord, num_units, micro_batches)
    coord.synchronize()
    for u in range(num_units):
        changed = coord.unit_master_parameter(u) != before[u]
        assert changed[in_fwd].float().mean() > 0.99


@pytest.mark.parametrize("offload", [False, True])
def test_split_state_files_and_resume(cuda, tmp_path, offload):
    """With two shares a unit has two files, `.swp.0` (forward share, unpadded) and `.swp.1` (backward
    share, padded to whole pages), as in the reference; a run resumed from them continues bit-exactly."""
    from flextrain_amd.state_files import opts_file_layout
    num_units, micro_batches, unit_numel = 2, 2, 1 << 16

    def build():
        torch.manual_seed(2)
        return _build(cuda, num_units=num_units, unit_numel=unit_numel, micro_batches=micro_batches, offload=offload, alpha=0.3)

    def iterate(opt, coord, seed):
        gen = torch.Generator(device=cuda).manual_seed(seed)
        _forward_pass(coord, num_units, micro_batches)
        opt.update_states()
        _backward_pass(coord, num_units, micro_batches, unit_numel, gen, cuda)

    flat_a, _, _, opt_a, coord_a, _ = build()
    iterate(opt_a, coord_a, 11)
    iterate(opt_a, coord_a, 12)
    _forward_pass(coord_a, num_units, micro_batches)
    coord_a.synchronize()

    flat_b, groups_b, _, opt_b, coord_b, _ = build()
    iterate(opt_b, coord_b, 11)
    with pytest.raises(RuntimeError, match="has not been applied"):
        coord_b.save_optimizer_states(str(tmp_path))  # forward shares of the iteration are still to come
    _forward_pass(coord_b, num_units, micro_batches)
    paths = coord_b.save_optimizer_states(str(tmp_path))
    assert [os.path.basename(p) for p in paths] == [f"rank0_OPTS_layer{u}.swp.{k}" for u in range(num_units) for k in (0, 1)]
    fwd_numel = coord_b._mb_fwd_numel * micro_batches
    for u in range(num_units):
        assert os.path.getsize(paths[2 * u]) == opts_file_layout(fwd_numel, 0)[2] == fwd_numel * 12
        assert os.path.getsize(paths[2 * u + 1]) == opts_file_layout(unit_numel - fwd_numel, 1)[2]
        assert os.path.getsize(paths[2 * u + 1]) % 4096 == 0
    for u in range(num_units):
        for forward in (True, False):
            for block in coord_b.unit_share_blocks(u, forward):
                block.fill_(float("nan"))
        flat_b[u].zero_()
    coord_b.load_optimizer_states(str(tmp_path))
    # the iteration that was interrupted by the save: its forward pass has run already
    opt_b.update_states()
    _backward_pass(coord_b, num_units, micro_batches, unit_numel, torch.Generator(device=cuda).manual_seed(12), cuda)
    _forward_pass(coord_b, num_units, micro_batches)
    coord_b.synchronize()
    assert groups_b[0]["step"] == 2
    for u in range(num_units):
        assert torch.equal(flat_a[u], flat_b[u])
        assert torch.equal(coord_a.unit_master_parameter(u).cpu(), coord_b.unit_master_parameter(u).cpu())
        for sa, sb in zip(coord_a.unit_optimizer_states(u), coord_b.unit_optimizer_states(u)):
            assert torch.equal(sa.cpu(), sb.cpu())


@pytest.mark.parametrize("offload,windows", [(False, False), (True, True)])
def test_a_unit_is_stepped_whole_or_not_at_all(cuda, oracle, offload, windows):
    """fp16 units, dynamic loss scale, alpha = 0.5, an inf in unit 1 on iteration 2. Unit 2 was stepped
    before the overflow was seen and keeps both shares of its update (the forward share with the scale
    its gradients were produced under, although the scaler has halved it by then); units 1 and 0 skip
    both shares. Scale trace = the reference's state machine."""
    from flextrain_amd.loss_scaler import DynamicLossScaler
    torch.manual_seed(12)
    num_units, micro_batches, unit_numel = 3, 2, 1 << 17
    scaler = DynamicLossScaler(init_scale=65536.0, delayed_shift=1, scale_window=1000)
    flat, groups, w_numel, opt, coord, state = _build(
        cuda, num_units=num_units, unit_numel=unit_numel, micro_batches=micro_batches, offload=offload, dtype=torch.float16,
        alpha=0.5, unit_windows=windows, loss_scaler=scaler)
    expected_half = [half_bits(f).copy() for f in flat]
    gen = torch.Generator(device=cuda).manual_seed(13)
    seen, overflows = [], []
    for iteration in (1, 2, 3):
        _forward_pass(coord, num_units, micro_batches)
        coord.synchronize()
        _check(f"whole-or-not offload={offload} before it={iteration}", coord, flat, state, expected_half, bf16=False)
        scale = coord.loss_scale
        seen.append(scale)
        opt.update_states()
        accumulated, decision = _backward_pass(coord, num_units, micro_batches, unit_numel, gen, cuda, dtype=torch.float16,
                                               scale=scale, plant=(1, 0) if iteration == 2 else None)
        overflows.append(decision.overflow)
        assert decision.overflow == (iteration == 2)
        assert coord.last_skipped_units == ([0, 1] if iteration == 2 else [])
        for u in range(num_units):
            if iteration == 2 and u <= 1:
                continue
            expected_half[u] = _oracle_unit(oracle, state[u], accumulated[u], groups, w_numel, unit_numel, iteration,
                                            torch.float16, torch.float16, grad_mult=float(np.float32(1.0 / scale)))
    _forward_pass(coord, num_units, micro_batches)
    coord.synchronize()
    _check(f"whole-or-not offload={offload} final", coord, flat, state, expected_half, bf16=False)
    assert seen + [coord.loss_scale] == oracle.loss_scale_trace(overflows, 65536.0, delayed_shift=1)


@pytest.mark.parametrize("alpha", [0.0, 0.5])
def test_device_resident_scalars_reach_the_unit_steps(cuda, oracle, alpha):
    """FlexTrainAdam(capturable=True) keeps every group's per-step scalars in device memory;
    update_states() only refreshes the pinned staging copies. The units' steps, which run before the
    optimizer's own step of the iteration (reference order: update_states, backward,
    optimizer.step()), must all the same read THIS iteration's step count and learning rate -- from the
    first iteration on, and under a learning-rate schedule."""
    torch.manual_seed(21)
    num_units, micro_batches, unit_numel = 2, 2, 1 << 16
    flat, groups, w_numel, opt, coord, state = _build(
        cuda, num_units=num_units, unit_numel=unit_numel, micro_batches=micro_batches, offload=False, alpha=alpha,
        capturable=True)
    assert all("hyper_record" in g for g in groups)
    gen = torch.Generator(device=cuda).manual_seed(22)
    expected_half = [half_bits(f).copy() for f in flat]
    pending = None
    lrs = {1: (1e-4, 3e-4), 2: (5e-5, 2e-4), 3: (2.5e-5, 1e-4)}
    for iteration in (1, 2, 3):
        _forward_pass(coord, num_units, micro_batches)
        coord.synchronize()
        if pending is not None:
            for u in range(num_units):
                expected_half[u] = _oracle_unit(oracle, state[u], pending[u], oracle_groups, w_numel, unit_numel, iteration - 1,
                                                torch.bfloat16, torch.bfloat16)
            _check(f"capturable alpha={alpha} after forward of it={iteration}", coord, flat, state, expected_half)
        groups[0]["lr"], groups[1]["lr"] = lrs[iteration]
        opt.update_states()
        oracle_groups = [dict(weight_decay=g["weight_decay"], lr=g["lr"]) for g in groups]
        pending, _ = _backward_pass(coord, num_units, micro_batches, unit_numel, gen, cuda)
        opt.step()  # non-layerwise parameters: none here, but the call is part of the reference's iteration
    _forward_pass(coord, num_units, micro_batches)
    coord.synchronize()
    for u in range(num_units):
        expected_half[u] = _oracle_unit(oracle, state[u], pending[u], oracle_groups, w_numel, unit_numel, 3, torch.bfloat16, torch.bfloat16)
    _check(f"capturable alpha={alpha} final", coord, flat, state, expected_half)
