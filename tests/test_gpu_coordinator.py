"""GPU test of the per-unit optimizer pipeline: the schedule of the reference's optimizer
coordinator (step unit u+1 share by share while unit u runs backward) must leave every unit with
exactly the AdamW result of its accumulated gradient, for resident and offloaded master state."""
import numpy as np
import pytest
import torch

from _util import CODE, HALF_ULP, MASTER_ULP, half_bits, max_ulp, to_np

pytestmark = pytest.mark.gpu


class _Unit:
    def __init__(self, paras):
        self.paras = paras


# How units whose state is in HBM are stepped: the default (the caller's stream, one launch per unit),
# the reference's shape (one share per micro-batch), and either on the coordinator's own stream.
RESIDENT_MODES = {
    "caller_stream_one_share": {},
    "own_stream_share_per_micro_batch": dict(step_stream=True, resident_shares="micro_batches"),
    "caller_stream_share_per_micro_batch": dict(resident_shares="micro_batches"),
    "own_stream_one_share": dict(step_stream=True),
    "caller_stream_two_shares": dict(resident_shares=2),
}


def _with_resident_modes(cases):
    """Every case in the default mode; the cases with all state in HBM also with one share per
    micro-batch on the coordinator's own stream."""
    out = []
    for case in cases:
        for mode in list(RESIDENT_MODES)[:1 if case[0] else 2]:
            out.append(pytest.param(*case, mode, id="-".join(map(str, case)) + "-" + mode))
    return out


def _resident_kwargs(mode, micro_batches):
    kwargs = dict(RESIDENT_MODES[mode])
    if kwargs.get("resident_shares") == "micro_batches":
        kwargs["resident_shares"] = micro_batches
    return kwargs


@pytest.mark.parametrize("offload,windows", [(True, "copy_back"), (True, "write_through"), (True, "off"), (True, "auto"), (False, "off")])
def test_backward_pipeline_matches_oracle(cuda, oracle, offload, windows):
    _run_backward_pipeline(cuda, oracle, offload, windows, "gpu")


@pytest.mark.parametrize("half_layout", ["split", "split_odd", "host"])
@pytest.mark.parametrize("offload,windows", [(True, "copy_back"), (True, "off"), (False, "off")])
def test_half_parameters_on_gpu_and_host_pieces(cuda, oracle, offload, windows, half_layout):
    """The reference keeps a unit's low-precision parameters as a GPU part and a CPU part
    (``coordinator/parameter.py:470-519``): the update must write each element's new 16-bit value
    into the piece that holds it, wherever the cut falls (also at an odd element, where the vector
    alignments of the arrays disagree), for resident and offloaded master state."""
    _run_backward_pipeline(cuda, oracle, offload, windows, half_layout)


@pytest.mark.parametrize("windows,resident", [("copy_back", 1), ("off", 2), ("auto", 4)])
def test_some_units_resident_the_others_streamed(cuda, oracle, windows, resident):
    """offload with resident_units: units 0..R-1 keep their master state in HBM, the others stream
    from pinned host memory; the same results either way."""
    _run_backward_pipeline(cuda, oracle, True, windows, "gpu", resident_units=resident)


@pytest.mark.parametrize("mode", list(RESIDENT_MODES)[1:])
@pytest.mark.parametrize("offload,resident", [(False, 0), (True, 2)])
def test_resident_units_on_either_stream_in_any_number_of_shares(cuda, oracle, offload, resident, mode):
    """A resident unit's update in one launch or one share per micro-batch, on the coordinator's own
    stream or on the caller's: the same bits (the other tests run the default, the caller's stream
    and one share). Low-precision parameters cut at an odd element."""
    _run_backward_pipeline(cuda, oracle, offload, "copy_back", "split_odd", resident_units=resident, mode=mode)


def test_step_stream_is_ordered_with_the_gradient_buffers(cuda, oracle):
    """Units long enough (16 Mi elements) that an update on the coordinator's stream is still running
    when the caller's stream is given the next unit's work: the buffer it reads must not be cleared
    or refilled under it, and the record it is skipped by must be complete."""
    _run_backward_pipeline(cuda, oracle, False, "off", "gpu", mode="own_stream_one_share", unit_numel=1 << 24, num_units=3)


def _run_backward_pipeline(cuda, oracle, offload, windows, half_layout, resident_units=0, mode="caller_stream_one_share",
                           unit_numel=1 << 20, num_units=4):
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    from flextrain_amd.memory import pinned_empty
    torch.manual_seed(0)
    micro_batches = 4
    real = unit_numel - 4097  # the tail of each unit is alignment padding
    # each unit: a weight (decay) and a bias (no decay); the boundary falls inside a share
    w_numel, b_numel = real - 5000, 5000
    flat = [torch.zeros(unit_numel, dtype=torch.bfloat16, device=cuda) for _ in range(num_units)]
    weights, biases = [], []
    for u in range(num_units):
        flat[u][:real] = (torch.randn(real, device=cuda) * 0.02).to(torch.bfloat16)
        weights.append(torch.nn.Parameter(flat[u][:w_numel]))
        biases.append(torch.nn.Parameter(flat[u][w_numel:real]))
    decay = {"params": weights, "weight_decay": 0.1}
    plain = {"params": biases, "weight_decay": 0.0, "lr": 3e-4}
    opt = FlexTrainAdam([decay, plain], lr=1e-4,
                        unit_parameter_map={u: _Unit([weights[u], biases[u]]) for u in range(num_units)},
                        aligned_unit_numel=unit_numel, offload=offload)
    assert opt.non_layerwise_numel == 0
    assert [(s.start, s.end) for s in opt.unit_group_segments[0]] == [(0, w_numel), (w_numel, unit_numel)]
    # where the coordinator finds (and leaves) the low-precision parameters of each unit
    cut = {"gpu": unit_numel, "split": 600_064, "split_odd": 600_001, "host": 0}[half_layout]
    halves = []
    for u in range(num_units):
        pieces = []
        if cut:
            pieces.append(flat[u] if cut == unit_numel else flat[u][:cut].clone())
        if cut < unit_numel:
            host_piece = pinned_empty(unit_numel - cut, torch.bfloat16)
            host_piece.copy_(flat[u][cut:])
            pieces.append(host_piece)
        halves.append(pieces[0] if half_layout == "gpu" else pieces)
    torch.cuda.synchronize()

    def half_of(u):
        pieces = [halves[u]] if half_layout == "gpu" else halves[u]
        return torch.cat([piece.to(cuda) for piece in pieces])

    coord = FlexTrainOptsCoordinator()
    coord.initialize(opt, halves, micro_batches, offload=offload, device=cuda,
                     unit_windows={"auto": None, "off": False}.get(windows, True),
                     window_write_through=windows == "write_through", resident_units=resident_units,
                     **_resident_kwargs(mode, micro_batches))
    assert (coord._step_stream is not None) == RESIDENT_MODES[mode].get("step_stream", False)
    assert coord._unit_windows == (offload and windows != "off")  # small shares: the automatic choice is windows
    assert [coord.unit_master_parameter(u).is_pinned() for u in range(num_units)] == \
        [offload and u >= resident_units for u in range(num_units)]
    assert all(coord.unit_master_parameter(u).is_cuda for u in range(num_units) if not offload or u < resident_units)

    # oracle state, seeded the same way
    state = [(to_np(flat[u].float()).copy(), np.zeros(unit_numel, np.float32), np.zeros(unit_numel, np.float32))
             for u in range(num_units)]
    gen = torch.Generator(device=cuda).manual_seed(7)
    for iteration in (1, 2):
        opt.update_states()
        accumulated = {}
        for u in reversed(range(num_units)):
            buf = coord.pre_unit_backward(u)
            for mb in range(micro_batches):
                g = (torch.randn(unit_numel, device=cuda, generator=gen) * 1e-3).to(torch.bfloat16)
                g[real:] = 0  # padding never receives gradient
                buf += g
                coord.post_micro_batch_backward(u, mb)
            accumulated[u] = buf.clone()
        coord.clear_backward_pipeline()
        for u in range(num_units):
            pn, mn, vn = state[u]
            gn = to_np(accumulated[u])
            hn = np.zeros(unit_numel, np.uint16)
            for lo, hi, group in ((0, w_numel, decay), (w_numel, unit_numel, plain)):
                hs = np.zeros(hi - lo, np.uint16)
                ps, ms, vs = pn[lo:hi].copy(), mn[lo:hi].copy(), vn[lo:hi].copy()
                oracle.adam_step(ps, np.ascontiguousarray(gn[lo:hi]), ms, vs, step=iteration, lr=group.get("lr", 1e-4),
                                 weight_decay=group["weight_decay"], g_dtype=CODE[torch.bfloat16], half_out=hs,
                                 half_dtype=CODE[torch.bfloat16])
                pn[lo:hi], mn[lo:hi], vn[lo:hi], hn[lo:hi] = ps, ms, vs, hs
            m, v = coord.unit_optimizer_states(u)
            worst = dict(p=max_ulp(to_np(coord.unit_master_parameter(u)), pn), m=max_ulp(to_np(m), mn),
                         v=max_ulp(to_np(v), vn), h=max_ulp(half_bits(half_of(u)), hn, bf16=True))
            print(f"[coordinator offload={offload} windows={windows} half={half_layout} it={iteration} unit={u}] worst ULP distance: {worst}", flush=True)
            assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP
    assert decay["step"] == 2 and plain["step"] == 2
    if half_layout == "gpu":  # the module's parameters are views of the flat unit buffers: they saw the update
        assert weights[0].data_ptr() == flat[0].data_ptr() and halves[0] is flat[0]


def test_wider_accumulation_type(cuda, oracle):
    """bf16 parameters and gradients, fp32 accumulation: each micro-batch is written into the extra
    buffer and folded in by one fused pass; the step then consumes fp32 gradients."""
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    torch.manual_seed(1)
    num_units, micro_batches, unit_numel = 3, 2, 1 << 18
    flat = [(torch.randn(unit_numel, device=cuda) * 0.02).to(torch.bfloat16) for _ in range(num_units)]
    params = [torch.nn.Parameter(f) for f in flat]
    group = {"params": params, "weight_decay": 0.01}
    opt = FlexTrainAdam([group], lr=1e-4, unit_parameter_map={u: _Unit([params[u]]) for u in range(num_units)},
                        aligned_unit_numel=unit_numel, offload=False)
    coord = FlexTrainOptsCoordinator()
    coord.initialize(opt, flat, micro_batches, gradacc_dtype=torch.float32, offload=False)
    state = [(to_np(flat[u].float()).copy(), np.zeros(unit_numel, np.float32), np.zeros(unit_numel, np.float32))
             for u in range(num_units)]
    opt.update_states()
    acc = {u: np.zeros(unit_numel, np.float32) for u in range(num_units)}
    for u in reversed(range(num_units)):
        buf = coord.pre_unit_backward(u)
        assert buf.dtype == torch.bfloat16
        for mb in range(micro_batches):
            g = (torch.randn(unit_numel, device=cuda) * 1e-3).to(torch.bfloat16)
            buf.copy_(g)  # backward of one micro-batch writes its gradients
            oracle.grad_accumulate(acc[u], CODE[torch.float32], to_np(g).copy(), CODE[torch.bfloat16])
            coord.post_micro_batch_backward(u, mb)
            assert not buf.any()  # cleared for the next micro-batch
    coord.clear_backward_pipeline()
    for u in range(num_units):
        pn, mn, vn = state[u]
        hn = np.zeros(unit_numel, np.uint16)
        oracle.adam_step(pn, acc[u], mn, vn, step=1, lr=1e-4, weight_decay=0.01, half_out=hn, half_dtype=CODE[torch.bfloat16])
        m, v = coord.unit_optimizer_states(u)
        assert max_ulp(to_np(coord.unit_master_parameter(u)), pn) == 0 and max_ulp(to_np(m), mn) == 0
        assert max_ulp(to_np(v), vn) == 0 and max_ulp(half_bits(flat[u]), hn, bf16=True) == 0


@pytest.mark.parametrize("offload,resident_units", [(True, 0), (False, 0), (True, 2)])
def test_state_files_resume_bit_exact(cuda, tmp_path, offload, resident_units):
    """Save the units' [master | m | v] blocks as swap-format files after one iteration, wreck the
    live state, load, run a second iteration: same bits as a run that never stopped."""
    import os

    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    from flextrain_amd.state_files import opts_file_layout
    num_units, micro_batches, unit_numel = 3, 2, (1 << 16) + 1000

    def build():
        torch.manual_seed(2)
        flat = [(torch.randn(unit_numel, device=cuda) * 0.02).to(torch.bfloat16) for _ in range(num_units)]
        params = [torch.nn.Parameter(f) for f in flat]
        group = {"params": params, "weight_decay": 0.01}
        opt = FlexTrainAdam([group], lr=1e-3, unit_parameter_map={u: _Unit([params[u]]) for u in range(num_units)},
                            aligned_unit_numel=unit_numel, offload=offload)
        coord = FlexTrainOptsCoordinator()
        coord.initialize(opt, flat, micro_batches, offload=offload, resident_units=resident_units)
        return flat, group, opt, coord

    def iterate(opt, coord, seed):
        gen = torch.Generator(device=cuda).manual_seed(seed)
        opt.update_states()
        for u in reversed(range(num_units)):
            buf = coord.pre_unit_backward(u)
            for mb in range(micro_batches):
                buf += (torch.randn(unit_numel, device=cuda, generator=gen) * 1e-3).to(torch.bfloat16)
                coord.post_micro_batch_backward(u, mb)
        coord.clear_backward_pipeline()

    flat_a, _, opt_a, coord_a = build()
    iterate(opt_a, coord_a, 11)
    iterate(opt_a, coord_a, 12)

    flat_b, group_b, opt_b, coord_b = build()
    iterate(opt_b, coord_b, 11)
    paths = coord_b.save_optimizer_states(str(tmp_path))
    assert [os.path.basename(p) for p in paths] == [f"rank0_OPTS_layer{u}.swp.1" for u in range(num_units)]
    assert all(os.path.getsize(p) == opts_file_layout(unit_numel, 1)[2] for p in paths)
    assert os.path.getsize(paths[0]) % 4096 == 0 and os.path.getsize(paths[0]) > unit_numel * 12
    for u in range(num_units):  # wreck everything the files are supposed to bring back
        coord_b.unit_master_parameter(u).fill_(float("nan"))
        for s in coord_b.unit_optimizer_states(u):
            s.fill_(7.0)
        flat_b[u].zero_()
    coord_b.load_optimizer_states(str(tmp_path))
    assert group_b["step"] == 1  # step counters are the caller's; untouched here
    iterate(opt_b, coord_b, 12)
    for u in range(num_units):
        assert torch.equal(flat_a[u], flat_b[u])
        assert torch.equal(coord_a.unit_master_parameter(u).cpu(), coord_b.unit_master_parameter(u).cpu())
        for sa, sb in zip(coord_a.unit_optimizer_states(u), coord_b.unit_optimizer_states(u)):
            assert torch.equal(sa.cpu(), sb.cpu())


# ---- mixed precision in the per-unit pipeline ---------------------------------------------------
def _fp16_units(cuda, num_units, unit_numel, offload, **coordinator_kwargs):
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    flat = [(torch.randn(unit_numel, device=cuda) * 0.02).to(torch.float16) for _ in range(num_units)]
    params = [torch.nn.Parameter(f) for f in flat]
    group = {"params": params, "weight_decay": 0.01}
    opt = FlexTrainAdam([group], lr=1e-3, unit_parameter_map={u: _Unit([params[u]]) for u in range(num_units)},
                        aligned_unit_numel=unit_numel, offload=offload)
    coord = FlexTrainOptsCoordinator()
    coord.initialize(opt, flat, offload=offload, device=cuda, **coordinator_kwargs)
    state = [(to_np(flat[u].float()).copy(), np.zeros(unit_numel, np.float32), np.zeros(unit_numel, np.float32))
             for u in range(num_units)]
    return flat, group, opt, coord, state


def _check_units(tag, coord, flat, state, expected_half):
    for u, (pn, mn, vn) in enumerate(state):
        m, v = coord.unit_optimizer_states(u)
        worst = dict(p=max_ulp(to_np(coord.unit_master_parameter(u)), pn), m=max_ulp(to_np(m), mn), v=max_ulp(to_np(v), vn),
                     h=max_ulp(half_bits(flat[u]).view(np.float16), expected_half[u].view(np.float16)))
        print(f"[{tag} unit={u}] worst ULP distance: {worst}", flush=True)
        assert max(worst["p"], worst["m"], worst["v"]) <= MASTER_ULP and worst["h"] <= HALF_ULP, (tag, u, worst)


@pytest.mark.parametrize("offload,windows,gradacc,mode", _with_resident_modes([
    (False, False, None), (True, True, None), (True, False, None), (False, False, torch.float32), (True, True, torch.float32)]))
def test_scaled_gradients_and_overflow_while_stepping_during_backward(cuda, oracle, offload, windows, gradacc, mode):
    """fp16 units, loss scale 65536, three iterations, an inf planted in unit 1 on iteration 2.
    Every share's update unscales on load; the policy for an overflow found after earlier units have
    been stepped: unit 1 and every unit stepped after it (unit 0) are skipped on the device, units 3
    and 2 keep their update, the iteration is flagged and the scale halves. State of every unit
    against the oracle under that policy; scale trace against the reference's state machine."""
    from flextrain_amd.loss_scaler import DynamicLossScaler
    torch.manual_seed(5)
    num_units, micro_batches, unit_numel = 4, 2, 1 << 18
    scaler = DynamicLossScaler(init_scale=65536.0, delayed_shift=1, scale_window=1000)
    flat, group, opt, coord, state = _fp16_units(
        cuda, num_units, unit_numel, offload, micro_batch_per_rank=micro_batches, unit_windows=windows,
        gradacc_dtype=gradacc, loss_scaler=scaler, **_resident_kwargs(mode, micro_batches))
    expected_half = [half_bits(f).copy() for f in flat]
    gen = torch.Generator(device=cuda).manual_seed(9)
    seen_scales, overflows = [], []
    for iteration in (1, 2, 3):
        scale = coord.loss_scale
        seen_scales.append(scale)
        opt.update_states()
        accumulated = {}
        for u in reversed(range(num_units)):
            buf = coord.pre_unit_backward(u)
            acc = np.zeros(unit_numel, np.float32) if gradacc is not None else None
            for mb in range(micro_batches):
                g = (torch.randn(unit_numel, device=cuda, generator=gen) * 1e-3 * scale).to(torch.float16)
                if iteration == 2 and u == 1 and mb == 0:
                    g[12345] = float("inf")
                if gradacc is None:
                    buf += g
                else:
                    buf.copy_(g)
                    oracle.grad_accumulate(acc, CODE[torch.float32], half_bits(g).copy(), CODE[torch.float16])
                if mb == micro_batches - 1:
                    accumulated[u] = buf.clone() if gradacc is None else acc
                coord.post_micro_batch_backward(u, mb)
        decision = coord.clear_backward_pipeline()
        overflows.append(decision.overflow)
        assert decision.overflow == (iteration == 2) and decision.nonfinite == (1 if iteration == 2 else 0)
        assert coord.last_skipped_units == ([0, 1] if iteration == 2 else [])
        for u in range(num_units):
            if iteration == 2 and u <= 1:
                continue  # skipped: the oracle's state stays as it is
            pn, mn, vn = state[u]
            gn = accumulated[u] if gradacc is not None else half_bits(accumulated[u])
            hn = np.zeros(unit_numel, np.uint16)
            oracle.adam_step(pn, gn, mn, vn, step=iteration, lr=1e-3, weight_decay=0.01,
                             grad_mult=float(np.float32(1.0 / scale)),
                             g_dtype=CODE[torch.float32] if gradacc is not None else CODE[torch.float16],
                             half_out=hn, half_dtype=CODE[torch.float16])
            expected_half[u] = hn
        _check_units(f"scaled offload={offload} windows={windows} gradacc={gradacc} it={iteration}", coord, flat, state, expected_half)
    assert seen_scales + [coord.loss_scale] == oracle.loss_scale_trace(overflows, 65536.0, delayed_shift=1)
    assert overflows == [False, True, False]


@pytest.mark.parametrize("offload,windows,gradacc,mode", _with_resident_modes([
    (False, False, None), (True, True, None), (True, False, torch.float32), (False, False, torch.float32)]))
def test_deferred_schedule_gives_a_global_decision(cuda, oracle, offload, windows, gradacc, mode):
    """defer_to_forward: backward only accumulates and gathers statistics; one decision per
    iteration after the first unit's backward; the updates run during the next forward pass.
    Iteration 2 carries a nan in the LAST unit to run backward (unit 0): every unit, also those whose
    gradients were complete long before, stays bit-unchanged. Iterations 1 and 3 are clipped with
    the norm over all units (against float64: 1e-6), and the state equals the oracle's."""
    from flextrain_amd.loss_scaler import DynamicLossScaler
    torch.manual_seed(6)
    num_units, micro_batches, unit_numel, max_norm = 3, 2, 1 << 18, 1.0
    scaler = DynamicLossScaler(init_scale=4096.0, delayed_shift=1, scale_window=1000)
    flat, group, opt, coord, state = _fp16_units(
        cuda, num_units, unit_numel, offload, micro_batch_per_rank=micro_batches, unit_windows=windows,
        gradacc_dtype=gradacc, loss_scaler=scaler, max_grad_norm=max_norm, defer_to_forward=True,
        **_resident_kwargs(mode, micro_batches))
    expected_half = [half_bits(f).copy() for f in flat]
    gen = torch.Generator(device=cuda).manual_seed(10)

    def forward_pass():
        coord.warmup_forward_pipeline()
        for u in range(num_units):
            coord.pre_unit_forward(u)
            for mb in range(micro_batches):
                coord.post_micro_batch_forward(u, mb)

    applied, seen_scales, overflows = 0, [], []
    for iteration in (1, 2, 3):
        forward_pass()  # applies the previous iteration's decision (nothing to apply in iteration 1)
        coord.synchronize()
        _check_units(f"deferred offload={offload} windows={windows} gradacc={gradacc} before it={iteration}", coord, flat, state, expected_half)
        scale = coord.loss_scale
        seen_scales.append(scale)
        accumulated, sumsq = {}, 0.0
        for u in reversed(range(num_units)):
            buf = coord.pre_unit_backward(u)
            acc = np.zeros(unit_numel, np.float32) if gradacc is not None else None
            for mb in range(micro_batches):
                g = (torch.randn(unit_numel, device=cuda, generator=gen) * 3e-3 * scale).to(torch.float16)
                if iteration == 2 and u == 0 and mb == 1:
                    g[777] = float("nan")
                if gradacc is None:
                    buf += g
                else:
                    buf.copy_(g)
                    oracle.grad_accumulate(acc, CODE[torch.float32], half_bits(g).copy(), CODE[torch.float16])
                if mb == micro_batches - 1:
                    accumulated[u] = buf.clone() if gradacc is None else acc
                coord.post_micro_batch_backward(u, mb)
            unscaled = (accumulated[u].double() if gradacc is None else torch.from_numpy(acc).double()) / scale
            sumsq += float((unscaled[torch.isfinite(unscaled)] ** 2).sum())
        decision = coord.clear_backward_pipeline()
        overflows.append(decision.overflow)
        assert decision.overflow == (iteration == 2)
        if decision.overflow:
            assert coord.last_skipped_units == list(range(num_units))
            continue
        norm = sumsq ** 0.5
        assert norm > max_norm and abs(decision.grad_norm - norm) <= 1e-6 * norm
        assert abs(decision.clip_coef - max_norm / (norm + 1e-6)) <= 1e-6 * decision.clip_coef
        assert np.float32(decision.grad_mult) == oracle.combined_multiplier(scale, decision.clip_coef)
        applied += 1
        opt.update_states()  # the caller advances the step counters of an iteration that will be applied
        for u in range(num_units):
            pn, mn, vn = state[u]
            gn = accumulated[u] if gradacc is not None else half_bits(accumulated[u])
            hn = np.zeros(unit_numel, np.uint16)
            oracle.adam_step(pn, gn, mn, vn, step=applied, lr=1e-3, weight_decay=0.01, grad_mult=decision.grad_mult,
                             g_dtype=CODE[torch.float32] if gradacc is not None else CODE[torch.float16],
                             half_out=hn, half_dtype=CODE[torch.float16])
            expected_half[u] = hn
    with pytest.raises(RuntimeError, match="have not been applied"):
        coord.pre_unit_backward(num_units - 1)
    forward_pass()
    coord.synchronize()
    _check_units(f"deferred offload={offload} windows={windows} gradacc={gradacc} final", coord, flat, state, expected_half)
    assert seen_scales + [coord.loss_scale] == oracle.loss_scale_trace(overflows, 4096.0, delayed_shift=1)
    assert group["step"] == 2


def test_clipping_needs_the_deferred_schedule(cuda):
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    flat = [torch.zeros(1024, dtype=torch.bfloat16, device=cuda)]
    params = [torch.nn.Parameter(flat[0])]
    opt = FlexTrainAdam([{"params": params}], unit_parameter_map={0: _Unit(params)}, aligned_unit_numel=1024, offload=False)
    with pytest.raises(ValueError, match="defer_to_forward"):
        FlexTrainOptsCoordinator().initialize(opt, flat, 2, offload=False, max_grad_norm=1.0)
