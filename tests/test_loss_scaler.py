"""The scale state machine of the product against hand-derived traces and the oracle's replay."""
import numpy as np
import pytest
import torch

from flextrain_amd.loss_scaler import DynamicLossScaler, LossScaler, create_loss_scaler, to_python_float


def run(scaler, overflows):
    seen = []
    for ov in overflows:
        seen.append(scaler.loss_scale)
        scaler.update_scale(ov)
    return seen + [scaler.loss_scale]


def test_eight_step_traces():
    ov = [i in (3, 6) for i in range(1, 9)]
    s = DynamicLossScaler(init_scale=65536.0, delayed_shift=1)
    assert run(s, ov) == [65536.0] * 3 + [32768.0] * 3 + [16384.0] * 3
    assert s.cur_hysteresis == 1 and s.cur_iter == 8 and s.last_overflow_iter == 5
    s = DynamicLossScaler(init_scale=65536.0, delayed_shift=2)
    assert run(s, ov) == [65536.0] * 6 + [32768.0] * 3
    assert s.cur_hysteresis == 1


def test_window_growth_floor_and_error():
    s = DynamicLossScaler(init_scale=4.0, scale_window=4)
    assert run(s, [False] * 8) == [4.0] * 4 + [8.0] * 4 + [16.0]
    s = DynamicLossScaler(init_scale=4.0, min_scale=1.0)
    assert run(s, [True] * 4) == [4.0, 2.0, 1.0, 1.0, 1.0]
    s = DynamicLossScaler(init_scale=1.0, min_scale=1.0, raise_error_at_min_scale=True)
    with pytest.raises(Exception):
        s.update_scale(True)
    # hysteresis refills only at a window boundary unless consecutive_hysteresis is set
    s = DynamicLossScaler(init_scale=16.0, delayed_shift=3, scale_window=1000)
    run(s, [True, False, True])
    assert s.cur_hysteresis == 1 and s.loss_scale == 16.0
    s.update_scale(True)
    assert s.loss_scale == 8.0
    s = DynamicLossScaler(init_scale=16.0, delayed_shift=3, consecutive_hysteresis=True)
    run(s, [True, False, True])
    assert s.cur_hysteresis == 2  # refilled by the clean iteration, then one burnt


def test_random_sequences_match_the_oracle_replay(oracle):
    rng = np.random.default_rng(0)
    for _ in range(200):
        ov = (rng.random(60) < 0.2).tolist()
        kw = dict(scale_window=int(rng.integers(1, 9)), delayed_shift=int(rng.integers(1, 4)),
                  consecutive_hysteresis=bool(rng.integers(0, 2)), min_scale=1.0)
        s = DynamicLossScaler(init_scale=2.0 ** 10, **kw)
        assert run(s, ov) == oracle.loss_scale_trace(ov, 2.0 ** 10, **kw)


def test_static_scaler_and_factory():
    s = LossScaler(128.0)
    s.update_scale(True)
    assert s.loss_scale == 128.0 and not s.dynamic and s.has_overflow(None) is False
    assert LossScaler._has_inf_or_nan(torch.tensor(float("inf"))) is False and s._has_inf_or_nan(None) is False
    assert to_python_float(torch.tensor([2.5])) == 2.5
    assert s.scale_gradient(None, (torch.ones(2),), None)[0].tolist() == [128.0, 128.0]
    d = create_loss_scaler(torch.float16)
    assert isinstance(d, DynamicLossScaler) and d.loss_scale == 65536 and d.delayed_shift == 2 and d.scale_window == 1000
    st = create_loss_scaler(torch.float16, dynamic_loss_scaling=False, initial_scale_power=8)
    assert isinstance(st, LossScaler) and st.loss_scale == 256
    for dt in (torch.bfloat16, torch.float32):
        b = create_loss_scaler(dt)
        assert isinstance(b, LossScaler) and b.loss_scale == 1.0
    loss = torch.tensor(2.0, requires_grad=True)
    LossScaler(8.0).backward(loss * 1.0)
    assert loss.grad.item() == 8.0
