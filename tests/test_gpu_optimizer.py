"""GPU tests of the optimizer front end (FlexTrainAdam / FlexTrainOptimizer): grouping, the
non-layerwise step, mixed-precision skipping and clipping, resident and offloaded state."""
import numpy as np
import pytest
import torch

from _util import to_np

pytestmark = pytest.mark.gpu


def _model(cuda, dtype):
    torch.manual_seed(0)
    emb = torch.nn.Parameter((torch.randn(1000, 64, device=cuda) * 0.02).to(dtype))
    head = torch.nn.Parameter((torch.randn(64, 1000, device=cuda) * 0.02).to(dtype))
    norm = torch.nn.Parameter(torch.ones(64, device=cuda, dtype=dtype))
    return emb, head, norm


@pytest.mark.parametrize("offload", [False, True])
def test_groups_step_and_match_torch_adamw(cuda, offload):
    """Two parameter groups with different weight decay, bf16 parameters, fp32 master copy: ten
    steps track torch.optim.AdamW run on fp32 copies of the same parameters."""
    from flextrain_amd import FlexTrainAdam
    emb, head, norm = _model(cuda, torch.bfloat16)
    ref_params = [torch.nn.Parameter(p.detach().float().clone()) for p in (emb, head, norm)]
    ref = torch.optim.AdamW([{"params": ref_params[:2], "weight_decay": 0.1}, {"params": ref_params[2:], "weight_decay": 0.0}],
                            lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
    groups = [{"params": [emb, head], "weight_decay": 0.1}, {"params": [norm], "weight_decay": 0.0}]
    opt = FlexTrainAdam(groups, lr=1e-3, offload=offload)
    assert opt.optimizer_state_per_element == 2
    assert opt.non_layerwise_numel == 1000 * 64 * 2 + 64
    assert len(opt.non_layerwise_step_contexts) == 2
    assert emb.data_ptr() == opt._device_para.data_ptr()  # parameters now live in the flat buffer
    gen = torch.Generator(device=cuda).manual_seed(1)
    for _ in range(10):
        opt.update_states()
        for p, r in zip((emb, head, norm), ref_params):
            g = torch.randn(p.shape, device=cuda, generator=gen) * 1e-2
            p.grad.copy_(g.to(p.dtype))
            r.grad = p.grad.float().clone()
        assert opt.step() is True
        ref.step()
        assert not opt._device_grad.any()  # gradients are zeroed after the step
    assert groups[0]["step"] == 10
    master = opt._master_para.to(cuda)
    want = torch.cat([r.detach().reshape(-1) for r in ref_params])
    assert torch.allclose(master, want, rtol=2e-5, atol=2e-7)
    # the bf16 parameters are the rounding of the master copy
    assert torch.equal(opt._device_para, master.to(torch.bfloat16))
    assert torch.equal(emb.reshape(-1), master[:64000].to(torch.bfloat16))


def test_fp16_training_skips_on_overflow_and_clips(cuda):
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.loss_scaler import DynamicLossScaler
    emb, head, norm = _model(cuda, torch.float16)
    scaler = DynamicLossScaler(init_scale=1024.0, delayed_shift=1)
    opt = FlexTrainAdam([{"params": [emb, head, norm]}], lr=1e-3, weight_decay=0.0, loss_scaler=scaler, max_grad_norm=1.0)
    before = opt._master_para.clone()
    opt.update_states()
    for p in (emb, head, norm):
        p.grad.copy_((torch.randn(p.shape, device=cuda) * 0.5 * 1024.0).to(torch.float16))
    emb.grad[3, 5] = float("inf")
    assert opt.step() is False and opt.last_step_skipped
    assert scaler.loss_scale == 512.0
    assert torch.equal(opt._master_para, before) and not opt._device_grad.any()

    for p in (emb, head, norm):
        p.grad.copy_((torch.randn(p.shape, device=cuda) * 0.5 * 512.0).to(torch.float16))
    g_unscaled = opt._device_grad.float() / 512.0
    norm64 = float(g_unscaled.double().norm())
    assert opt.step() is True
    assert abs(opt.last_grad_norm - norm64) <= 1e-6 * norm64
    # first Adam step with clipped gradients: |delta p| = lr * |g| / (|g| + eps) ~ lr wherever g != 0
    delta = (opt._master_para - before).abs()
    moved = g_unscaled.abs() * (1.0 / norm64) > 1e-6
    assert torch.allclose(delta[moved], torch.full_like(delta[moved], 1e-3), rtol=2e-2)
    assert scaler.loss_scale == 512.0


def test_unit_segments_and_gradacc_dtype(cuda):
    """Layer units are recorded as group segments (stretched to the aligned unit size) and left to
    the caller; a wider accumulation dtype is fed by hooks."""
    from flextrain_amd import FlexTrainAdam

    class Unit:
        def __init__(self, paras):
            self.paras = paras
    w1 = torch.nn.Parameter(torch.randn(10, 10, device=cuda).half())
    b1 = torch.nn.Parameter(torch.randn(10, device=cuda).half())
    extra = torch.nn.Parameter(torch.randn(7, device=cuda).half())
    g_decay, g_plain = {"params": [w1, extra]}, {"params": [b1], "weight_decay": 0.0}
    opt = FlexTrainAdam([g_decay, g_plain], unit_parameter_map={0: Unit([w1, b1])}, aligned_unit_numel=2048,
                        gradacc_dtype=torch.float32)
    segs = opt.unit_group_segments[0]
    assert [(s.start, s.end) for s in segs] == [(0, 100), (100, 2048)]
    assert segs[0].param_group is g_decay and segs[1].param_group is g_plain
    assert opt.non_layerwise_numel == 7
    (extra.float() * 2).sum().backward()
    assert torch.equal(opt._device_acc_grad, torch.full((7,), 2.0, device=cuda))
    opt.update_states()
    opt.step()
    assert not opt._device_acc_grad.any()


@pytest.mark.parametrize("offload", [False, True])
def test_training_loop_with_autograd(cuda, offload):
    """A small fp16 network trained end to end the way a user would: autograd fills the gradients
    of parameters that live in the optimizer's flat buffer, the loss is scaled by a dynamic scaler,
    the optimizer unscales, checks, clips and steps. The loss must fall like that of an fp32
    torch.optim.AdamW twin fed the same batches, and an injected overflow must cost exactly one
    skipped step and a halved scale."""
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.loss_scaler import DynamicLossScaler
    torch.manual_seed(3)
    d_in, d_hid = 32, 64
    w1 = torch.nn.Parameter((torch.randn(d_in, d_hid, device=cuda) * 0.2).half())
    b1 = torch.nn.Parameter(torch.zeros(d_hid, device=cuda).half())
    w2 = torch.nn.Parameter((torch.randn(d_hid, 1, device=cuda) * 0.2).half())
    twin = [torch.nn.Parameter(p.detach().float().clone()) for p in (w1, b1, w2)]
    ref = torch.optim.AdamW([{"params": [twin[0], twin[2]], "weight_decay": 0.01}, {"params": [twin[1]], "weight_decay": 0.0}],
                            lr=3e-3)
    scaler = DynamicLossScaler(init_scale=2.0 ** 12, delayed_shift=1, scale_window=10_000)
    opt = FlexTrainAdam([{"params": [w1, w2], "weight_decay": 0.01}, {"params": [b1], "weight_decay": 0.0}], lr=3e-3,
                        loss_scaler=scaler, max_grad_norm=10.0, offload=offload)

    def forward(params, x):
        a, b, c = params
        return (torch.tanh(x @ a + b) @ c).squeeze(-1)

    target_w = torch.randn(d_in, device=cuda)
    losses, ref_losses, skipped = [], [], 0
    for it in range(60):
        x = torch.randn(256, d_in, device=cuda)
        y = torch.sin(x @ target_w)
        loss = ((forward((w1, b1, w2), x.half()).float() - y) ** 2).mean()
        opt.update_states()
        scaler.backward(loss)
        if it == 20:
            w1.grad[0, 0] = float("inf")  # what an fp16 overflow in backward looks like
        stepped = opt.step()
        if not stepped:
            skipped += 1
            for g in opt.param_groups:  # a skipped step does not count (the caller's policy)
                g["step"] -= 1
        losses.append(float(loss.detach()))
        ref_loss = ((forward(twin, x) - y) ** 2).mean()
        ref.zero_grad()
        ref_loss.backward()
        if it != 20:
            ref.step()
        ref_losses.append(float(ref_loss.detach()))
    assert skipped == 1 and scaler.loss_scale == 2.0 ** 11
    assert opt.param_groups[0]["step"] == 59
    first, last = sum(losses[:5]) / 5, sum(losses[-5:]) / 5
    ref_last = sum(ref_losses[-5:]) / 5
    print(f"[training loop offload={offload}] loss {first:.4f} -> {last:.4f} (fp32 twin {ref_last:.4f})", flush=True)
    assert last < 0.6 * first
    assert abs(last - ref_last) <= 0.1 * ref_last + 5e-3
    # parameters are the fp16 rounding of the master copy, and close to the fp32 twin's
    master = opt._master_para.to(cuda)
    assert torch.equal(opt._device_para, master.half())
    flat_twin = torch.cat([twin[0].detach().reshape(-1), twin[2].detach().reshape(-1), twin[1].detach().reshape(-1)])
    assert (master - flat_twin).abs().max() < 0.05


def test_device_arrays_share_one_allocation(cuda):
    """The arrays of an update come zero-filled out of one allocation, each of the right type and
    length, 2 MiB-aligned plus a 2 KiB stagger, without overlap; a step on them equals a step on
    separately allocated tensors bit for bit (placement changes speed, never results)."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.memory import allocate_device_arrays
    n = (3 << 20) + 5
    specs = [(n, torch.float32)] * 3 + [(n, torch.bfloat16)] * 2
    arrays = allocate_device_arrays(specs, cuda)
    assert [(a.numel(), a.dtype) for a in arrays] == specs
    assert [a.data_ptr() % (2 << 20) for a in arrays] == [0, 2048, 4096, 6144, 8192]
    spans = sorted((a.data_ptr(), a.data_ptr() + a.numel() * a.element_size()) for a in arrays)
    assert all(spans[k][1] <= spans[k + 1][0] for k in range(len(spans) - 1))
    assert all(not a.any() for a in arrays)
    p, m, v, g, h = arrays
    gen = torch.Generator(device=cuda).manual_seed(5)
    p.normal_(0, 0.02, generator=gen); g.normal_(0, 1e-3, generator=gen)
    p2, m2, v2, g2, h2 = p.clone(), m.clone(), v.clone(), g.clone(), h.clone()
    eng = FlexTrainCPUAdam(lr=1e-3, weight_decay=0.01)
    for t in (1, 2):
        eng._step({"step": t}, h, p, g, m, v)
        eng._step({"step": t}, h2, p2, g2, m2, v2)
    for a, b in ((p, p2), (m, m2), (v, v2), (h, h2)):
        assert torch.equal(a, b)
    with pytest.raises(ValueError):
        allocate_device_arrays(specs, "cpu")


@pytest.mark.parametrize("state_device", ["cuda", "cpu"])
def test_profile_step_runs_on_private_buffers(cuda, state_device):
    """The reference's own micro-benchmark entry (``flextrain/optimizer.py:71-95``): buffers are
    made once, every call is one more step, and the parameters move."""
    from flextrain_amd import FlexTrainCPUAdam
    eng = FlexTrainCPUAdam(lr=1e-2)
    eng.state_device = state_device
    eng.profile_step(1 << 18, torch.bfloat16, torch.float32)
    first = eng._full_parameter.clone()
    buffers = (eng._half_parameter.data_ptr(), eng._full_parameter.data_ptr(), eng._gradient.data_ptr())
    eng.profile_step(1 << 18, torch.bfloat16, torch.float32)
    eng.synchronize()
    assert eng._param_group["step"] == 2
    assert buffers == (eng._half_parameter.data_ptr(), eng._full_parameter.data_ptr(), eng._gradient.data_ptr())
    assert not torch.equal(first, eng._full_parameter)
    assert torch.equal(eng._half_parameter.float().cpu(), eng._full_parameter.bfloat16().float().cpu())
    assert eng._full_parameter.is_cuda == (state_device == "cuda")
