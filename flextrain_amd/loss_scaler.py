"""Loss scaling: the reference's scale state machine plus the gradient check it never had.

``LossScalerBase`` / ``LossScaler`` / ``DynamicLossScaler`` / ``create_loss_scaler`` mirror
``flextrain/loss_scaler.py`` (same names, attributes and ``update_scale`` transitions, ``:134-179``).

The reference multiplies the loss by the scale (``flextrain/engine.py:249``) but nothing ever
divides the gradients, looks for inf/nan or calls ``update_scale``. ``GradientGuard`` supplies
that missing half on the GPU: one read of the gradients gives the inf/nan count and the sum of
squares of the *unscaled* gradient, from which the step decision follows:

    overflow  = any gradient element is inf or nan          -> skip the step, update_scale(True)
    norm      = sqrt(sum of squares)                         (of g / loss_scale)
    clip_coef = min(1, max_norm / (norm + 1e-6))             (torch.nn.utils.clip_grad_norm_ rule)
    grad_mult = clip_coef * (1 / loss_scale)                 (applied inside the update kernel)
"""
from __future__ import annotations

from abc import ABC
from dataclasses import dataclass
from typing import Optional

import torch

from . import _C

INITIAL_LOSS_SCALE = 'init_scale'
SCALE_WINDOW = 'scale_window'
DELAYED_SHIFT = 'delayed_shift'
CONSECUTIVE_HYSTERESIS = 'consecutive_hysteresis'
MIN_LOSS_SCALE = 'min_scale'


def to_python_float(tensor: torch.Tensor) -> float:
    """One-element tensor to a Python number (reference ``loss_scaler.py:23-27``)."""
    if hasattr(tensor, "item"):
        return tensor.item()
    assert tensor.nelement() == 1
    return tensor[0]


class LossScalerBase(ABC):
    """Holds the current scale (reference ``loss_scaler.py:30-49``)."""

    def __init__(self, cur_scale: float):
        self.cur_scale = cur_scale
        self.dynamic = False

    @property
    def loss_scale(self):
        return self.cur_scale

    def scale_gradient(self, module, grad_in, grad_out):
        return tuple(self.loss_scale * g for g in grad_in)

    def update_scale(self, overflow):
        pass

    def backward(self, loss: torch.Tensor, retain_graph=False):
        (loss * self.loss_scale).backward(retain_graph=retain_graph)


class LossScaler(LossScalerBase):
    """Static scale (reference ``:52-66``)."""

    def __init__(self, scale=1):
        super().__init__(scale)

    def has_overflow(self, params):
        return False

    @staticmethod
    def _has_inf_or_nan(x):
        """A static scale never reports an overflow (reference ``:65-66``, there a method without
        ``self``; callable both ways here)."""
        return False


class DynamicLossScaler(LossScalerBase):
    """Dynamic scale with hysteresis (reference ``:69-179``).

    On overflow the scale is divided by ``scale_factor`` (not below ``min_scale``) once the
    hysteresis budget ``delayed_shift`` is used up; after ``scale_window`` iterations since the
    last overflow it is multiplied by ``scale_factor``.
    """

    def __init__(
        self,
        init_scale,
        scale_factor=2.0,
        scale_window=1000,
        min_scale=1.0,
        delayed_shift=1,
        consecutive_hysteresis=False,
        raise_error_at_min_scale=False,
        dtype=torch.half,
    ):
        super().__init__(init_scale)
        self.cur_iter = 0
        self.last_overflow_iter = -1
        self.scale_factor = scale_factor
        self.scale_window = scale_window
        self.min_scale = min_scale
        self.delayed_shift = delayed_shift
        self.cur_hysteresis = delayed_shift
        self.consecutive_hysteresis = consecutive_hysteresis
        self.raise_error_at_min_scale = raise_error_at_min_scale
        self.dynamic = True
        self.dtype = dtype

    def update_scale(self, overflow):
        if overflow:
            out_of_budget = self.delayed_shift == 1 or self.cur_hysteresis == 1
            if out_of_budget:
                if self.cur_scale == self.min_scale and self.raise_error_at_min_scale:
                    raise Exception(
                        "Current loss scale already at minimum - cannot decrease scale anymore. Exiting run.")
                self.cur_scale = max(self.cur_scale / self.scale_factor, self.min_scale)
            else:
                self.cur_hysteresis -= 1
            self.last_overflow_iter = self.cur_iter
        else:
            if self.consecutive_hysteresis:
                self.cur_hysteresis = self.delayed_shift
            if (self.cur_iter - self.last_overflow_iter) % self.scale_window == 0:
                if not self.consecutive_hysteresis:
                    self.cur_hysteresis = self.delayed_shift
                self.cur_scale *= self.scale_factor
        self.cur_iter += 1


def create_loss_scaler(
    device_dtype: torch.dtype = torch.float16,
    dynamic_loss_scaling: bool = True,
    initial_scale_power: int = 16,
    loss_scale_window: int = 1000,
    hysteresis: int = 2,
    consecutive_hysteresis: bool = False,
    min_loss_scale: float = 1.0,
):
    """Scaler for a mixed-precision setup (reference ``loss_scaler.py:184-204``; the defaults are
    those of ``flextrain/defaults.py:143-193``).

    fp16 + dynamic -> ``DynamicLossScaler``; fp16 + static -> ``LossScaler(2**initial_scale_power)``;
    any other dtype -> ``LossScaler(1.0)``. The reference means the same but, because of two
    trailing commas (``:188-189``), always returns the dynamic scaler for fp16 and would pass a
    tuple as the static scale; that accident is not reproduced.
    """
    if device_dtype == torch.half:
        init_scale = 2 ** initial_scale_power
        if dynamic_loss_scaling:
            return DynamicLossScaler(
                dtype=device_dtype,
                **{
                    INITIAL_LOSS_SCALE: init_scale,
                    SCALE_WINDOW: loss_scale_window,
                    MIN_LOSS_SCALE: min_loss_scale,
                    DELAYED_SHIFT: hysteresis,
                    CONSECUTIVE_HYSTERESIS: consecutive_hysteresis,
                })
        return LossScaler(scale=init_scale)
    return LossScaler(scale=1.0)


@dataclass
class GuardDecision:
    overflow: bool      #: an inf/nan was found: skip the step
    nonfinite: int      #: how many
    sumsq: float        #: sum of squares of the finite unscaled gradient elements (double)
    grad_norm: float    #: sqrt(sumsq) as fp32
    clip_coef: float    #: fp32
    grad_mult: float    #: fp32 factor for the update kernel


class GradientGuard:
    """Overflow check + global-norm clip decision for one optimizer step, on the GPU.

    ``begin()``, then ``add(grads)`` once per gradient buffer that belongs to the step, then
    ``decide()`` (reads 32 bytes back) or ``decide_async()`` (stays on the device and returns the
    control buffer to hand to ``_step(control=...)``).
    """

    def __init__(self, device=None, capturable: bool = False):
        """``capturable``: 1/loss_scale is read by the kernels from device memory instead of travelling
        by value, so that a step recorded into a HIP graph follows a loss scale that changes between
        replays: ``set_scale()`` writes a pinned staging copy (outside any capture), and
        ``add_and_decide`` first enqueues the 4-byte copy to the device (recorded, it re-reads the
        staging copy at every replay)."""
        self.device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        self._lib = _C.lib()
        self.capturable = bool(capturable)
        if self.capturable:
            self._scale_host = torch.ones(1, dtype=torch.float32, pin_memory=True)
            self._scale_dev = torch.ones(1, dtype=torch.float32, device=self.device)
        # 32 bytes: ft_grad_stats_t followed by ft_step_control_t, read back with one copy
        self._buf = torch.zeros(4, dtype=torch.float64, device=self.device)
        self._ws_bytes = int(self._lib.ft_grad_stats_workspace_bytes())
        self._ws = torch.empty(self._ws_bytes, dtype=torch.uint8, device=self.device)
        self._fresh = True

    @property
    def stats_ptr(self) -> int:
        return self._buf.data_ptr()

    @property
    def control(self) -> torch.Tensor:
        """Device view of the ft_step_control_t (4 x 32 bit)."""
        return self._buf[2:4].view(torch.float32)

    def begin(self) -> None:
        self._fresh = True

    def add(self, grads: torch.Tensor, loss_scale: float = 1.0) -> None:
        if not grads.is_cuda or not grads.is_contiguous():
            raise ValueError("gradients must be a contiguous GPU tensor")
        pre_mult = float(1.0 / float(loss_scale))
        with torch.cuda.device(grads.device):
            _C.check("ft_grad_stats", self._lib.ft_grad_stats(
                grads.data_ptr(), _C.dtype_code(grads.dtype), grads.numel(), pre_mult, self.stats_ptr,
                0 if self._fresh else 1, self._ws.data_ptr(), self._ws_bytes, _C.current_stream_ptr(grads.device)))
        self._fresh = False

    def set_scale(self, loss_scale: float) -> None:
        """Capturable guards: the loss scale the next (recorded or eager) ``add_and_decide`` works with."""
        torch.cuda.synchronize(self.device)  # a step in flight still reads the present value
        self._scale_host[0] = float(1.0 / float(loss_scale))

    def add_and_decide(self, grads: torch.Tensor, loss_scale: float = 1.0, max_grad_norm: Optional[float] = None,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``add(grads)`` followed by ``decide_async(...)`` with one launch fewer: the kernel that
        finishes the statistics writes the decision as well. For the last (or only) gradient buffer
        of a step. Returns the control record like ``decide_async``."""
        if not grads.is_cuda or not grads.is_contiguous():
            raise ValueError("gradients must be a contiguous GPU tensor")
        target = self.control if out is None else out
        if out is not None and (not out.is_cuda or out.numel() * out.element_size() < 16 or out.data_ptr() % 16):
            raise ValueError("out must be 16 bytes of 16-byte aligned device memory")
        inv_scale = float(1.0 / float(loss_scale))
        with torch.cuda.device(grads.device):
            if self.capturable:  # the scale comes from device memory; `loss_scale` is not used (see set_scale)
                self._scale_dev.copy_(self._scale_host, non_blocking=True)
                _C.check("ft_grad_decide_dev", self._lib.ft_grad_decide_dev(
                    grads.data_ptr(), _C.dtype_code(grads.dtype), grads.numel(), self._scale_dev.data_ptr(), self.stats_ptr,
                    0 if self._fresh else 1, float(max_grad_norm) if max_grad_norm else 0.0, target.data_ptr(),
                    self._ws.data_ptr(), self._ws_bytes, _C.current_stream_ptr(grads.device)))
            else:
                _C.check("ft_grad_decide", self._lib.ft_grad_decide(
                    grads.data_ptr(), _C.dtype_code(grads.dtype), grads.numel(), inv_scale, self.stats_ptr,
                    0 if self._fresh else 1, inv_scale, float(max_grad_norm) if max_grad_norm else 0.0, target.data_ptr(),
                    self._ws.data_ptr(), self._ws_bytes, _C.current_stream_ptr(grads.device)))
        self._fresh = False
        return target

    def accumulate(self, acc: torch.Tensor, grads: torch.Tensor, scale: float = 1.0, zero_grads: bool = False,
                   with_stats: bool = False, loss_scale: float = 1.0, decide: bool = False,
                   max_grad_norm: Optional[float] = None) -> Optional[torch.Tensor]:
        """``acc += scale * grads`` in one pass (one fused multiply-add per element, rounded to
        ``acc``'s dtype), optionally clearing ``grads`` and -- ``with_stats`` -- gathering the
        statistics of the new ``acc`` as ``add(acc, loss_scale)`` would, so that the last
        accumulation of a step needs no separate statistics pass. Replaces the reference's
        per-micro-batch ``gradacc_buffer += extra_grads`` and ``zero_`` pair
        (``flextrain/memory/coordinator/optimizer.py:743,775-777``).

        ``decide`` (implies ``with_stats``): the pass also takes the step decision from the record as
        it then stands, like ``decide_async``, and returns the control record -- for the last
        accumulation before an update of the same buffer. The tail of ``acc`` is then left in the
        memory-side cache for that update to find."""
        with_stats = with_stats or decide
        for name, t in (("acc", acc), ("grads", grads)):
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous GPU tensor")
        if acc.numel() != grads.numel():
            raise ValueError("acc and grads must have the same number of elements")
        stats_ptr = self.stats_ptr if with_stats else None
        if with_stats:
            need = int(self._lib.ft_grad_accumulate_workspace_bytes(acc.numel()))
            if need > self._ws_bytes:  # grows with the largest buffer seen (16 bytes per 256 elements)
                self._ws = torch.empty(need, dtype=torch.uint8, device=self.device)
                self._ws_bytes = need
        inv_scale = float(1.0 / float(loss_scale))
        with torch.cuda.device(acc.device):
            if decide:
                _C.check("ft_grad_accumulate_decide", self._lib.ft_grad_accumulate_decide(
                    acc.data_ptr(), _C.dtype_code(acc.dtype), grads.data_ptr(), _C.dtype_code(grads.dtype), acc.numel(),
                    float(scale), int(bool(zero_grads)), inv_scale, stats_ptr, 0 if self._fresh else 1, inv_scale,
                    float(max_grad_norm) if max_grad_norm else 0.0, self.control.data_ptr(), self._ws.data_ptr(),
                    self._ws_bytes, _C.current_stream_ptr(acc.device)))
            else:
                _C.check("ft_grad_accumulate", self._lib.ft_grad_accumulate(
                    acc.data_ptr(), _C.dtype_code(acc.dtype), grads.data_ptr(), _C.dtype_code(grads.dtype), acc.numel(),
                    float(scale), int(bool(zero_grads)), inv_scale, stats_ptr,
                    0 if self._fresh else 1, self._ws.data_ptr(), self._ws_bytes, _C.current_stream_ptr(acc.device)))
        if with_stats:
            self._fresh = False
        return self.control if decide else None

    def decide_async(self, loss_scale: float = 1.0, max_grad_norm: Optional[float] = None,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Turns the statistics gathered so far into a control record on the device and returns it
        (the guard's own record, or ``out``: 16 bytes of device memory, 16-byte aligned, for callers
        that keep one record per unit of work)."""
        if self._fresh:
            raise RuntimeError("decide() before any add()")
        inv_scale = float(1.0 / float(loss_scale))
        target = self.control if out is None else out
        if out is not None and (not out.is_cuda or out.numel() * out.element_size() < 16 or out.data_ptr() % 16):
            raise ValueError("out must be 16 bytes of 16-byte aligned device memory")
        with torch.cuda.device(self.device):
            _C.check("ft_grad_control", self._lib.ft_grad_control(
                self.stats_ptr, inv_scale, float(max_grad_norm) if max_grad_norm else 0.0,
                target.data_ptr(), _C.current_stream_ptr(self.device)))
        return target

    def decide(self, loss_scale: float = 1.0, max_grad_norm: Optional[float] = None) -> GuardDecision:
        self.decide_async(loss_scale, max_grad_norm)
        return self.read()

    def read(self) -> GuardDecision:
        """The decision last taken by ``decide_async`` (reads 32 bytes back; waits for the stream)."""
        host = self._buf.cpu()  # synchronises with the current stream
        nonfinite = int(host[0:1].view(torch.int64).item())
        sumsq = float(host[1].item())
        ctl = host[2:4].view(torch.float32)
        return GuardDecision(
            overflow=nonfinite != 0, nonfinite=nonfinite, sumsq=sumsq,
            grad_norm=float(ctl[2].item()), clip_coef=float(ctl[3].item()), grad_mult=float(ctl[1].item()),
        )
