"""Optimizer front end: the reference's ``flextrain/optimizer.py`` surface over GPU kernels.

``FlexTrainCPUOptimizer`` keeps its reference name and abstract methods
(``flextrain/optimizer.py:24-95``) so that a coordinator written against it keeps working; the
"CPU" in the name is historical here, the arithmetic runs on the GPU.

``FlexTrainOptimizer`` (reference ``:98-272``) groups parameters, owns the flat buffers of the
parameters that do not belong to a layer unit, and steps them. What changes against the
reference is where the data lives: gradients are consumed on the GPU where backward left them
(no converting D2H copy, ``:253-254``), the master parameters and Adam states are either resident
in HBM or streamed from pinned host memory, and the low-precision parameters are written by the
update kernel itself (no converting H2D copy, ``:263``).
"""
from __future__ import annotations

from abc import ABC, abstractmethod
from collections.abc import Iterable
from typing import Callable, Dict, List, Optional, Union

import torch
from torch import Tensor

from .param_group import (
    GroupSegment,
    ParamGroup,
    StepContext,
    create_group_segments,
    create_step_contexts,
)

STEP_KEY = "step"
PARAMS_KEY = "params"


class FlexTrainCPUOptimizer(ABC):
    """Abstract step engine: subclasses implement the arithmetic for one contiguous segment."""

    #: where ``_init_optimizer_states`` and ``profile_step`` place master state:
    #: "cuda" keeps it resident in HBM, "cpu" keeps it in pinned host memory (streamed step)
    state_device: str = "cuda"

    @abstractmethod
    def __init__(self):
        pass

    @abstractmethod
    def _init_optimizer_states(self, numel: int, dtype: torch.dtype) -> List[Tensor]:
        pass

    @abstractmethod
    def _step(
        self, param_group: ParamGroup,
        half_parameter: Optional[Tensor], full_parameter: Tensor,
        gradient: Tensor, *optimizer_states: Tensor, **extensions
    ):
        pass

    @torch.no_grad()
    def step(self, step_contexts: Union[StepContext, List[StepContext]], *, loss_scale: float = 1.0,
             max_grad_norm: Optional[float] = None, check_overflow: bool = False, **extensions):
        """Steps every context; contexts without gradient elements are skipped
        (reference ``flextrain/optimizer.py:44-69``).

        Keyword-only additions, whose defaults give the reference's behaviour:
          loss_scale: the gradients were produced from ``loss * loss_scale``; the update divides
            them by it (one fp32 multiply by ``1/loss_scale``) on the fly.
          check_overflow: look for inf/nan in the gradients of ALL the given contexts first; if any
            is found no context is stepped (parameters and states keep their bits).
          max_grad_norm: clip the L2 norm of the unscaled gradients of all the given contexts
            together to this value.
        With ``check_overflow`` or ``max_grad_norm`` the decision is taken on the device and the
        call returns a ``GuardDecision`` (a 32-byte read-back after the update is enqueued; the
        caller advances ``group["step"]`` and the loss scale from it); otherwise it returns None.
        Gradients must then be GPU tensors. Other ``extensions`` (``grad_mult``, ``control``,
        ``blocking``) are forwarded to ``_step`` unchanged.
        """
        if isinstance(step_contexts, StepContext):
            step_contexts = [step_contexts]
        guard = None
        if check_overflow or max_grad_norm is not None:
            if "control" in extensions or "grad_mult" in extensions:
                raise ValueError("check_overflow / max_grad_norm compute the control record themselves; "
                                 "do not pass control or grad_mult as well")
            live = [ctx.gradient for ctx in step_contexts if ctx.gradient.numel()]
            if live:
                from .loss_scaler import GradientGuard  # local import: keeps module load light
                guard = getattr(self, "_step_guard", None)
                if guard is None or guard.device != live[0].device:
                    guard = self._step_guard = GradientGuard(live[0].device)
                guard.begin()
                for g in live[:-1]:
                    guard.add(g, loss_scale=loss_scale)
                extensions["control"] = guard.add_and_decide(live[-1], loss_scale=loss_scale, max_grad_norm=max_grad_norm)
        elif loss_scale != 1.0:
            if "control" in extensions:
                raise ValueError("loss_scale is already part of the control record passed in")
            extensions["grad_mult"] = float(extensions.get("grad_mult", 1.0)) * float(1.0 / float(loss_scale))
        self._step_all(step_contexts, extensions)
        return guard.read() if guard is not None else None

    def _step_all(self, step_contexts: List[StepContext], extensions) -> None:
        """One native call per context as in the reference's loop -- unless the engine can take
        several resident contexts in one launch (``_step_many``) and there is more than one."""
        many = getattr(self, "_step_many", None)
        if many is not None and len(step_contexts) > 1:
            live = [ctx for ctx in step_contexts if ctx.gradient.numel()]
            resident = [ctx for ctx in live if ctx.full_parameter.is_cuda]
            if len(resident) > 1 and len({(c.full_parameter.device, c.gradient.dtype) for c in resident}) == 1 \
                    and len({c.half_parameter.dtype for c in resident if c.half_parameter is not None}) <= 1 \
                    and set(extensions) <= {"grad_mult", "control", "blocking", "guard_stream"}:
                many(resident, grad_mult=extensions.get("grad_mult", 1.0), control=extensions.get("control"))
                step_contexts = [ctx for ctx in live if not ctx.full_parameter.is_cuda]
        for ctx in step_contexts:
            if not ctx.gradient.numel():
                continue
            self._step(
                ctx.param_group, ctx.half_parameter, ctx.full_parameter,
                ctx.gradient, *ctx.optimizer_states, **extensions
            )

    def _allocate(self, numel: int, dtype: torch.dtype, fill: str) -> Tensor:
        """A flat buffer on ``state_device`` (pinned, exact size, when that is the host)."""
        if self.state_device == "cpu":
            from .memory import pinned_empty
            t = pinned_empty(numel, dtype)
        else:
            t = torch.empty(numel, dtype=dtype, device=torch.device("cuda", torch.cuda.current_device()))
        if fill == "zeros":
            t.zero_()
        elif fill == "randn":
            t.normal_()
        return t

    @torch.no_grad()
    def profile_step(self, numel: int, device_dtype: torch.dtype, master_dtype: torch.dtype):
        """One step on private scratch buffers, for throughput probes
        (reference ``flextrain/optimizer.py:71-95``; driven by ``flextrain/auto_config.py:281-317``).
        Buffers are created on first use and reused; every call advances a private step counter.
        """
        if not hasattr(self, "_param_group"):
            self._param_group = {STEP_KEY: 0}
            if self.state_device == "cpu":
                self._half_parameter = self._allocate(numel, device_dtype, "empty")
                self._full_parameter = self._allocate(numel, master_dtype, "randn")
                self._gradient = self._allocate(numel, master_dtype, "randn")
                self._optimizer_states = self._init_optimizer_states(numel, master_dtype)
            else:  # resident: all arrays of the update in one allocation with staggered starts
                from .memory import allocate_device_arrays
                states = len(self._init_optimizer_states(1, master_dtype))
                arrays = allocate_device_arrays(
                    [(numel, device_dtype)] + [(numel, master_dtype)] * (2 + states),
                    torch.device("cuda", torch.cuda.current_device()))
                self._half_parameter, self._full_parameter, self._gradient = arrays[:3]
                self._full_parameter.normal_()
                self._gradient.normal_()
                self._optimizer_states = tuple(arrays[3:])
        self._param_group[STEP_KEY] += 1
        self._step(
            self._param_group,
            self._half_parameter, self._full_parameter,
            self._gradient, *self._optimizer_states
        )


class FlexTrainOptimizer:
    """Groups parameters for optimisation and steps those that belong to no layer unit.

    Args:
        param_groups: list of dicts with a ``"params"`` list plus optional hyper-parameters, or a
            bare iterable of parameters (wrapped into one group).
        unit_parameter_map: ``{unit_index: object with .paras}`` -- the layer units whose
            parameters another component steps unit by unit (in the reference this comes from
            the parameter coordinator, ``flextrain/optimizer.py:131-152``). Default: none, every
            parameter is stepped here.
        aligned_unit_numel: padded element count of one unit; the last segment of each unit is
            stretched to it (``:147-150``).
        device_dtype / master_dtype / gradacc_dtype: the reference reads these from its global
            config (``:159-163``); here they are arguments. ``device_dtype`` defaults to the dtype
            of the first parameter, ``gradacc_dtype`` to ``device_dtype``.
        offload: keep master parameters and optimizer state in pinned host memory and stream
            them through the GPU each step, instead of keeping them resident in HBM.
        loss_scaler: object with ``loss_scale`` and ``update_scale(overflow)``
            (``flextrain_amd.loss_scaler``); when given, gradients are unscaled by
            ``1/loss_scale`` inside the update and an inf/nan anywhere skips the step.
        max_grad_norm: clip the global L2 norm of the unscaled gradients to this value.
        grad_reduce_fn: called with the flat gradient buffer before anything else (the place of
            the reference's ``all_reduce(AVG)``, ``:250``); default none (one GPU).
        capturable: keep every group's per-step scalars (and 1/loss_scale) in device memory, so that
            ``enqueue_step()`` can be recorded into a HIP graph once and replayed every iteration:
            ``update_states()`` refreshes the pinned staging copies, the recorded region copies them
            to the device. Resident state only.
    """

    cpu_optimizer: FlexTrainCPUOptimizer = None

    def __init__(
        self,
        param_groups: List[Dict],
        *,
        unit_parameter_map: Optional[Dict[int, object]] = None,
        aligned_unit_numel: Optional[int] = None,
        device_dtype: Optional[torch.dtype] = None,
        master_dtype: torch.dtype = torch.float32,
        gradacc_dtype: Optional[torch.dtype] = None,
        offload: bool = False,
        loss_scaler=None,
        max_grad_norm: Optional[float] = None,
        grad_reduce_fn: Optional[Callable[[Tensor], None]] = None,
        capturable: bool = False,
    ):
        assert isinstance(param_groups, Iterable)
        assert self.cpu_optimizer is not None, "a subclass must create self.cpu_optimizer first"
        param_groups = list(param_groups)
        if not all(isinstance(group, dict) for group in param_groups):
            param_groups = [{PARAMS_KEY: param_groups}]
        self.param_groups = param_groups
        self.loss_scaler = loss_scaler
        self.max_grad_norm = max_grad_norm
        self._grad_reduce_fn = grad_reduce_fn
        self._offload = bool(offload)
        self.cpu_optimizer.state_device = "cpu" if self._offload else "cuda"

        # parameter -> (its group, its position in the caller's order)
        param_group_map: Dict[Tensor, Dict] = {}
        param_id_map: Dict[Tensor, int] = {}
        for group in self.param_groups:
            assert isinstance(group[PARAMS_KEY], list)
            for param in group[PARAMS_KEY]:
                param_group_map[param] = group
                param_id_map[param] = len(param_id_map)

        # Layer units: record their group segments, and leave their parameters to the caller.
        self.unit_group_segments: Dict[int, List[GroupSegment]] = {}
        remaining = dict.fromkeys(param_group_map.keys())
        for index, unit in (unit_parameter_map or {}).items():
            paras = list(unit.paras)
            for p in paras:
                remaining.pop(p, None)
            segments = create_group_segments(paras, [param_group_map[p] for p in paras])
            if aligned_unit_numel is not None and segments:
                assert segments[-1].end <= aligned_unit_numel
                segments[-1].end = aligned_unit_numel
            self.unit_group_segments[index] = segments
        non_layerwise_params = sorted(remaining.keys(), key=lambda p: param_id_map[p])

        if device_dtype is None:
            device_dtype = non_layerwise_params[0].dtype if non_layerwise_params else torch.float32
        if gradacc_dtype is None:
            gradacc_dtype = device_dtype
        if master_dtype != torch.float32:
            raise ValueError("master parameters and optimizer states are fp32 on this path")
        self._device_dtype, self._master_dtype, self._gradacc_dtype = device_dtype, master_dtype, gradacc_dtype
        self._gradacc_dtype_incompatible = device_dtype != gradacc_dtype

        device = torch.device("cuda", torch.cuda.current_device())
        total_numel = sum(p.numel() for p in non_layerwise_params)
        self._device_para = torch.zeros(total_numel, dtype=device_dtype, device=device)
        self._device_grad = torch.zeros(total_numel, dtype=device_dtype, device=device)
        if self._gradacc_dtype_incompatible:
            self._device_acc_grad = torch.zeros(total_numel, dtype=gradacc_dtype, device=device)

        # Gather the parameters into the flat device buffer (views replace the originals).
        offset = 0
        for param in non_layerwise_params:
            n = param.numel()
            view = self._device_para[offset:offset + n]
            view.copy_(param.data.reshape(-1))
            param.data = view.view(param.shape)
            offset += n

        # fp32 master copy: resident (aliases the device buffer when that is fp32 already) or
        # pinned host memory when offloaded.
        if self._offload:
            from .memory import pinned_empty
            self._master_para = pinned_empty(total_numel, master_dtype)
            self._master_para.copy_(self._device_para)
        elif device_dtype == master_dtype:
            self._master_para = self._device_para
        else:
            self._master_para = self._device_para.to(master_dtype)
        # Wire gradients: backward writes into the flat device buffer (or accumulates into the
        # wider one through a hook, reference :194-215).
        self.non_layerwise_master_params: List[torch.nn.Parameter] = []
        acc_views: List[Tensor] = []

        def _accumulate_into(i: int):
            def hook(grad: Tensor):
                acc_views[i] += grad.flatten()
            return hook

        offset = 0
        for i, param in enumerate(non_layerwise_params):
            end = offset + param.numel()
            self.non_layerwise_master_params.append(torch.nn.Parameter(self._master_para[offset:end]))
            param.grad = self._device_grad[offset:end].view_as(param)
            if self._gradacc_dtype_incompatible:
                acc_views.append(self._device_acc_grad[offset:end])
                param.register_hook(_accumulate_into(i))
            offset = end

        grad_buffer = self._device_acc_grad if self._gradacc_dtype_incompatible else self._device_grad
        self._step_grad = grad_buffer
        self.non_layerwise_step_contexts = create_step_contexts(
            group_segments=create_group_segments(
                non_layerwise_params, [param_group_map[p] for p in non_layerwise_params]),
            half_parameter=self._device_para if device_dtype != master_dtype else None,
            full_parameter=self._master_para,
            gradient=grad_buffer,
            optimizer_states=self.cpu_optimizer._init_optimizer_states(total_numel, master_dtype),
        )
        self.last_step_skipped = False
        self.last_grad_norm: Optional[float] = None
        self.capturable = bool(capturable)
        if self.capturable:
            if self._offload:
                raise ValueError("capturable=True needs resident state (offload=False): the streamed step blocks on the host")
            for group in self.param_groups:
                self.cpu_optimizer.make_capturable(group, device)

    @property
    def optimizer_state_per_element(self) -> int:
        """Number of optimizer-state tensors per parameter element (2 for Adam)."""
        return len(self.cpu_optimizer._init_optimizer_states(1, self._master_dtype))

    @property
    def non_layerwise_numel(self) -> int:
        return self._device_para.numel()

    def step(self, *args, **kwargs):
        """Steps the non-layerwise parameters (reference ``flextrain/optimizer.py:244-263``).

        Returns True if the update was applied, False if it was skipped because of inf/nan.
        ``enqueue_step()`` followed by ``complete_step()``: nothing is read back from the GPU before
        the update has been enqueued.
        """
        self.enqueue_step()
        return self.complete_step()

    def enqueue_step(self) -> None:
        """Everything of a step that runs on the GPU, enqueued on the current stream: statistics of
        the gradients, the skip / unscale / clip decision (a 16-byte record that stays on the
        device), the update reading that record, clearing the gradients. With resident state the
        call does not wait for the GPU, allocates nothing after its first use and clears with
        kernels, so a caller may record it into a HIP graph and replay it -- as long as the
        hyper-parameters that travel by value (``group["step"]``, ``lr``, the loss scale) are meant
        to stay what they were at capture. Offloaded state: the streamed update blocks until the
        host arrays hold the new values, as the reference's host step does."""
        grads = self._step_grad
        if self._grad_reduce_fn is not None:
            self._grad_reduce_fn(grads)
        extensions = {}
        self._step_guarded = (self.loss_scaler is not None or self.max_grad_norm is not None) and grads.numel() > 0
        if self.capturable:
            for group in self.param_groups:  # 48-byte copies; recorded, they re-read the staging copies at every replay
                group["hyper_record"].sync()
        if self._step_guarded:
            scale = float(self.loss_scaler.loss_scale) if self.loss_scaler is not None else 1.0
            self._step_guard(grads.device)
            self._guard.begin()
            extensions["control"] = self._guard.add_and_decide(grads, loss_scale=scale, max_grad_norm=self.max_grad_norm)
        self.cpu_optimizer.step(self.non_layerwise_step_contexts, **extensions)
        self._zero_grads()
        if self._offload and self._device_dtype == self._master_dtype:
            self._device_para.copy_(self._master_para, non_blocking=True)

    def _step_guard(self, device):
        if not hasattr(self, "_guard"):
            from .loss_scaler import GradientGuard  # local import: keeps module load light
            self._guard = GradientGuard(device=device, capturable=self.capturable)
            if self.capturable:
                self._guard.set_scale(float(self.loss_scaler.loss_scale) if self.loss_scaler is not None else 1.0)
        return self._guard

    def complete_step(self) -> bool:
        """Host side of a step, after ``enqueue_step()`` (or after replaying a graph that holds it):
        reads the 32-byte statistics + decision record, hands the overflow flag to the loss scaler,
        sets ``last_step_skipped`` / ``last_grad_norm``. Returns True if the update was applied."""
        self.last_step_skipped = False
        if not getattr(self, "_step_guarded", False):
            return True
        decision = self._guard.read()
        self.last_grad_norm = decision.grad_norm
        if self.loss_scaler is not None:
            self.loss_scaler.update_scale(decision.overflow)
            if self.capturable:  # what the next (replayed) step unscales with
                self._guard.set_scale(float(self.loss_scaler.loss_scale))
        self.last_step_skipped = bool(decision.overflow)
        return not decision.overflow

    def _zero_grads(self):
        self._device_grad.zero_()
        if self._gradacc_dtype_incompatible:
            self._device_acc_grad.zero_()

    def update_states(self):
        """Advances ``group["step"]`` of every group (reference ``:265-272``)."""
        if self.capturable:
            # a step in flight (or a graph replay) must have read the staging copies before they change:
            # one wait for all groups
            torch.cuda.synchronize()
        for group in self.param_groups:
            group[STEP_KEY] = group.get(STEP_KEY, 0) + 1
            if self.capturable:  # staging copy only: whatever steps next brings it to the device first
                group["hyper_record"].fill(group, wait=False)
