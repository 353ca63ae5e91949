"""Adam / AdamW on the GPU behind the reference's ``flextrain.ops.adam`` surface.

``FlexTrainCPUAdam`` mirrors the reference class of that name (``flextrain/ops/adam/cpu_adam.py:17-135``):
same constructor arguments and defaults, same ``_init_optimizer_states`` / ``_step`` contract, an
optimizer id registered with the native library on construction and released on deletion.
The native side is libftadam.so (hand-written gfx950 kernels) instead of the AVX/OpenMP extension,
so the tensors handed to ``_step`` are GPU tensors (resident mode) or pinned host tensors that are
streamed through the GPU in chunks (offloaded mode).

``FlexTrainAdam`` mirrors ``flextrain/ops/adam/__init__.py:10-34``.

Additions over the reference, all optional and neutral by default:
  * gradients may be fp32, fp16 or bf16; the low-precision copy is written in *its own* dtype
    (the reference writes fp16 bit patterns whatever the tensor's dtype, ``simd.h:35-37``);
  * ``grad_mult`` (one fp32 multiply applied to each gradient element on load: unscale x clip) and
    ``control`` (a device-side skip / multiplier decision) for mixed-precision training.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Dict, List, Optional

import torch
from torch import Tensor

from . import _C
from .optimizer import STEP_KEY, FlexTrainCPUOptimizer, FlexTrainOptimizer

#: elements per chunk of the offloaded step (64 Mi elements = 256 MiB per fp32 array)
DEFAULT_OFFLOAD_CHUNK = 64 * 1024 * 1024
DEFAULT_OFFLOAD_SLOTS = 3


#: key under which a parameter group carries its device-resident scalars (``make_capturable``)
HYPER_KEY = "hyper_record"


class HyperRecord:
    """The per-step scalars of one parameter group (step count folded into the bias corrections,
    learning rate, betas, epsilon, weight decay) in device memory, with a pinned host staging copy.

    By default those scalars reach the kernels by value, so a HIP graph that records a step replays
    the step count and learning rate of the moment it was recorded. A group that carries a record
    has them read from device memory instead: ``fill()`` computes them on the host exactly as the
    by-value path does and writes the pinned staging copy (call it whenever ``group["step"]`` or a
    hyper-parameter changes; outside any capture; it waits for the device first, so that a step still
    in flight reads the values it was enqueued with); ``sync()`` enqueues the 48-byte copy to the device
    on the current stream -- recorded into a graph, that copy re-reads the staging copy at every
    replay, so a recorded step follows the group from iteration to iteration. A step that meets a
    record changed since its last ``sync()`` calls ``sync()`` itself first (eager callers need not
    think of it; a recorded region should still hold its own ``sync()``, since a replay runs no
    Python)."""

    def __init__(self, engine: "FlexTrainCPUAdam", device: torch.device):
        self._engine = engine
        self.host = torch.zeros(12, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(12, dtype=torch.int32, device=device)
        #: the staging copy has changed since it last went to the device: a step that finds the flag
        #: set copies the record over first (``_step`` / ``_step_many``), so that no caller can
        #: consume a record that was never, or not since its last change, brought to the device
        self.dirty = True

    def fill(self, group_args: Dict, grad_mult: float = 1.0, wait: bool = True) -> "HyperRecord":
        """``wait=False``: the caller has already waited for the device since the last step was
        enqueued (one wait for all the groups of an optimizer instead of one per group)."""
        assert STEP_KEY in group_args, f"Key '{STEP_KEY}' not found in parameter group arguments."
        # A step enqueued earlier (or a graph replay) may not have copied the staging values yet:
        # they may only change once that work is done.
        if wait:
            torch.cuda.synchronize(self.dev.device)
        self.dirty = True
        self._engine._set_defaults_args(group_args)
        beta1, beta2 = group_args["betas"]
        _C.check("ft_adam_hyper_fill", self._engine._lib.ft_adam_hyper_fill(
            self._engine.opt_id, int(group_args[STEP_KEY]), float(group_args["lr"]), float(beta1), float(beta2),
            float(group_args["eps"]), float(group_args["weight_decay"]), int(bool(group_args["bias_correction"])),
            float(grad_mult), self.host.data_ptr()))
        return self

    def sync(self) -> "HyperRecord":
        self.dev.copy_(self.host, non_blocking=True)
        self.dirty = False
        return self


def _flat(name: str, t: Tensor, dtype_ok, numel: int) -> Tensor:
    if t.dtype not in dtype_ok:
        raise ValueError(f"{name} has dtype {t.dtype}, expected one of {sorted(map(str, dtype_ok))}")
    if t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, expected {numel}")
    if not t.is_contiguous():
        # The reference calls .contiguous() and then updates the temporary, losing the result
        # (cpu_adam_impl.cpp:225-228); refusing is the only safe reading of "in place".
        raise ValueError(f"{name} must be contiguous: the update is in place")
    return t


class FlexTrainCPUAdam(FlexTrainCPUOptimizer):
    """Fused Adam/AdamW step engine (GPU kernels; the class keeps its reference name)."""

    optimizer_id = 0
    _id_lock = threading.Lock()

    def __init__(
        self,
        lr=1e-3,
        bias_correction=True,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=0.01,
        amsgrad=False,
        adamw_mode=True,
        *args,
        offload_chunk_elems: int = DEFAULT_OFFLOAD_CHUNK,
        offload_slots: int = DEFAULT_OFFLOAD_SLOTS,
        offload_mode: int = 0,
        offload_window_piece_elems: int = 0,
        should_log: bool = False,
        **kwargs,
    ):
        # amsgrad is accepted and ignored, as in the reference (cpu_adam.py:63-66).
        self.default_args = dict(
            lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
            bias_correction=bias_correction, amsgrad=amsgrad,
        )
        FlexTrainCPUOptimizer.__init__(self)
        with FlexTrainCPUAdam._id_lock:
            self.opt_id = FlexTrainCPUAdam.optimizer_id
            FlexTrainCPUAdam.optimizer_id += 1
        self.adam_w_mode = adamw_mode
        self._lib = _C.lib()  # raises if the native library is missing: there is no fallback
        self._window_tensors = {}  # window token -> the host tensors it mirrors (kept alive while open)
        self._offload_chunk = int(offload_chunk_elems)
        self._offload_slots = int(offload_slots)
        self._offload_mode = int(offload_mode)  # FT_OFFLOAD_* of include/ft_adam.h; 0 = automatic
        self._offload_window_piece = int(offload_window_piece_elems)  # elements per piece of a window's copies; 0 = default
        self._engine: Optional[ctypes.c_void_p] = None
        _C.check("ft_adam_create", self._lib.ft_adam_create(
            self.opt_id, lr, betas[0], betas[1], eps, weight_decay, int(bool(adamw_mode)), int(bool(should_log))))

    def __del__(self):
        try:
            if self._engine is not None:
                self._lib.ft_offload_destroy(self._engine)
                self._engine = None
            self._lib.ft_adam_destroy(self.opt_id)
        except BaseException:
            pass

    def _set_defaults_args(self, group_args: Dict):
        for k, v in self.default_args.items():
            group_args.setdefault(k, v)

    def _init_optimizer_states(self, numel: int, dtype: torch.dtype) -> List[Tensor]:
        """exp_avg and exp_avg_sq, zero-filled, where the master state lives
        (reference ``cpu_adam.py:104-106`` returns two pinned host tensors)."""
        return [self._allocate(numel, dtype, "zeros") for _ in range(2)]

    # ------------------------------------------------------------------------------------------
    def _offload_engine(self) -> ctypes.c_void_p:
        if self._engine is None:
            handle = ctypes.c_void_p()
            _C.check("ft_offload_create", self._lib.ft_offload_create(
                self._offload_chunk, self._offload_slots, ctypes.byref(handle)))
            _C.check("ft_offload_set_mode", self._lib.ft_offload_set_mode(handle, self._offload_mode))
            _C.check("ft_offload_set_window_piece", self._lib.ft_offload_set_window_piece(handle, self._offload_window_piece))
            self._engine = handle
        return self._engine

    def _step(
        self, group_args: Dict,
        half_parameter: Optional[Tensor], full_parameter: Tensor,
        gradient: Tensor, *optimizer_states: Tensor,
        grad_mult: float = 1.0,
        control: Optional[Tensor] = None,
        blocking: Optional[bool] = None,
        guard_stream: bool = True,
    ):
        """One Adam/AdamW update of a contiguous segment, in place.

        Same contract as the reference ``_step`` (``cpu_adam.py:108-135``): ``group_args`` must hold
        ``"step"``; missing hyper-parameters are filled from the constructor's. With
        ``half_parameter`` the new parameters are also written there in its dtype.

        Resident mode (``full_parameter`` on the GPU): the kernel is enqueued on torch's current
        stream and the call returns at once. ``half_parameter`` alone may then live in pinned host
        memory: the kernel writes it there itself, and the host sees it once the stream has passed
        the kernel. Offloaded mode (``full_parameter`` in pinned host
        memory): the chunk pipeline is enqueued; with ``blocking`` (default in this mode) the call
        returns when the host arrays hold the new values, as the reference's host step does. With
        ``blocking=False`` the call returns at once; torch's current stream is then made to wait
        for the step's kernels (so that the gradients may be overwritten and the new copy read)
        unless ``guard_stream=False``, in which case the caller orders its own work with
        ``stream_wait()`` / ``synchronize()``.
        """
        assert STEP_KEY in group_args, f"Key '{STEP_KEY}' not found in parameter group arguments."
        self._set_defaults_args(group_args)
        if len(optimizer_states) != 2:
            raise ValueError("Adam needs exactly two optimizer states (exp_avg, exp_avg_sq)")
        exp_avg, exp_avg_sq = optimizer_states
        n = full_parameter.numel()
        f32 = {torch.float32}
        _flat("full_parameter", full_parameter, f32, n)
        _flat("exp_avg", exp_avg, f32, n)
        _flat("exp_avg_sq", exp_avg_sq, f32, n)
        _flat("gradient", gradient, set(_C.DTYPE_CODE), n)
        if half_parameter is not None:
            _flat("half_parameter", half_parameter, {torch.float16, torch.bfloat16}, n)
        if n == 0:
            return
        g_code = _C.dtype_code(gradient.dtype)
        h_code = _C.dtype_code(half_parameter.dtype) if half_parameter is not None else _C.F16
        h_ptr = half_parameter.data_ptr() if half_parameter is not None else None
        ctl_ptr = None
        if control is not None:
            if not control.is_cuda or control.numel() * control.element_size() < 16:
                raise ValueError("control must be a 16-byte device buffer (ft_step_control_t)")
            ctl_ptr = control.data_ptr()
        beta1, beta2 = group_args["betas"]
        hyper = (int(group_args[STEP_KEY]), float(group_args["lr"]), float(beta1), float(beta2),
                 float(group_args["eps"]), float(group_args["weight_decay"]),
                 int(bool(group_args["bias_correction"])), float(grad_mult))

        if full_parameter.is_cuda:
            for name, t in (("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq), ("gradient", gradient),
                            ("half_parameter", half_parameter)):
                if t is not None and t.device != full_parameter.device:
                    if name == "half_parameter" and not t.is_cuda and t.is_pinned():
                        continue  # the kernel writes the copy into pinned host memory over the link
                    raise ValueError(f"{name} is on {t.device} but full_parameter is on {full_parameter.device}")
            record = group_args.get(HYPER_KEY)
            with torch.cuda.device(full_parameter.device):
                if record is not None:  # the scalars are read from device memory (see HyperRecord)
                    if record.dirty:
                        record.sync()
                    if grad_mult != 1.0:
                        raise ValueError("a group with device-resident scalars takes its multiplier from the record "
                                         "(HyperRecord.fill(group, grad_mult=...)) or from a control record")
                    _C.check("ft_adam_step_hyper", self._lib.ft_adam_step_hyper(
                        self.opt_id, record.dev.data_ptr(), full_parameter.data_ptr(), gradient.data_ptr(), g_code,
                        exp_avg.data_ptr(), exp_avg_sq.data_ptr(), h_ptr, h_code, n, ctl_ptr,
                        _C.current_stream_ptr(full_parameter.device)))
                else:
                    _C.check("ft_adam_step", self._lib.ft_adam_step(
                        self.opt_id, *hyper, full_parameter.data_ptr(), gradient.data_ptr(), g_code,
                        exp_avg.data_ptr(), exp_avg_sq.data_ptr(), h_ptr, h_code, n, ctl_ptr,
                        _C.current_stream_ptr(full_parameter.device)))
            return

        # offloaded: master state in pinned host memory
        for name, t in (("full_parameter", full_parameter), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
            if t.is_cuda or not t.is_pinned():
                raise ValueError(f"{name} must be pinned host memory when full_parameter is on the host")
        for name, t in (("gradient", gradient), ("half_parameter", half_parameter)):
            if t is not None and not t.is_cuda and not t.is_pinned():
                raise ValueError(f"{name} must be on the GPU or in pinned host memory")
        g_on_host = int(not gradient.is_cuda)
        h_on_host = int(half_parameter is not None and not half_parameter.is_cuda)
        engine = self._offload_engine()
        _C.check("ft_offload_step", self._lib.ft_offload_step(
            engine, self.opt_id, *hyper, full_parameter.data_ptr(), gradient.data_ptr(), g_code, g_on_host,
            exp_avg.data_ptr(), exp_avg_sq.data_ptr(), h_ptr, h_code, h_on_host, n, ctl_ptr,
            _C.current_stream_ptr()))
        if blocking is None or blocking:
            _C.check("ft_offload_wait", self._lib.ft_offload_wait(engine))
        elif guard_stream and (gradient.is_cuda or (half_parameter is not None and half_parameter.is_cuda) or control is not None):
            # later work on the caller's stream may overwrite the gradients, read the new copy, or be
            # given the control record's memory once the caller lets go of it
            _C.check("ft_offload_stream_wait", self._lib.ft_offload_stream_wait(engine, _C.current_stream_ptr(), 0))

    def _step_many(self, step_contexts, grad_mult: float = 1.0, control: Optional[Tensor] = None) -> None:
        """Steps resident contexts -- each what one ``_step`` call would take, with its own group
        hyper-parameters and step count -- in as few kernel launches as possible: up to 16 contexts
        per launch (``ft_adam_step_multi``), instead of up to three launches per context. The
        reference loops over the contexts and calls the native step once for each
        (``flextrain/optimizer.py:44-69``). Results are those of ``_step`` context by context, bit
        for bit. All contexts must be on one GPU with one gradient dtype; the contexts of a call must
        not overlap."""
        live = [ctx for ctx in step_contexts if ctx.gradient.numel()]
        if not live:
            return
        first = live[0]
        device, g_dtype = first.full_parameter.device, first.gradient.dtype
        half_dtype = next((c.half_parameter.dtype for c in live if c.half_parameter is not None), torch.float16)
        ctl_ptr = None
        if control is not None:
            if not control.is_cuda or control.numel() * control.element_size() < 16:
                raise ValueError("control must be a 16-byte device buffer (ft_step_control_t)")
            ctl_ptr = control.data_ptr()
        segs = (_C.AdamSegment * len(live))()
        f32 = {torch.float32}
        for seg, ctx in zip(segs, live):
            group = ctx.param_group
            assert STEP_KEY in group, f"Key '{STEP_KEY}' not found in parameter group arguments."
            self._set_defaults_args(group)
            if len(ctx.optimizer_states) != 2:
                raise ValueError("Adam needs exactly two optimizer states (exp_avg, exp_avg_sq)")
            full, grad, half = ctx.full_parameter, ctx.gradient, ctx.half_parameter
            exp_avg, exp_avg_sq = ctx.optimizer_states
            n = full.numel()
            _flat("full_parameter", full, f32, n)
            _flat("exp_avg", exp_avg, f32, n)
            _flat("exp_avg_sq", exp_avg_sq, f32, n)
            _flat("gradient", grad, {g_dtype}, n)
            for name, t in (("full_parameter", full), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq), ("gradient", grad)):
                if t.device != device:
                    raise ValueError(f"{name} is on {t.device}, expected {device}: one call steps one GPU's contexts")
            if half is not None:
                _flat("half_parameter", half, {half_dtype}, n)
                if half.device != device and not (not half.is_cuda and half.is_pinned()):
                    raise ValueError(f"half_parameter is on {half.device}; it must be on {device} or in pinned host memory")
                seg.half_out = half.data_ptr()
            seg.p, seg.g, seg.m, seg.v, seg.n = full.data_ptr(), grad.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), n
            seg.step, seg.lr = int(group[STEP_KEY]), float(group["lr"])
            seg.beta1, seg.beta2 = group["betas"]
            seg.eps, seg.weight_decay = float(group["eps"]), float(group["weight_decay"])
            seg.bias_correction, seg.grad_mult = int(bool(group["bias_correction"])), float(grad_mult)
            record = group.get(HYPER_KEY)
            if record is not None:
                if grad_mult != 1.0:
                    raise ValueError("a group with device-resident scalars takes its multiplier from the record or a control record")
                if record.dirty:
                    with torch.cuda.device(device):
                        record.sync()
                seg.hyper = record.dev.data_ptr()
        with torch.cuda.device(device):
            _C.check("ft_adam_step_multi", self._lib.ft_adam_step_multi(
                self.opt_id, segs, len(live), _C.dtype_code(g_dtype), _C.dtype_code(half_dtype), ctl_ptr,
                _C.current_stream_ptr(device)))

    def make_capturable(self, group_args: Dict, device=None) -> HyperRecord:
        """Gives the parameter group a ``HyperRecord`` (kept under ``group_args["hyper_record"]``) and
        fills it from the group's present values: resident steps of that group then read their scalars
        from device memory and may be recorded into a HIP graph once and replayed across iterations.
        The caller keeps the record current: ``record.fill(group)`` after changing ``step`` or a
        hyper-parameter, ``record.sync()`` in front of the step (inside the recorded region)."""
        device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        record = group_args.get(HYPER_KEY)
        if record is None:
            group_args.setdefault(STEP_KEY, 0)
            record = group_args[HYPER_KEY] = HyperRecord(self, device)
        return record.fill(group_args)

    def open_window(self, full_parameter: Tensor, exp_avg: Tensor, exp_avg_sq: Tensor, write_through: bool = False) -> int:
        """Brings the whole master state of one unit (three pinned host tensors of equal length) to
        the GPU with large copies and keeps it there until ``close_window``: every ``_step`` on
        slices of these tensors in between is a plain in-place kernel on the device copy, and the
        host tensors are stale until the close has written them back (``synchronize()`` or
        ``stream_wait(write_back=True)`` after the close). For callers that step a unit in many
        small shares, where one copy per share would use the link badly. Returns a token."""
        n = full_parameter.numel()
        for name, t in (("full_parameter", full_parameter), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
            _flat(name, t, {torch.float32}, n)
            if t.is_cuda or not t.is_pinned():
                raise ValueError(f"{name} must be pinned host memory")
        token = ctypes.c_int(-1)
        _C.check("ft_offload_window_open", self._lib.ft_offload_window_open(
            self._offload_engine(), full_parameter.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), n,
            int(bool(write_through)), ctypes.byref(token)))
        # the engine holds raw addresses: keep the tensors alive until the write-back is enqueued
        self._window_tensors[int(token.value)] = (full_parameter, exp_avg, exp_avg_sq)
        return int(token.value)

    def close_window(self, token: int) -> None:
        """Enqueues the write-back of a window opened with ``open_window`` and returns."""
        _C.check("ft_offload_window_close", self._lib.ft_offload_window_close(self._offload_engine(), int(token)))
        self._window_tensors.pop(int(token), None)

    def synchronize(self):
        """Waits for every offloaded step enqueued so far (no-op if none was)."""
        if self._engine is not None:
            _C.check("ft_offload_wait", self._lib.ft_offload_wait(self._engine))

    def stream_wait(self, write_back: bool = False):
        """Makes torch's current stream wait for the last offloaded step: for its kernels, or with
        ``write_back`` for its copies back to host memory."""
        if self._engine is not None:
            _C.check("ft_offload_stream_wait", self._lib.ft_offload_stream_wait(
                self._engine, _C.current_stream_ptr(), 1 if write_back else 0))

    def last_offload_ms(self) -> float:
        """Device time of the last finished offloaded step, first H2D to last D2H."""
        ms = ctypes.c_float()
        _C.check("ft_offload_elapsed_ms", self._lib.ft_offload_elapsed_ms(self._offload_engine(), ctypes.byref(ms)))
        return float(ms.value)


class FlexTrainAdam(FlexTrainOptimizer):
    """User-facing Adam: creates the step engine, then groups parameters
    (reference ``flextrain/ops/adam/__init__.py:10-34``). Extra keyword arguments go to
    ``FlexTrainOptimizer`` (dtypes, ``offload``, ``loss_scaler``, ``max_grad_norm``...)."""

    def __init__(
        self,
        param_groups: List[Dict],
        lr=1e-3,
        bias_correction=True,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=0.01,
        amsgrad=False,
        adamw_mode=True,
        **optimizer_kwargs,
    ):
        self.cpu_optimizer = FlexTrainCPUAdam(
            lr=lr, bias_correction=bias_correction, betas=betas, eps=eps,
            weight_decay=weight_decay, amsgrad=amsgrad, adamw_mode=adamw_mode,
        )
        super().__init__(param_groups=param_groups, **optimizer_kwargs)
