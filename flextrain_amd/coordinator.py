"""Per-unit optimizer pipeline: the caller of the step, re-expressed for a GPU optimizer.

Mirror of the optimizer-step part of the reference's ``FlexTrainOptsCoordinator``
(``flextrain/memory/coordinator/optimizer.py``): the hooks a training loop calls around each
unit's forward and backward pass (``:733-794,825-888``), buffer rotation (``:494-498``), the split
of every unit's step into a forward share and a backward share (``:144-175,352-492``), planning a
share's step contexts (``:605-682``) and executing one micro-batch's part of them (``:684-696``).

What is kept: the schedule. While unit ``u`` runs backward, the optimizer steps the backward share
of unit ``u+1``, whose gradients are complete, one equal part per micro-batch, so the update is
spread between the backward kernels instead of arriving as one burst; the forward share of every
unit (the first ``alpha`` of each micro-batch's slice, the reference's alpha split) keeps its
gradients and is stepped during the NEXT iteration's forward pass, unit ``u+1`` while unit ``u``
runs forward, so that transfers of streamed state are spread over both passes. Master parameters
and Adam states of every unit live in pinned host memory as ``[master | exp_avg | exp_avg_sq]``
blocks, one per share (``:201-210``) -- or in HBM when ``offload=False`` -- and are seeded from the
units' low-precision parameters (``:239-350``).

What changes because the optimizer runs on the GPU:
  * gradients never leave the GPU: there is no reduce-scatter + converting D2H hop
    (``:534-583``), so the step of a unit follows its backward by one unit, not two, and the forward
    share's gradients stay where backward left them instead of moving into borrowed host buffers
    (``:352-421``): every unit then keeps a gradient buffer of its own (27 GB for a 7B model in
    bf16: what 288 GB of HBM are for);
  * the master state of the unit being stepped streams H2D / D2H through the offload engine,
    share by share, overlapping with the next unit's pass -- or, with ``unit_windows``, comes
    to the GPU in one piece one unit before its steps start (prefetch) and is stepped part by
    part from there; ordering is by events on the buffers involved, never by a device-wide
    synchronisation (``:819-823``);
  * the updated low-precision parameters are written by the update kernel straight into the
    unit's parameter buffer in HBM: no H2D copy of new parameters afterwards. A unit whose
    parameters are kept partly or wholly in pinned host memory (the reference's GPU part + CPU
    part, ``coordinator/parameter.py:470-519``) gets each element's new value in the piece that
    holds it, written over the link by the same step;
  * a unit whose master state is resident in HBM is stepped by one launch per share rather than a
    part per micro-batch (``resident_shares``): the parts exist to spread host work or transfers,
    and it has neither.
Left out (other subsystems): the NVMe tier, gradient reduce-scatter across ranks.

Mixed precision. The reference scales the loss (``flextrain/engine.py:249``) and never unscales
(``flextrain/loss_scaler.py:134-179`` is a state machine nobody drives). With ``loss_scaler=`` every
update multiplies its gradients by ``1/loss_scale`` on load, every unit's finished gradients are
checked for inf/nan (for free where the fused accumulation pass runs anyway, else one read of the
gradients) into ONE device-side record per iteration, and ``clear_backward_pipeline()`` returns the
iteration's ``GuardDecision`` and drives ``update_scale``. What a share can know when it is stepped
decides its policy:

  * the backward share of a unit is stepped before the units in front of it have produced their
    gradients, so its decision cannot be global. It is skipped (by its kernels, on the device, no
    host round trip) when an inf/nan has been seen in the unit's own gradients or in those of any
    unit that finished before it in this iteration; backward shares already stepped keep their
    update; the iteration counts as overflowed and the scale goes down. Clipping by the global
    norm is impossible here and refused.
  * the forward share of a unit that also has a backward share follows that unit's record: a unit
    is stepped whole or not at all, whichever pass a share runs in, and with the loss scale its
    gradients were produced under.
  * with ``alpha == 1`` (``defer_to_forward``) nothing is stepped before the iteration's one global
    decision, taken on the device after the first unit's backward: every unit is skipped or none,
    with one clip coefficient from the norm over ALL units.
"""
from __future__ import annotations

import contextlib
import math
from typing import List, Optional, Sequence, Tuple, Union

import torch
from torch import Tensor

from .memory import RotateContainer, allocate_device_arrays, allocate_memory_chunks
from .optimizer import FlexTrainOptimizer
from .param_group import StepContextContainer, flatten_list, slice_segments

FORWARD, BACKWARD = True, False


def _unpack_task(unit_or_task, micro_batch_index) -> Tuple[int, int]:
    """The hooks take ``(unit_index, micro_batch_index)`` or, as the reference's engine passes them
    (``coordinator/optimizer.py:733-782``; ``LLMTask``, ``flextrain/scheduler.py:5-13``), one object
    with ``.unit`` and ``.micro_batch``."""
    if micro_batch_index is None:
        return int(unit_or_task.unit), int(unit_or_task.micro_batch)
    return int(unit_or_task), int(micro_batch_index)


def _merge_ranges(ranges: Sequence[Tuple[int, int]]) -> List[Tuple[int, int]]:
    """Drops empty ranges and joins ranges that touch."""
    out: List[Tuple[int, int]] = []
    for lo, hi in ranges:
        if hi <= lo:
            continue
        if out and out[-1][1] == lo:
            out[-1] = (out[-1][0], hi)
        else:
            out.append((lo, hi))
    return out


def _slice_pieces(pieces: Sequence[Tensor], ranges: Sequence[Tuple[int, int]]) -> List[Tensor]:
    """Views of consecutive flat ``pieces`` (laid end to end) that cover the element ``ranges`` in
    order; a range that crosses a piece boundary yields one view per piece."""
    views: List[Tensor] = []
    edges, begin = [], 0
    for t in pieces:
        edges.append((begin, begin + t.numel(), t))
        begin += t.numel()
    for lo, hi in ranges:
        for p_lo, p_hi, t in edges:
            a, b = max(lo, p_lo), min(hi, p_hi)
            if a < b:
                views.append(t[a - p_lo:b - p_lo])
    return views


class _Share:
    """One of the two shares of every unit's step: which elements of a unit belong to it, the
    state blocks of every unit for those elements, and the step contexts."""

    def __init__(self, forward: bool, ranges: List[Tuple[int, int]]):
        self.forward = forward
        self.ranges = ranges                      # element ranges of a unit, ascending, merged
        self.numel = sum(hi - lo for lo, hi in ranges)
        self.opts: List[List[Tensor]] = []        # per unit: [master, exp_avg, exp_avg_sq] of `numel` elements
        self.ctxts: List[StepContextContainer] = []
        self.open_windows = {}                    # unit index -> window token


class FlexTrainOptsCoordinator:

    def __init__(self):
        self._initialized = False

    @property
    def is_initialized(self) -> bool:
        return self._initialized

    def _is_invalid_unit(self, unit_index: int) -> bool:
        return unit_index < 0 or unit_index >= self._num_units

    def _is_invalid_micro_batch(self, micro_batch_index: int) -> bool:
        return micro_batch_index < 0 or micro_batch_index >= self._micro_batch_per_rank

    def _is_invalid_task(self, unit_index: int, micro_batch_index: int) -> bool:
        return self._is_invalid_unit(unit_index) or self._is_invalid_micro_batch(micro_batch_index)

    # ------------------------------------------------------------------------------------------
    def initialize(
        self,
        optimizer: FlexTrainOptimizer,
        unit_half_parameters: Sequence[Union[Tensor, Sequence[Tensor]]],
        micro_batch_per_rank: int,
        *,
        device: Optional[torch.device] = None,
        gradacc_dtype: Optional[torch.dtype] = None,
        offload: bool = True,
        unit_windows: Optional[bool] = None,
        window_write_through: bool = False,
        resident_units: int = 0,
        resident_shares: Optional[int] = None,
        step_stream: Optional[bool] = None,
        loss_scaler=None,
        check_overflow: Optional[bool] = None,
        max_grad_norm: Optional[float] = None,
        alpha: float = 0.0,
        defer_to_forward: bool = False,
    ) -> None:
        """
        Args:
            optimizer: supplies ``cpu_optimizer`` (the step engine) and ``unit_group_segments``
                (which parameter group owns which element range of each unit).
            unit_half_parameters: per unit, the flat buffer holding the unit's low-precision
                parameters, all units of the same (padded) length: one GPU tensor, or a list of
                pieces that follow one another, each on the GPU or in pinned host memory, cut
                alike in every unit (the reference keeps a unit's parameters as a GPU part and a
                CPU part, ``coordinator/parameter.py:470-519``). The update writes the new values
                into whichever piece holds an element; pieces on the host are written over the
                link by the step itself and are complete after ``clear_backward_pipeline()``.
            device: GPU the gradients live on (default: that of the first GPU piece, else the
                current device).
            micro_batch_per_rank: number of equal parts a share's step is cut into; the unit
                length must be divisible by it.
            gradacc_dtype: dtype of the gradient buffers (default: the parameters' dtype).
            offload: master state in pinned host memory (streamed) or resident in HBM.
            unit_windows: with ``offload``, bring the whole state of a unit's share to the GPU with a
                few large copies one unit before its steps start (``FlexTrainCPUAdam.open_window``)
                and step its parts there, instead of streaming every part's own slice. Default
                (None): decided from the sizes -- per-part streaming only pays while each part
                has at least 32 Mi elements and a pass has at most 96 of them (measured on 24
                units: 4 parts 49.3 GB/s each way streamed against 47.2 with windows; 16 parts
                43.4 against 47.2).
            window_write_through: a window's results are written to the host by the step kernels
                themselves instead of being copied back in one piece after the share's last part
                (slower: 43.7 GB/s on the same schedule).
            resident_units: with ``offload``, keep the master state of units ``0 .. resident_units-1``
                in HBM all the same and stream only the others. Those are the units stepped last in
                an iteration (and needed first by the next forward pass), where no backward work is
                left to hide their transfers behind; every resident unit takes 12 bytes per
                element each way off the host link. The reference keeps all optimizer state on
                the host (``:133-136`` refuses a GPU optimizer); with 288 GB of HBM how much to
                offload is a dial, not a yes or no.
            resident_shares: how many launches the update of one share of a unit whose state is in
                HBM is cut into (a divisor of ``micro_batch_per_rank``; launch ``j`` is enqueued after
                micro-batch ``j * micro_batch_per_rank / resident_shares``). Equal parts per
                micro-batch spread a host-side step, or the transfers of a streamed one, evenly under
                the GPU's work; an update whose operands are all in HBM has nothing to spread and
                only pays two launch gaps per part. Default (None): one (32 Llama-7B layers, 32
                micro-batches, a gradient copy standing in for backward: 36.1 ms an iteration
                against 39.5 ms with a part per micro-batch). Streamed units always take one part
                per micro-batch.
            step_stream: enqueue the statistics passes and the updates on a stream of the
                coordinator's own instead of the caller's, so that they run beside the caller's
                kernels rather than between them. Ordering is by events: the step stream waits for
                the gradients it reads, the caller's stream waits for the step stream before it
                reuses a gradient buffer, before a forward pass reads the parameters the update
                wrote, and where an iteration ends. Default (None): off. It pays where the
                caller's kernels are many and short (the same 32 micro-batches: 34.4 ms); beside
                matrix products that fill every compute unit nothing overlaps (bf16 products
                costing a layer's backward over 2048 tokens per micro-batch, 16 layers x 4
                micro-batches: 129.6 ms against 128.7 ms on the caller's stream), and beside few
                long memory-bound kernels the two contend (4 micro-batches: 34.5 against 33.5 ms).
            loss_scaler: object with ``loss_scale`` and ``update_scale(overflow)``
                (``flextrain_amd.loss_scaler``): the gradients were produced from
                ``loss * loss_scale`` and are divided by it inside the update.
            check_overflow: look for inf/nan in every unit's gradients and skip on the device
                (default: on when a loss scaler is given).
            max_grad_norm: clip the L2 norm of the unscaled gradients of all units together to this
                value; needs ``alpha == 1`` (``defer_to_forward``).
            alpha: the share of every unit's step that runs during the next iteration's forward pass
                instead of during backward (the reference's ``split_ratio.alpha``, ``:148-175``): of
                each micro-batch's slice of a unit (``unit_numel / micro_batch_per_rank`` elements)
                the first ``ceil(alpha * slice)`` elements, rounded up to a multiple of 256, belong
                to the forward share, the rest to the backward share. 0 (default): everything during
                backward; 1: everything during forward. With ``0 < alpha`` every unit keeps its
                gradients in a buffer of its own until the forward share has been stepped. The
                caller follows the reference's order (``flextrain/engine.py:353-399``): forward pass
                with the forward-side hooks, ``update_states()``, backward pass, so that both shares
                of an iteration see the same step count.
            defer_to_forward: ``alpha = 1`` with the decision known before ANY update: backward only
                accumulates and gathers statistics, ``clear_backward_pipeline()`` takes one decision
                (skip everything or nothing, one clip coefficient), and the caller advances the step
                counters afterwards, only for an iteration that will be applied.
        """
        units = [[u] if isinstance(u, Tensor) else list(u) for u in unit_half_parameters]
        assert units and all(units)
        pieces = [t for u in units for t in u]
        assert all(t.dim() == 1 and t.is_contiguous() and (t.is_cuda or t.is_pinned()) for t in pieces), \
            "low-precision parameter pieces must be flat and on the GPU or in pinned host memory"
        assert all(t.dtype == pieces[0].dtype for t in pieces)
        self._optimizer = optimizer
        self._num_units = len(units)
        self._half_piece_numels = [t.numel() for t in units[0]]
        self._unit_numel = sum(self._half_piece_numels)
        assert all([t.numel() for t in u] == self._half_piece_numels for u in units), \
            "every unit must be cut into the same pieces"
        assert self._unit_numel % micro_batch_per_rank == 0
        self._micro_batch_per_rank = micro_batch_per_rank
        self._unit_half_parameters = units
        self._offload = bool(offload)

        # The alpha split: of every micro-batch's slice the first `fwd` elements go forward.
        if defer_to_forward:
            alpha = 1.0
        if not 0.0 <= float(alpha) <= 1.0:
            raise ValueError("alpha must lie in [0, 1]")
        self._alpha = float(alpha)
        slice_numel = self._unit_numel // micro_batch_per_rank
        fwd = 0 if alpha <= 0 else slice_numel if alpha >= 1 else min(slice_numel, -(-math.ceil(alpha * slice_numel) // 256) * 256)
        self._mb_fwd_numel, self._mb_bwd_numel = fwd, slice_numel - fwd
        self._fwd = _Share(FORWARD, _merge_ranges([(k * slice_numel, k * slice_numel + fwd) for k in range(micro_batch_per_rank)]))
        self._bwd = _Share(BACKWARD, _merge_ranges([(k * slice_numel + fwd, (k + 1) * slice_numel) for k in range(micro_batch_per_rank)]))
        self._has_fwd, self._has_bwd = self._fwd.numel > 0, self._bwd.numel > 0
        self._defer = self._has_fwd and not self._has_bwd  # no update before the iteration's one decision

        resident_units = max(0, min(int(resident_units), self._num_units)) if self._offload else self._num_units
        self._unit_resident = [u < resident_units for u in range(self._num_units)]
        if resident_shares is None:
            resident_shares = 1
        resident_shares = int(resident_shares)
        if resident_shares < 1 or micro_batch_per_rank % resident_shares:
            raise ValueError("resident_shares must divide micro_batch_per_rank")
        self._unit_shares = [resident_shares if r else micro_batch_per_rank for r in self._unit_resident]
        if unit_windows is None:
            part_numel = max(self._mb_fwd_numel, self._mb_bwd_numel)
            streamed_units = self._num_units - sum(self._unit_resident)
            unit_windows = not (part_numel >= 32 * 1024 * 1024 and streamed_units * micro_batch_per_rank <= 96)
        self._unit_windows = bool(unit_windows) and self._offload
        self._window_write_through = bool(window_write_through)
        if device is None:
            on_gpu = [t.device for t in pieces if t.is_cuda]
            device = on_gpu[0] if on_gpu else torch.device("cuda", torch.cuda.current_device())
        device = torch.device(device)
        device_dtype = pieces[0].dtype
        master_dtype = torch.float32
        self._emit_half = device_dtype != master_dtype
        if not self._emit_half:
            raise NotImplementedError("units must hold fp16 or bf16 parameters; the fp32 master copy is kept beside them")
        gradacc_dtype = gradacc_dtype or device_dtype
        self._gradacc_dtype_incompatible = gradacc_dtype != device_dtype
        self._device = device
        self._step_stream = torch.cuda.Stream(device=device) if step_stream else None

        self._loss_scaler = loss_scaler
        self._check_overflow = bool(loss_scaler is not None if check_overflow is None else check_overflow)
        self._max_grad_norm = float(max_grad_norm) if max_grad_norm else None
        if self._max_grad_norm is not None and not self._defer:
            raise ValueError("clipping by the global norm needs every unit's gradients before the first update: "
                             "use defer_to_forward=True (alpha = 1)")
        self._guarded = self._check_overflow or self._max_grad_norm is not None
        self._iter_guard = None       # the iteration's statistics record and scratch
        self._unit_controls = None    # one ft_step_control_t per unit (row u) + the global one (last row), 16 bytes each
        self._iteration_open = False  # statistics of the running iteration have been started
        self._pending_steps = False   # a decision has been taken and the forward shares not yet stepped
        self._deferred_skip = False
        self._deferred_grad_mult = 1.0
        self.last_decision = None
        self.last_skipped_units: List[int] = []
        if self._guarded:
            from .loss_scaler import GradientGuard
            self._iter_guard = GradientGuard(device)
            self._unit_controls = torch.zeros(self._num_units + 1, 4, dtype=torch.float32, device=device)
            self._unit_controls[:, 1] = 1.0
            self._unit_controls[:, 3] = 1.0

        # Everything during backward: two gradient buffers trade places every unit, [0] receives the
        # unit in backward, [1] holds the finished gradients of the unit being stepped. With a
        # forward share every unit keeps a buffer of its own until that share has been stepped, one
        # iteration later.
        # (Separately aligned arrays, not rows of one matrix: a unit length that is no multiple of the
        # vector width would leave every second row off its alignment.)
        self._gpu_bwd_grad_buffers = RotateContainer(tuple(
            allocate_device_arrays([(self._unit_numel, gradacc_dtype)] * 2, device))) if not self._has_fwd else None
        self._unit_grads = allocate_device_arrays([(self._unit_numel, gradacc_dtype)] * self._num_units, device) \
            if self._has_fwd else None
        self._bwd_unit = -1  # with per-unit buffers: the unit whose backward is running
        # When gradients are accumulated in a wider type than backward produces them in, backward
        # writes each micro-batch into this extra buffer and one fused pass per micro-batch adds it
        # to the receive buffer and clears it (reference ``:187-190,743,775-777``: a zero_ before
        # and a += after every micro-batch).
        self._gpu_bwd_extra_grads = None
        if self._gradacc_dtype_incompatible:
            from .loss_scaler import GradientGuard
            self._gpu_bwd_extra_grads = allocate_device_arrays([(self._unit_numel, device_dtype)], device)[0]
            self._guard = self._iter_guard if self._iter_guard is not None else GradientGuard(device)

        # [master | exp_avg | exp_avg_sq] per unit and share.
        per_element = 1 + optimizer.optimizer_state_per_element
        # Resident units: the arrays of an update in one allocation with staggered starts (the layout
        # the update kernel was never slow with); streamed units: exact-size pinned blocks.
        shares = [s for s in (self._fwd, self._bwd) if s.numel]
        for u in range(self._num_units):
            if self._unit_resident[u]:
                arrays = list(allocate_device_arrays([(s.numel, master_dtype) for s in shares for _ in range(per_element)], device))
                for k, s in enumerate(shares):
                    s.opts.append(arrays[k * per_element:(k + 1) * per_element])
            else:
                for s in shares:
                    s.opts.append(list(allocate_memory_chunks(s.numel, per_element, master_dtype, torch.device("cpu"))))

        # Seed the master copy from the low-precision parameters (exact: widening conversion).
        for u in range(self._num_units):
            self._copy_master_to_or_from_half(u, to_half=False)
        torch.cuda.current_stream(device).synchronize()

        # One container per unit and share: equal parts x parameter groups x buffer pieces.
        slice_plan = [self._mb_fwd_numel, self._mb_bwd_numel] * micro_batch_per_rank
        for u in range(self._num_units):
            segments = optimizer.unit_group_segments[u]
            assert segments and segments[-1].end == self._unit_numel, \
                "unit group segments must cover the padded unit (see FlexTrainOptimizer(aligned_unit_numel=...))"
            windows = slice_segments(segments, slice_plan)  # (forward, backward) per micro-batch, as ``:438-447``
            for s, mine in ((self._fwd, windows[0::2]), (self._bwd, windows[1::2])):
                if not s.numel:
                    continue
                half_numels = [t.numel() for t in _slice_pieces(units[u], s.ranges)]
                grad_numels = [hi - lo for lo, hi in s.ranges]
                s.ctxts.append(StepContextContainer(self._unit_shares[u], flatten_list(list(mine)), half_numels,
                                                    [s.numel], grad_numels))
        self._initialized = True

    # ---- the two shares --------------------------------------------------------------------------
    def _share(self, forward: bool) -> _Share:
        return self._fwd if forward else self._bwd

    def _shares(self) -> List[_Share]:
        return [s for s in (self._fwd, self._bwd) if s.numel]

    def _copy_master_to_or_from_half(self, unit_index: int, to_half: bool) -> None:
        """Range by range and piece by piece: seeds the fp32 master copies from the low-precision
        parameters (exact), or rounds the master copies back into them."""
        for s in self._shares():
            master, offset = s.opts[unit_index][0], 0
            for piece in _slice_pieces(self._unit_half_parameters[unit_index], s.ranges):
                part = master[offset:offset + piece.numel()]
                if to_half:
                    piece.copy_(part)
                else:
                    part.copy_(piece)
                offset += piece.numel()

    # ---- buffers -------------------------------------------------------------------------------
    @property
    def _gpu_bwd_receive_grads(self) -> Tensor:
        return self._unit_grads[self._bwd_unit] if self._has_fwd else self._gpu_bwd_grad_buffers[0]

    def _finished_grads(self, unit_index: int) -> Tensor:
        """The complete gradients of a unit whose backward has run."""
        return self._unit_grads[unit_index] if self._has_fwd else self._gpu_bwd_grad_buffers[1]

    @property
    def loss_scale(self) -> float:
        """What the training loop multiplies the loss by (reference ``flextrain/engine.py:249``)."""
        return float(self._loss_scaler.loss_scale) if self._loss_scaler is not None else 1.0

    def _gather(self, unit_index: int, which: int) -> Tensor:
        """Array `which` of the unit's state (0 master, 1 exp_avg, 2 exp_avg_sq) in the unit's element
        order. With one share that is the share's own array; with two a copy put together from both."""
        shares = self._shares()
        if len(shares) == 1:
            return shares[0].opts[unit_index][which]
        parts = [s.opts[unit_index][which] for s in shares]
        out = torch.empty(self._unit_numel, dtype=parts[0].dtype, device=parts[0].device)
        for s, part in zip(shares, parts):
            offset = 0
            for lo, hi in s.ranges:
                out[lo:hi] = part[offset:offset + hi - lo]
                offset += hi - lo
        return out

    def unit_master_parameter(self, unit_index: int) -> Tensor:
        """The unit's fp32 master parameters in element order (with ``0 < alpha < 1`` a gathered copy:
        the two shares keep their elements in blocks of their own)."""
        return self._gather(unit_index, 0)

    def unit_optimizer_states(self, unit_index: int) -> List[Tensor]:
        return [self._gather(unit_index, k) for k in range(1, 1 + self._optimizer.optimizer_state_per_element)]

    def unit_share_blocks(self, unit_index: int, forward: bool) -> List[Tensor]:
        """``[master, exp_avg, exp_avg_sq]`` of one share of a unit as they are kept (what the state
        files hold); empty list when the share has no elements."""
        s = self._share(forward)
        return list(s.opts[unit_index]) if s.numel else []

    def unit_step_contexts(self, unit_index: int, forward: bool = False) -> Optional[StepContextContainer]:
        """The step-context container of one share of a unit (None when the share has no elements)."""
        s = self._share(forward)
        return s.ctxts[unit_index] if s.numel else None

    def _rotate_buffers(self) -> None:
        if not self._has_fwd:
            self._gpu_bwd_grad_buffers.rotate()

    # ---- the step stream -----------------------------------------------------------------------
    def _on_step_stream(self):
        """Context under which statistics passes and updates are enqueued."""
        return torch.cuda.stream(self._step_stream) if self._step_stream is not None else contextlib.nullcontext()

    def _steps_follow_caller(self) -> None:
        """What is given to the step stream from here on runs after everything the caller's stream
        holds so far: the gradients and the records the steps read."""
        if self._step_stream is not None:
            self._step_stream.wait_stream(torch.cuda.current_stream(self._device))

    def _caller_follows_steps(self) -> None:
        """What the caller's stream is given from here on runs after every statistics pass and
        update enqueued so far: before a gradient buffer they read is written again, before a
        forward pass reads the parameters they wrote, before their records are read back."""
        if self._step_stream is not None:
            torch.cuda.current_stream(self._device).wait_stream(self._step_stream)

    # ---- steps ---------------------------------------------------------------------------------
    def _plan_optimizer_steps(self, unit_index: int, forward: bool, execute_now: bool = False) -> None:
        """Bind the step contexts of one share of the unit to its buffers (reference ``:605-682``)."""
        s = self._share(forward)
        if self._is_invalid_unit(unit_index) or not s.numel:
            return
        if forward and self._deferred_skip:
            return  # the whole iteration is skipped: nothing to bind, nothing to bring to the GPU
        blocks = s.opts[unit_index]
        s.ctxts[unit_index].plan(
            half_parameter=_slice_pieces(self._unit_half_parameters[unit_index], s.ranges),
            full_parameter=blocks[0],
            gradient=_slice_pieces([self._finished_grads(unit_index)], s.ranges),
            optimizer_states=[[b] for b in blocks[1:]],
        )
        self._sync_capturable_records()
        if forward:
            self._steps_follow_caller()  # the global decision was taken on the caller's stream
        elif self._gradacc_dtype_incompatible:
            # the unit's statistics came out of the accumulation passes on the caller's stream, which
            # will add the next unit's to the same record: the decision is taken there, before them
            self._decide_unit(unit_index)
            self._steps_follow_caller()
        else:
            self._steps_follow_caller()
            with self._on_step_stream():
                self._decide_unit(unit_index)
        self._open_unit_window(unit_index, forward)
        if execute_now:
            for mb in range(self._micro_batch_per_rank):
                self._execute_optimizer_step(unit_index, mb, forward)

    def _sync_capturable_records(self) -> None:
        """Groups whose per-step scalars live in device memory (``FlexTrainAdam(capturable=True)``):
        a record refreshed on the host since it last went to the device is copied there in front of
        the steps that read it, on the stream they run on."""
        with self._on_step_stream():
            for group in self._optimizer.param_groups:
                record = group.get("hyper_record")
                if record is not None and record.dirty:
                    record.sync()

    def _open_unit_window(self, unit_index: int, forward: bool) -> None:
        """Starts bringing one share of a unit's master state to the GPU (no-op without windows, for
        an invalid unit, or when it is already on its way). Called one unit ahead of the share's
        steps, so the copies run while the previous unit is still being stepped."""
        s = self._share(forward)
        if not s.numel or (forward and self._deferred_skip):
            return
        if self._unit_windows and not self._is_invalid_unit(unit_index) and not self._unit_resident[unit_index] \
                and unit_index not in s.open_windows:
            s.open_windows[unit_index] = self._optimizer.cpu_optimizer.open_window(
                *s.opts[unit_index], write_through=self._window_write_through)

    def _execute_optimizer_step(self, unit_index: int, micro_batch_index: int, forward: bool) -> None:
        """Step one micro-batch's part of one share of a unit (reference ``:684-696``). Returns as soon
        as the work is enqueued."""
        s = self._share(forward)
        if self._is_invalid_task(unit_index, micro_batch_index) or not s.numel:
            return
        if forward and self._deferred_skip:
            return
        every = self._micro_batch_per_rank // self._unit_shares[unit_index]
        if micro_batch_index % every:
            return  # a resident unit's launches are fewer than the micro-batches
        contexts = s.ctxts[unit_index][micro_batch_index // every]
        extensions = {}
        if self._guarded:  # skip and the gradient multiplier come from a device-side record: the unit's, or the global one
            extensions["control"] = self._unit_controls[self._num_units if self._defer else unit_index]
        elif self._loss_scaler is not None:
            # forward share: the scale the gradients were produced under, not what the scaler holds by now
            extensions["grad_mult"] = self._deferred_grad_mult if forward else float(1.0 / self.loss_scale)
        with self._on_step_stream():
            if self._unit_resident[unit_index]:
                self._optimizer.cpu_optimizer.step(contexts, **extensions)
            else:
                self._optimizer.cpu_optimizer.step(contexts, blocking=False, guard_stream=False, **extensions)
                if micro_batch_index == self._micro_batch_per_rank - 1 and unit_index in s.open_windows:
                    self._optimizer.cpu_optimizer.close_window(s.open_windows.pop(unit_index))

    # ---- statistics and decisions ---------------------------------------------------------------
    def _begin_iteration_statistics(self) -> None:
        if self._guarded and not self._iteration_open:
            self._iter_guard.begin()
            self._iteration_open = True

    def _gather_unit_statistics(self, grads: Tensor) -> None:
        """Adds one finished unit's gradients to the iteration's record -- unless the fused
        accumulation pass of its last micro-batch has done so already."""
        if self._guarded and not self._gradacc_dtype_incompatible:
            self._iter_guard.add(grads, loss_scale=self.loss_scale)

    def _decide_unit(self, unit_index: int) -> None:
        """Backward share: the unit's control record from everything seen so far in this iteration
        (its own gradients, forward share included, and those of the units that finished before it)."""
        if not self._guarded:
            return
        if self._gradacc_dtype_incompatible:  # the fused accumulation pass has gathered the unit's statistics
            self._iter_guard.decide_async(loss_scale=self.loss_scale, out=self._unit_controls[unit_index])
        else:
            self._iter_guard.add_and_decide(self._finished_grads(unit_index), loss_scale=self.loss_scale,
                                            out=self._unit_controls[unit_index])

    def _finish_iteration_statistics(self):
        """Reads the iteration's record back (one small copy), drives the loss scaler and returns the
        ``GuardDecision``; None when nothing is checked."""
        if not self._guarded:
            return None
        from .loss_scaler import GuardDecision
        self._caller_follows_steps()
        stats = self._iter_guard._buf[:2].cpu()  # waits for the stream: every statistics pass has run
        controls = self._unit_controls.cpu()
        nonfinite = int(stats[0:1].view(torch.int64).item())
        final = controls[self._num_units if self._defer else 0]  # the record that saw every unit
        skipped = (controls[:, 0].contiguous().view(torch.int32) != 0).tolist()
        if self._defer:
            self.last_skipped_units = list(range(self._num_units)) if skipped[self._num_units] else []
        else:
            self.last_skipped_units = [u for u in range(self._num_units) if skipped[u]]
        decision = GuardDecision(overflow=nonfinite != 0, nonfinite=nonfinite, sumsq=float(stats[1].item()),
                                 grad_norm=float(final[2].item()), clip_coef=float(final[3].item()),
                                 grad_mult=float(final[1].item()))
        self.last_decision = decision
        self._iteration_open = False
        if self._loss_scaler is not None:
            self._loss_scaler.update_scale(decision.overflow)
        return decision

    # ---- hooks of the training loop: backward ----------------------------------------------------
    def warmup_backward_pipeline(self) -> None:
        """Before the first unit's backward (reference ``:849-853``: completes its alpha-split set-up,
        which ``initialize`` has done here). Nothing to do; kept so that the reference's caller runs
        unchanged."""

    def pre_micro_batch_backward(self, unit_or_task, micro_batch_index: Optional[int] = None) -> None:
        """Before each micro-batch's backward (reference ``:740-756``: clears the extra buffer and
        queues the gradient transfer of the unit behind). Nothing to do: the fused accumulation pass
        clears the extra buffer itself and gradients stay on the GPU."""

    def pre_unit_backward(self, unit_index: int) -> Tensor:
        """Called before the backward pass of ``unit_index`` (units run from last to first).
        Returns the zeroed buffer backward must write the unit's gradients into: the accumulation
        buffer itself (backward accumulates over micro-batches), or -- when accumulation happens in
        a wider type -- the buffer for one micro-batch's gradients."""
        if self._pending_steps:
            raise RuntimeError("the previous iteration's forward shares have not been applied: run the forward-side hooks "
                               "(warmup_forward_pipeline, pre_unit_forward, post_micro_batch_forward) for every unit first")
        self._begin_iteration_statistics()
        self._rotate_buffers()
        if self._offload:
            # The buffer that now receives gradients fed a step enqueued earlier (of unit_index + 2,
            # or of this unit's forward share in the forward pass); its kernels must have read it
            # before backward overwrites it. A wait on the device, not the host.
            self._optimizer.cpu_optimizer.stream_wait()
        self._caller_follows_steps()  # the same, for the steps on the coordinator's own stream
        if self._has_fwd:
            self._bwd_unit = unit_index
        if self._has_bwd:
            self._plan_optimizer_steps(unit_index + 1, BACKWARD)
            self._open_unit_window(unit_index, BACKWARD)  # prefetch for the steps that start one unit from now
        receive = self._gpu_bwd_receive_grads
        receive.zero_()
        return self._gpu_bwd_extra_grads if self._gradacc_dtype_incompatible else receive

    def post_micro_batch_backward(self, unit_or_task, micro_batch_index: Optional[int] = None) -> None:
        """Called after each micro-batch's backward of a unit: folds the micro-batch's gradients into
        the accumulation buffer when the two differ in type (the last micro-batch's pass also yields
        the unit's overflow statistics), then steps the same part of the backward share of the unit
        that finished before it -- or, with no backward share, only gathers the finished unit's
        statistics."""
        unit_index, micro_batch_index = _unpack_task(unit_or_task, micro_batch_index)
        last = micro_batch_index == self._micro_batch_per_rank - 1
        if self._gradacc_dtype_incompatible:
            self._guard.accumulate(self._gpu_bwd_receive_grads, self._gpu_bwd_extra_grads, zero_grads=True,
                                   with_stats=self._guarded and last, loss_scale=self.loss_scale)
        if not self._has_bwd:
            if last:
                self._gather_unit_statistics(self._unit_grads[unit_index])
            return
        self._execute_optimizer_step(unit_index + 1, micro_batch_index, BACKWARD)

    def clear_backward_pipeline(self):
        """After the first unit's backward: step that unit's backward share and wait for everything
        in flight; with nothing but forward shares, take the iteration's one global decision (skip,
        clip coefficient) on the device. Forward shares follow in the next forward pass. Returns
        the iteration's ``GuardDecision`` (None when neither overflow checking nor clipping is on)
        after handing its overflow flag to the loss scaler."""
        if self._has_bwd:
            self._rotate_buffers()
            self._plan_optimizer_steps(0, BACKWARD, execute_now=True)
        if self._defer and self._guarded:
            self._iter_guard.decide_async(loss_scale=self.loss_scale, max_grad_norm=self._max_grad_norm,
                                          out=self._unit_controls[self._num_units])
        if self._has_fwd:
            self._deferred_grad_mult = float(1.0 / self.loss_scale)
        decision = self._finish_iteration_statistics()
        if self._has_fwd:
            self._pending_steps = True
            self._deferred_skip = bool(self._defer and decision is not None and decision.overflow)
        if self._has_bwd:
            self.synchronize()
        return decision

    # ---- hooks of the training loop: forward -----------------------------------------------------
    def warmup_forward_pipeline(self) -> None:
        """Before the forward pass of the first unit (reference ``:825-847``): its parameters must be
        the updated ones, so its whole forward share is enqueued now; the second unit's state starts
        on its way to the GPU. No-op unless forward shares are waiting to be stepped. With
        ``defer_to_forward`` the caller advances the groups' step counters (``update_states``)
        before this call when the decision was not an overflow."""
        if not self._pending_steps:
            return
        self._plan_optimizer_steps(0, FORWARD, execute_now=True)
        self._open_unit_window(1, FORWARD)
        self._fwd_guard_parameters()
        if self._num_units == 1:
            self._finish_deferred_steps()

    def pre_micro_batch_forward(self, unit_or_task, micro_batch_index: Optional[int] = None) -> None:
        """Before each micro-batch's forward (reference ``:733-738``: returns at once). Nothing to do."""

    def pre_unit_forward(self, unit_index: int) -> None:
        """Before the forward pass of ``unit_index`` (reference ``:784-794``): bind the forward-share
        step contexts of the next unit and start prefetching the state of the one after it."""
        if not self._pending_steps:
            return
        self._plan_optimizer_steps(unit_index + 1, FORWARD)
        self._open_unit_window(unit_index + 2, FORWARD)

    def post_micro_batch_forward(self, unit_or_task, micro_batch_index: Optional[int] = None) -> None:
        """After each micro-batch's forward of a unit (reference ``:758-769``): step the same part of
        the next unit's forward share; after the last part the next unit's forward may read its new
        parameters."""
        if not self._pending_steps:
            return
        unit_index, micro_batch_index = _unpack_task(unit_or_task, micro_batch_index)
        self._execute_optimizer_step(unit_index + 1, micro_batch_index, FORWARD)
        if micro_batch_index == self._micro_batch_per_rank - 1:
            self._fwd_guard_parameters()
            if unit_index + 1 >= self._num_units - 1:
                self._finish_deferred_steps()

    def _fwd_guard_parameters(self) -> None:
        """The forward pass that follows on the caller's stream reads the low-precision parameters the
        step's kernels (on the offload engine's stream, or on the step stream) have just written."""
        if self._offload and not self._deferred_skip:
            self._optimizer.cpu_optimizer.stream_wait()
        self._caller_follows_steps()

    def _finish_deferred_steps(self) -> None:
        self._pending_steps = False
        self._deferred_skip = False

    def synchronize(self) -> None:
        if self._offload:
            self._optimizer.cpu_optimizer.stream_wait()
            self._optimizer.cpu_optimizer.synchronize()
        if self._step_stream is not None:
            self._step_stream.synchronize()
        if any(self._unit_resident):
            torch.cuda.current_stream().synchronize()

    # ---- state files ---------------------------------------------------------------------------
    def _open_window_units(self) -> List[int]:
        return sorted(set(self._fwd.open_windows) | set(self._bwd.open_windows))

    def save_optimizer_states(self, directory: str, *, rank: int = 0, checkpoint_interval: int = 1,
                              fsync: bool = False) -> List[str]:
        """Writes every unit's ``[master | exp_avg | exp_avg_sq]`` blocks as the reference's swap files:
        ``rank{r}_OPTS_layer{i}.swp.0`` for the forward share, ``.swp.1`` for the backward share, no
        file for a share without elements. Waits for the steps in flight first. Returns the paths."""
        from .state_files import BACKWARD_SHARE, FORWARD_SHARE, write_unit_opts
        if self._pending_steps:
            raise RuntimeError("a decided iteration has not been applied yet; save after the forward-side hooks have run")
        if self._open_window_units():
            raise RuntimeError("units %s are being stepped on the GPU; save after clear_backward_pipeline()" % self._open_window_units())
        self.synchronize()
        paths = []
        for u in range(self._num_units):
            for s in self._shares():
                blocks = [b.cpu() for b in s.opts[u]] if self._unit_resident[u] else s.opts[u]
                paths.append(write_unit_opts(directory, u, blocks, share=FORWARD_SHARE if s.forward else BACKWARD_SHARE,
                                             rank=rank, checkpoint_interval=checkpoint_interval, fsync=fsync))
        return paths

    def load_optimizer_states(self, directory: str, *, rank: int = 0, checkpoint_interval: int = 1) -> None:
        """Reads the files ``save_optimizer_states`` wrote back into the units' blocks and rounds
        the master parameters into the units' low-precision parameters (what the update's copy-out
        would have left there). Group step counters are the caller's to restore."""
        from .state_files import BACKWARD_SHARE, FORWARD_SHARE, read_unit_opts
        if self._open_window_units():
            raise RuntimeError("units %s are being stepped on the GPU; load after clear_backward_pipeline()" % self._open_window_units())
        self.synchronize()
        for u in range(self._num_units):
            for s in self._shares():
                share = FORWARD_SHARE if s.forward else BACKWARD_SHARE
                if not self._unit_resident[u]:
                    read_unit_opts(directory, u, s.opts[u], share=share, rank=rank, checkpoint_interval=checkpoint_interval)
                else:
                    staging = [torch.empty(b.shape, dtype=b.dtype) for b in s.opts[u]]
                    read_unit_opts(directory, u, staging, share=share, rank=rank, checkpoint_interval=checkpoint_interval)
                    for dst, src in zip(s.opts[u], staging):
                        dst.copy_(src)
            self._copy_master_to_or_from_half(u, to_half=True)
        torch.cuda.current_stream().synchronize()


_OPTS_COORDINATOR = FlexTrainOptsCoordinator()


def get_opts_coordinator() -> FlexTrainOptsCoordinator:
    """Process-wide coordinator (reference ``:891-901``)."""
    return _OPTS_COORDINATOR
