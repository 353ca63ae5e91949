"""MI355X-native optimizer step for FlexTrain-style training.

Fused unscale / clip / Adam(W) / low-precision recast kernels for gfx950 behind the reference's
optimizer interface, plus the chunked pinned-host <-> HBM pipeline for offloaded state.
Importing the package does not touch the GPU; the native library is loaded on first use and its
absence is an error (there is no CPU fallback).
"""
from .adam import FlexTrainAdam, FlexTrainCPUAdam
from .optimizer import PARAMS_KEY, STEP_KEY, FlexTrainCPUOptimizer, FlexTrainOptimizer
from .param_group import GroupSegment, StepContext, StepContextContainer

__all__ = [
    "FlexTrainAdam", "FlexTrainCPUAdam", "FlexTrainCPUOptimizer", "FlexTrainOptimizer",
    "GroupSegment", "StepContext", "StepContextContainer", "STEP_KEY", "PARAMS_KEY",
]
