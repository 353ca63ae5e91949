// ft_types.hpp -- plain structs passed from the host launchers to the kernels.
#pragma once

#include <stdint.h>

#include "ft_adam.h"

namespace ftk {

// Scalars of one step, computed on the host exactly as the reference does
// (cpu_adam.h:67-102,148-166) and passed by value so host and device agree bit for bit.
struct AdamConsts {
    float beta1, beta2, omb1, omb2;
    float bias2, eps, step_size, wd_coef;
    float grad_mult;
    int wd_mode;  // 0 none, 1 AdamW (decoupled), 2 Adam (L2 folded into g)
};

struct AdamArgs {
    const float* p;  // inputs ...
    const void* g;
    const float* m;
    const float* v;
    float* p_out;    // ... and where the new values go (the same arrays for an in-place update)
    float* m_out;
    float* v_out;
    void* h;                       // low-precision copy or nullptr
    const ft_step_control_t* ctl;  // device decision or nullptr
    const AdamConsts* hyper;       // the scalars in device memory (they replace c), or nullptr
    uint64_t n;                    // elements (scalar kernel) or 4-element units (vector kernel)
    AdamConsts c;
};

// ---- many segments in one launch -------------------------------------------------------------
// One contiguous piece of an in-place update with its own hyper-parameters: what the reference
// hands to one adam_update call per StepContext (flextrain/optimizer.py:44-69).
constexpr int kMultiMaxSegments = 16;

struct AdamSegment {
    float* p;
    const void* g;
    float* m;
    float* v;
    void* h;              // low-precision copy of this segment, or nullptr for every segment of a launch
    uint64_t n;           // elements
    uint32_t head;        // elements in front of the first tile (they reach the alignment the tiles want)
    uint32_t body_tiles;  // whole 256-element tiles behind the head
    const AdamConsts* hyper;  // the scalars in device memory (they replace c), or nullptr
    AdamConsts c;
};

// The HIP runtime refuses a launch whose gridDim.x * blockDim.x exceeds 2^32 - 1 work-items
// (hipErrorInvalidConfiguration), so a grid of 64-lane workgroups holds at most (2^32 - 1) / 64 of
// them; whatever needs more is cut into several launches (plan_launch_pieces in ft_launch_plan.hpp).
constexpr uint64_t kMaxThreadsPerLaunch = 0xffffffffull;
constexpr uint64_t kMaxWorkgroupsPerLaunch = kMaxThreadsPerLaunch / 64;  // 67,108,863 workgroups of one wavefront

// The whole table travels in the kernel-argument segment (1.6 KB): no device allocation, no upload.
// first_wg[s] = (number of workgroups that belong to the segments before s) << 4 | s; unused
// entries hold 0xffffffff: the encoding leaves room for 2^28 - 1 workgroups, the runtime's limit on a
// launch for fewer.
constexpr uint64_t kMultiEncodingWorkgroups = (1ull << 28) - 1;
constexpr uint64_t kMultiMaxWorkgroups =
    kMultiEncodingWorkgroups < kMaxWorkgroupsPerLaunch ? kMultiEncodingWorkgroups : kMaxWorkgroupsPerLaunch;
struct AdamMultiArgs {
    uint32_t first_wg[kMultiMaxSegments];
    const ft_step_control_t* ctl;
    AdamSegment seg[kMultiMaxSegments];
};

}  // namespace ftk
