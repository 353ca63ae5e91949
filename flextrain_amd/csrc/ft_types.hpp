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
    uint64_t n;                    // elements (scalar kernel) or 4-element units (vector kernel)
    AdamConsts c;
};

}  // namespace ftk
