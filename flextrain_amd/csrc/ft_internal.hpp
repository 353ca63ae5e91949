// ft_internal.hpp -- helpers shared by the translation units of libftadam.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "ft_adam.h"
#include "ft_types.hpp"

namespace fth {

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define FT_HIP(call)                                                                      \
    do {                                                                                  \
        hipError_t _e = (call);                                                           \
        if (_e != hipSuccess)                                                             \
            return ::fth::fail(FT_EHIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(_e), \
                               __FILE__, __LINE__);                                       \
    } while (0)

struct AdamObject {
    float lr, beta1, beta2, eps, weight_decay;
    bool adamw_mode;
};

// Looks the optimizer up; returns FT_ENOENT if absent.
int find_adam(int id, AdamObject* out);

// Host scalars of one step (cpu_adam.h:67-102,148-166 of the reference).
ftk::AdamConsts make_consts(uint64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                            bool bias_correction, bool adamw_mode, float grad_mult);

// Validates and launches the update over n elements on `stream` (device of the current context).
// p_out/m_out/v_out: where the new values are written; nullptr = in place.
int launch_adam(const ftk::AdamConsts& c, float* p, const void* g, int g_dtype, float* m, float* v,
                void* half_out, int half_dtype, size_t n, const ft_step_control_t* ctl, hipStream_t stream,
                float* p_out = nullptr, float* m_out = nullptr, float* v_out = nullptr,
                const ftk::AdamConsts* hyper = nullptr);  // hyper: the scalars in device memory (they replace c)

// Elements of a segment that go in front of its vector body (see the definition).
size_t segment_head(const void* p, size_t n);

// One launch of the many-segment update kernel over the table in `a` (see ft_types.hpp).
int launch_adam_multi(const ftk::AdamMultiArgs& a, int g_dtype, bool with_half, int half_dtype, bool with_hyper,
                      unsigned workgroups, hipStream_t stream);

int cu_count();  // compute units of the current device (cached)

// Dynamic LDS per 64-lane workgroup that keeps the bytes in flight per CU at the tuned level for a
// kernel whose lanes each have `load_bytes_per_lane` bytes of loads outstanding.
// `percent` scales the resulting number of resident wavefronts (a measured correction for a kernel
// whose stores weigh differently).
unsigned throttle_lds_bytes(unsigned load_bytes_per_lane, unsigned percent = 100);

}  // namespace fth
