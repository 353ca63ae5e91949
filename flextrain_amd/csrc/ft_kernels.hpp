// ft_kernels.hpp -- gfx950 device code of the optimizer-step hot path.
//
// Two kernels carry the traffic:
//   adam_tile_kernel   fused unscale/clip multiply + Adam/AdamW + low-precision recast. One pass:
//                     reads p, m, v (fp32) and g (fp32/fp16/bf16), writes p, m, v and optionally
//                     the 16-bit copy. HBM-bound: 28 bytes per element with 16-bit g and copy.
//   grad_stats_kernel one read of g: inf/nan count and sum of squares (2 or 4 bytes per element).
//
// Arithmetic contract of adam_element(): one IEEE-754 round-to-nearest fp32 operation per
// statement, in the order of the reference's vector loop
// (flextrain/ops/csrc/includes/cpu_adam.h:188-205). The translation unit must be compiled with
// -ffp-contract=off; fused multiply-adds appear only where written as __builtin_fmaf. Division
// and square root are the correctly rounded expansions hipcc emits by default.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "ft_adam.h"
#include "ft_types.hpp"

namespace ftk {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

__device__ __forceinline__ void adam_element(float& p, float g, float& m, float& v, const AdamConsts& c)
{
    g = g * c.grad_mult;
    if (c.wd_mode == 2) g = __builtin_fmaf(p, c.wd_coef, g);
    float mi = m * c.beta1;
    mi = __builtin_fmaf(g, c.omb1, mi);
    float vi = v * c.beta2;
    const float g2 = g * g;
    vi = __builtin_fmaf(g2, c.omb2, vi);
    float d = __builtin_sqrtf(vi);
    d = __builtin_fmaf(d, c.bias2, c.eps);
    const float u = mi / d;
    float pi = p;
    if (c.wd_mode == 1) pi = __builtin_fmaf(pi, c.wd_coef, pi);
    pi = __builtin_fmaf(u, c.step_size, pi);
    // The new value is materialised in a register before any narrowing conversion, so that the
    // 16-bit copy is the rounding of the stored fp32 value and never a mixed-precision fma.
    asm volatile("" : "+v"(pi));
    p = pi;
    m = mi;
    v = vi;
}

// Four consecutive elements held in vector registers.
__device__ __forceinline__ void adam_unit(f32x4& p, const f32x4& g, f32x4& m, f32x4& v, const AdamConsts& c)
{
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float pk = p[k], mk = m[k], vk = v[k];
        adam_element(pk, g[k], mk, vk, c);
        p[k] = pk;
        m[k] = mk;
        v[k] = vk;
    }
}

// ---- 16-bit <-> 32-bit helpers ------------------------------------------------------------
template <int DT>
__device__ __forceinline__ float half_to_float(uint32_t bits16);
template <>
__device__ __forceinline__ float half_to_float<FT_BF16>(uint32_t b)
{
    return __builtin_bit_cast(float, b << 16);
}
template <>
__device__ __forceinline__ float half_to_float<FT_F16>(uint32_t b)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<FT_BF16>(float lo, float hi)
{
    f32x2 x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
}
template <>
__device__ __forceinline__ uint32_t pack2<FT_F16>(float lo, float hi)
{
    f32x2 x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
}

template <bool NT, typename T>
__device__ __forceinline__ T ld(const T* p)
{
    if constexpr (NT)
        return __builtin_nontemporal_load(p);
    else
        return *p;
}
template <bool NT, typename T>
__device__ __forceinline__ void st(T* p, T x)
{
    if constexpr (NT)
        __builtin_nontemporal_store(x, p);
    else
        *p = x;
}

// Streaming stores of a whole tile go through buffer instructions, because those let the cache
// policy be chosen: `nt` (what a non-temporal global store sets) plus agent scope `sc1`, which
// makes the L2 write the line through instead of holding it dirty. Measured on the update kernel
// at 2e8 elements: 0.827 ms against 0.842 ms with `nt` alone (`sc0 sc1 nt` the same; no policy on
// the loads made a difference). The descriptor covers exactly one array's share of the tile
// (base = wave-uniform tile start, num_records = its bytes), so the hardware also drops any store
// that would fall outside it.
constexpr int kAuxStreamStore = 18;  // bit 1: nt, bit 4: sc1
constexpr int kRawBufferFlags = 0x00027000;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(void* tile_base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(tile_base, 0, (int)bytes, kRawBufferFlags);
}
__device__ __forceinline__ void st_stream(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, f32x4 x)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, x), r, (int)byte_offset, 0, kAuxStreamStore);
}
__device__ __forceinline__ void st_stream(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, u32x2 x)
{
    __builtin_amdgcn_raw_buffer_store_b64(x, r, (int)byte_offset, 0, kAuxStreamStore);
}

// The same stores with the default cache policy: for the part of an array that its next reader
// should find in the memory-side cache.
__device__ __forceinline__ void st_keep(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, f32x4 x)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, x), r, (int)byte_offset, 0, 0);
}
__device__ __forceinline__ void st_keep(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, u32x2 x)
{
    __builtin_amdgcn_raw_buffer_store_b64(x, r, (int)byte_offset, 0, 0);
}

// Gradient unit = 4 consecutive elements.
template <int GT, bool NT>
__device__ __forceinline__ f32x4 load_g4(const void* g, uint64_t unit)
{
    if constexpr (GT == FT_F32) {
        return ld<NT>(reinterpret_cast<const f32x4*>(g) + unit);
    } else {
        const u32x2 w = ld<NT>(reinterpret_cast<const u32x2*>(g) + unit);
        f32x4 r;
        r.x = half_to_float<GT>(w.x & 0xffffu);
        r.y = half_to_float<GT>(w.x >> 16);
        r.z = half_to_float<GT>(w.y & 0xffffu);
        r.w = half_to_float<GT>(w.y >> 16);
        return r;
    }
}

// The update over whole tiles. One 64-lane workgroup per tile of 64 units (256 elements), one unit
// per lane, straight-line code: the host launches exactly one workgroup per full tile (tile0 lets
// it split a grid that would overflow) and sends the remainder through the scalar kernel, so there
// is no bounds check and no loop.
// Inputs and outputs are the same arrays for an in-place update; the offloaded step may point the
// outputs elsewhere (staging buffer -> host memory, or the reverse), hence no __restrict__.
// HT == -1: no low-precision copy. HAS_CTL: a.ctl is read first; a skipped in-place step touches
// nothing else (measured: looking at the decision before or after issuing the vector loads makes no
// difference to a normal step, 0.835 against 0.833 ms; a skipped step costs 0.17 ms of workgroup
// dispatch the first way and 0.40 ms the second). The low-precision copy is never written on a
// skip: it has no input to copy from, so a caller that skips must not stage it.
// HAS_HYPER: the step's scalars come from a.hyper (device memory, wave-uniform scalar loads) instead
// of by value. A variant of its own rather than a test of the pointer: a branch in front of the
// loads of the decision record and of the tile costs the common by-value path a dependent round of
// scalar loads (and anything that looks like a memory write before them, even an empty asm
// statement, turns the decision's scalar loads into vector loads: 0.81 -> 0.91 ms on the
// mixed-precision step).
template <int GT, int HT, bool HAS_CTL, bool HAS_HYPER>
__global__ __launch_bounds__(kWave) void adam_tile_kernel(AdamArgs a, uint64_t tile0)
{
    AdamConsts c;
    if constexpr (HAS_HYPER)
        c = *a.hyper;
    else
        c = a.c;
    const uint64_t t0 = (tile0 + blockIdx.x) * kWave;  // first unit of the tile: wave-uniform
    const uint64_t i = t0 + threadIdx.x;
    if constexpr (HAS_CTL) {  // wave-uniform scalar loads: one decision per step
        if (a.ctl->skip) {
            // A skipped step leaves the state as it is. Where the outputs are other arrays than
            // the inputs (a staging buffer on one side of the host link) "as it is" still has to
            // arrive there: whatever is copied onwards from the outputs must be the old state.
            if (a.p_out != a.p) st_stream(tile_rsrc(reinterpret_cast<f32x4*>(a.p_out) + t0, kWave * 16), threadIdx.x * 16,
                                          ld<true>(reinterpret_cast<const f32x4*>(a.p) + i));
            if (a.m_out != a.m) st_stream(tile_rsrc(reinterpret_cast<f32x4*>(a.m_out) + t0, kWave * 16), threadIdx.x * 16,
                                          ld<true>(reinterpret_cast<const f32x4*>(a.m) + i));
            if (a.v_out != a.v) st_stream(tile_rsrc(reinterpret_cast<f32x4*>(a.v_out) + t0, kWave * 16), threadIdx.x * 16,
                                          ld<true>(reinterpret_cast<const f32x4*>(a.v) + i));
            return;
        }
        c.grad_mult = a.ctl->grad_mult;
    }
    f32x4 g = load_g4<GT, true>(a.g, i);
    f32x4 p = ld<true>(reinterpret_cast<const f32x4*>(a.p) + i);
    f32x4 m = ld<true>(reinterpret_cast<const f32x4*>(a.m) + i);
    f32x4 v = ld<true>(reinterpret_cast<const f32x4*>(a.v) + i);
    adam_unit(p, g, m, v, c);
    const __amdgpu_buffer_rsrc_t rp = tile_rsrc(reinterpret_cast<f32x4*>(a.p_out) + t0, kWave * 16),
                                 rm = tile_rsrc(reinterpret_cast<f32x4*>(a.m_out) + t0, kWave * 16),
                                 rv = tile_rsrc(reinterpret_cast<f32x4*>(a.v_out) + t0, kWave * 16);
    st_stream(rp, threadIdx.x * 16, p);
    st_stream(rm, threadIdx.x * 16, m);
    st_stream(rv, threadIdx.x * 16, v);
    if constexpr (HT == FT_F16 || HT == FT_BF16) {
        const __amdgpu_buffer_rsrc_t rh = tile_rsrc(reinterpret_cast<u32x2*>(a.h) + t0, kWave * 8);
        u32x2 w;
        w.x = pack2<HT>(p.x, p.y);
        w.y = pack2<HT>(p.z, p.w);
        st_stream(rh, threadIdx.x * 8, w);
    }
}

// The update over whole tiles for arrays whose alignments disagree (a 16-bit copy cut at an odd
// element, a state array one element off): the same tile shape, but every array is accessed through
// vector types that promise only the alignment of one element, so the compiler emits whatever the
// hardware takes at that alignment (whole 16-byte accesses at dword alignment, split ones below it).
// An array whose tiles start inside a cache line shares a line with the neighbouring tile at either
// end; the template parameter CACHED and `flags` say how each array is treated so that this costs
// as little as it can (what the host chooses, and why, is at its call site; all of it is measured,
// none of it changes a result):
// * kRelaxedOnLines bits (p_out, m_out, v_out, h): the output's tiles do start on lines and it is
//   stored like the aligned kernel's (write-through streaming stores); the others get non-temporal
//   stores that the L2 may hold until the neighbouring tile has filled the line;
// * CACHED == 1: one of p, m, v (which: kRelaxedCachedShift) is read with the default cache policy,
//   so that the second reader of a shared line finds it in a cache, instead of streaming;
//   CACHED == 2: the gradient is. Variants of their own whose loads are always the same
//   instructions (for the state arrays with the pointers chosen by scalar selects): a run-time
//   choice of the load instruction per array made the compiler wait for each load before issuing the
//   next (0.93 ms instead of 0.84), and the same global load with and without the streaming hint in
//   two branches gets merged into one without it (hence buffer loads for the cached kind);
// * kRelaxedCopyCached: the 16-bit copy, off the lines, is stored with the default cache policy;
// * kRelaxedRuns: workgroups go to the eight dies in turn and each die has an L2 of its own, so
//   inside every group of 64 workgroups, workgroup r takes tile (r mod 8) * 8 + r / 8 of the group:
//   eight consecutive tiles run on one die back to back, and seven of eight shared edge lines are
//   completed (loads: found) in one L2. Workgroups behind the last whole group take their own index.
// The scalars may come from a.hyper.
typedef float f32x4_e __attribute__((ext_vector_type(4), aligned(4)));
typedef uint16_t u16x4_e __attribute__((ext_vector_type(4), aligned(2)));
constexpr uint32_t kRelaxedRun = 8;                 // consecutive tiles per die
constexpr uint32_t kRelaxedGroup = 8 * kRelaxedRun;  // workgroups permuted among themselves
constexpr uint32_t kRelaxedOnLinesP = 1u, kRelaxedOnLinesM = 2u, kRelaxedOnLinesV = 4u, kRelaxedOnLinesH = 8u;
constexpr uint32_t kRelaxedCachedShift = 4;  // bits 4-5, CACHED == 1 only: 0 p, 1 m, 2 v
constexpr uint32_t kRelaxedCopyCached = 1u << 6;
constexpr uint32_t kRelaxedRuns = 1u << 31;

__device__ __forceinline__ uint32_t relaxed_tile_of_workgroup(uint32_t b, uint32_t workgroups)
{
    if (b >= (workgroups & ~(kRelaxedGroup - 1))) return b;
    const uint32_t r = b & (kRelaxedGroup - 1);
    return (b & ~(kRelaxedGroup - 1)) + (r & 7u) * kRelaxedRun + (r >> 3);
}

template <int GT, int HT, bool HAS_CTL, int CACHED>
__global__ __launch_bounds__(kWave) void adam_tile_relaxed_kernel(AdamArgs a, uint64_t tile0, uint32_t flags)
{
    AdamConsts c = a.c;
    if (a.hyper) c = *a.hyper;
    const uint32_t tile = (flags & kRelaxedRuns) ? relaxed_tile_of_workgroup(blockIdx.x, gridDim.x) : blockIdx.x;
    const uint64_t t0 = (tile0 + tile) * kWave;  // first unit of the tile
    const uint64_t i = t0 + threadIdx.x;         // this lane's 4-element unit
    auto store_state = [&](float* out, f32x4 x, uint32_t on_lines) {
        if (flags & on_lines)  // wave-uniform
            st_stream(tile_rsrc(reinterpret_cast<f32x4*>(out) + t0, kWave * 16), threadIdx.x * 16, x);
        else
            __builtin_nontemporal_store(static_cast<f32x4_e>(x), reinterpret_cast<f32x4_e*>(out) + i);
    };
    if constexpr (HAS_CTL) {
        if (a.ctl->skip) {
            // A skipped step leaves the state as it is; where the outputs are other arrays than the
            // inputs (a staging buffer on one side of the host link) the old state still has to
            // arrive there. The low-precision copy is never written on a skip.
            if (a.p_out != a.p) store_state(a.p_out, __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.p) + i), kRelaxedOnLinesP);
            if (a.m_out != a.m) store_state(a.m_out, __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.m) + i), kRelaxedOnLinesM);
            if (a.v_out != a.v) store_state(a.v_out, __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.v) + i), kRelaxedOnLinesV);
            return;
        }
        c.grad_mult = a.ctl->grad_mult;
    }
    // Straight-line from here: the gradient unit and the three state units are fetched before
    // anything waits for one of them.
    f32x4 g;
    if constexpr (GT == FT_F32) {
        if constexpr (CACHED == 2) {
            const __amdgpu_buffer_rsrc_t r =
                tile_rsrc(const_cast<f32x4_e*>(reinterpret_cast<const f32x4_e*>(a.g)) + t0, kWave * 16);
            g = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(threadIdx.x * 16), 0, 0));
        } else {
            g = __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.g) + i);
        }
    } else {
        u16x4_e w;
        if constexpr (CACHED == 2) {
            const __amdgpu_buffer_rsrc_t r =
                tile_rsrc(const_cast<u16x4_e*>(reinterpret_cast<const u16x4_e*>(a.g)) + t0, kWave * 8);
            w = __builtin_bit_cast(u16x4_e, __builtin_amdgcn_raw_buffer_load_b64(r, (int)(threadIdx.x * 8), 0, 0));
        } else {
            w = __builtin_nontemporal_load(reinterpret_cast<const u16x4_e*>(a.g) + i);
        }
        g.x = half_to_float<GT>(w.x);
        g.y = half_to_float<GT>(w.y);
        g.z = half_to_float<GT>(w.z);
        g.w = half_to_float<GT>(w.w);
    }
    f32x4 p, m, v;
    if constexpr (CACHED == 1) {
        const uint32_t k = (flags >> kRelaxedCachedShift) & 3u;  // wave-uniform
        const float* odd = k == 0 ? a.p : k == 1 ? a.m : a.v;
        const float* first = k == 0 ? a.m : a.p;  // the other two, in order
        const float* second = k == 2 ? a.m : a.v;
        const __amdgpu_buffer_rsrc_t r =
            tile_rsrc(const_cast<f32x4_e*>(reinterpret_cast<const f32x4_e*>(odd)) + t0, kWave * 16);
        const f32x4 xo = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(threadIdx.x * 16), 0, 0));
        const f32x4 x1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(first) + i);
        const f32x4 x2 = __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(second) + i);
        p = k == 0 ? xo : x1;
        m = k == 0 ? x1 : (k == 1 ? xo : x2);
        v = k == 2 ? xo : x2;
    } else {
        p = __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.p) + i);
        m = __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.m) + i);
        v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_e*>(a.v) + i);
    }
    adam_unit(p, g, m, v, c);
    store_state(a.p_out, p, kRelaxedOnLinesP);
    store_state(a.m_out, m, kRelaxedOnLinesM);
    store_state(a.v_out, v, kRelaxedOnLinesV);
    if constexpr (HT == FT_F16 || HT == FT_BF16) {
        const uint32_t lo = pack2<HT>(p.x, p.y), hi = pack2<HT>(p.z, p.w);
        u32x2 w2;
        w2.x = lo;
        w2.y = hi;
        if (flags & kRelaxedOnLinesH) {
            st_stream(tile_rsrc(reinterpret_cast<u32x2*>(a.h) + t0, kWave * 8), threadIdx.x * 8, w2);
        } else if (flags & kRelaxedCopyCached) {
            st_keep(tile_rsrc(reinterpret_cast<u16x4_e*>(a.h) + t0, kWave * 8), threadIdx.x * 8, w2);
        } else {
            u16x4_e w;
            w.x = (uint16_t)(lo & 0xffffu);
            w.y = (uint16_t)(lo >> 16);
            w.z = (uint16_t)(hi & 0xffffu);
            w.w = (uint16_t)(hi >> 16);
            __builtin_nontemporal_store(w, reinterpret_cast<u16x4_e*>(a.h) + i);
        }
    }
}

// Element-at-a-time kernel for heads, tails and arrays whose alignments disagree. a.n counts
// elements. Same arithmetic, so the result of an element never depends on which kernel took it.
template <int GT, int HT>
__global__ __launch_bounds__(256) void adam_scalar_kernel(AdamArgs a)
{
    AdamConsts c = a.c;
    if (a.hyper) c = *a.hyper;
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    if (a.ctl) {
        if (a.ctl->skip) {  // out of place: the old state still has to reach the outputs
            if (a.p_out != a.p || a.m_out != a.m || a.v_out != a.v)
                for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += stride) {
                    a.p_out[i] = a.p[i];
                    a.m_out[i] = a.m[i];
                    a.v_out[i] = a.v[i];
                }
            return;
        }
        c.grad_mult = a.ctl->grad_mult;
    }
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += stride) {
        float g;
        if constexpr (GT == FT_F32)
            g = reinterpret_cast<const float*>(a.g)[i];
        else
            g = half_to_float<GT>(reinterpret_cast<const uint16_t*>(a.g)[i]);
        float p = a.p[i], m = a.m[i], v = a.v[i];
        adam_element(p, g, m, v, c);
        a.p_out[i] = p;
        a.m_out[i] = m;
        a.v_out[i] = v;
        if constexpr (HT == FT_F16 || HT == FT_BF16)
            reinterpret_cast<uint16_t*>(a.h)[i] = (uint16_t)(pack2<HT>(p, 0.0f) & 0xffffu);
    }
}

// Many segments, one launch: the per-(unit, micro-batch) loop of the reference steps one StepContext
// after the other (flextrain/optimizer.py:44-69), dozens of short calls per unit; here up to
// kMultiMaxSegments of them, each with its own pointers, length and hyper-parameters, are one grid.
// Workgroup w belongs to the segment s whose first workgroup is the last one not after w (a scalar
// compare chain over the table in the kernel-argument segment, then one scalar load of the
// segment's record from there: no table in device memory). Inside a segment, workgroup
// k < body_tiles is a full 256-element tile behind the segment's head and runs the straight-line
// code of adam_tile_kernel; the one workgroup after them takes the segment's edge elements (the
// head in front of the first tile, up to 255 elements behind the last whole tile) one element per
// lane and round, through the same adam_element. In place only.
typedef const char __attribute__((address_space(4))) * KernargBytes;

template <int GT, int HT, bool HAS_CTL, bool HAS_HYPER>
__global__ __launch_bounds__(kWave) void adam_multi_kernel(AdamMultiArgs a)
{
    // Table entry k = (first workgroup of segment k) << 4 | k, ascending, unused entries all ones:
    // the largest entry that does not exceed (my workgroup << 4 | 15) names my segment and where
    // it starts, at one scalar compare and one scalar select per entry.
    const uint32_t wg = blockIdx.x;
    const uint32_t mine = (wg << 4) | 15u;
    uint32_t best = a.first_wg[0];
#pragma unroll
    for (int k = 1; k < kMultiMaxSegments; ++k) {
        const uint32_t f = a.first_wg[k];
        best = f <= mine ? f : best;
    }
    const uint32_t s = best & 15u, base = best >> 4;
    // The record is read through the kernel-argument pointer at a computed offset, so that the
    // dynamic index turns into an address and not into a private copy of the table.
    const KernargBytes ka = (KernargBytes)__builtin_amdgcn_kernarg_segment_ptr();
    typedef const AdamSegment __attribute__((address_space(4))) * SegPtr;
    const SegPtr sg = reinterpret_cast<SegPtr>(ka + __builtin_offsetof(AdamMultiArgs, seg) + s * sizeof(AdamSegment));
    AdamConsts c;
    if constexpr (HAS_HYPER) {  // every segment of the launch keeps its scalars in device memory
        c = *sg->hyper;
    } else {
        c.beta1 = sg->c.beta1;
        c.beta2 = sg->c.beta2;
        c.omb1 = sg->c.omb1;
        c.omb2 = sg->c.omb2;
        c.bias2 = sg->c.bias2;
        c.eps = sg->c.eps;
        c.step_size = sg->c.step_size;
        c.wd_coef = sg->c.wd_coef;
        c.grad_mult = sg->c.grad_mult;
        c.wd_mode = sg->c.wd_mode;
    }
    if constexpr (HAS_CTL) {
        if (a.ctl->skip) return;
        c.grad_mult = a.ctl->grad_mult;
    }
    const uint32_t local = wg - base;
    const uint32_t head = sg->head, body_tiles = sg->body_tiles;
    float* const p = sg->p;
    float* const m = sg->m;
    float* const v = sg->v;
    const char* const g = static_cast<const char*>(sg->g);
    char* const h = static_cast<char*>(sg->h);
    constexpr uint32_t gsz = (GT == FT_F32) ? 4 : 2;
    if (local < body_tiles) {
        const uint64_t t0 = (uint64_t)local * kWave;  // first unit of the tile behind the head
        const uint64_t i = t0 + threadIdx.x;
        f32x4 g4 = load_g4<GT, true>(g + (uint64_t)head * gsz, i);
        f32x4 p4 = ld<true>(reinterpret_cast<const f32x4*>(p + head) + i);
        f32x4 m4 = ld<true>(reinterpret_cast<const f32x4*>(m + head) + i);
        f32x4 v4 = ld<true>(reinterpret_cast<const f32x4*>(v + head) + i);
        adam_unit(p4, g4, m4, v4, c);
        const __amdgpu_buffer_rsrc_t rp = tile_rsrc(reinterpret_cast<f32x4*>(p + head) + t0, kWave * 16),
                                     rm = tile_rsrc(reinterpret_cast<f32x4*>(m + head) + t0, kWave * 16),
                                     rv = tile_rsrc(reinterpret_cast<f32x4*>(v + head) + t0, kWave * 16);
        st_stream(rp, threadIdx.x * 16, p4);
        st_stream(rm, threadIdx.x * 16, m4);
        st_stream(rv, threadIdx.x * 16, v4);
        if constexpr (HT == FT_F16 || HT == FT_BF16) {
            const __amdgpu_buffer_rsrc_t rh = tile_rsrc(reinterpret_cast<u32x2*>(h + (uint64_t)head * 2) + t0, kWave * 8);
            u32x2 w;
            w.x = pack2<HT>(p4.x, p4.y);
            w.y = pack2<HT>(p4.z, p4.w);
            st_stream(rh, threadIdx.x * 8, w);
        }
        return;
    }
    // edge workgroup of the segment
    const uint64_t n = sg->n;
    const uint64_t tail0 = head + (uint64_t)body_tiles * (kWave * 4);
    const uint32_t edge = head + (uint32_t)(n - tail0);
    for (uint32_t e = threadIdx.x; e < edge; e += kWave) {
        const uint64_t i = e < head ? e : tail0 + (e - head);
        float gi;
        if constexpr (GT == FT_F32)
            gi = reinterpret_cast<const float*>(g)[i];
        else
            gi = half_to_float<GT>(reinterpret_cast<const uint16_t*>(g)[i]);
        float pi = p[i], mi = m[i], vi = v[i];
        adam_element(pi, gi, mi, vi, c);
        p[i] = pi;
        m[i] = mi;
        v[i] = vi;
        if constexpr (HT == FT_F16 || HT == FT_BF16)
            reinterpret_cast<uint16_t*>(h)[i] = (uint16_t)(pack2<HT>(pi, 0.0f) & 0xffffu);
    }
}

// ---- reductions ----------------------------------------------------------------------------
// Sum across the 64 lanes of a wavefront with DPP lane permutes (no LDS): xor-1 and xor-2 inside
// each quad, then mirror inside half rows and rows; every lane of a 16-lane row then holds the
// row total, and the four row totals are read with v_readlane and added in a fixed order.
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t x)
{
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x140, 0xF, 0xF, false);
    return (uint32_t)__builtin_amdgcn_readlane((int)x, 0) + (uint32_t)__builtin_amdgcn_readlane((int)x, 16) +
           (uint32_t)__builtin_amdgcn_readlane((int)x, 32) + (uint32_t)__builtin_amdgcn_readlane((int)x, 48);
}

// The same reduction for doubles: the two halves of every value travel through the same lane
// permutes, the additions are fp64.
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double x)
{
    const uint64_t b = __builtin_bit_cast(uint64_t, x);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)b, CTRL, 0xF, 0xF, false);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(b >> 32), CTRL, 0xF, 0xF, false);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ double readlane_f64(double x, const int lane)
{
    const uint64_t b = __builtin_bit_cast(uint64_t, x);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), lane);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ double wave_sum_f64(double x)
{
    x += dpp_f64<0xB1>(x);   // quad_perm:[1,0,3,2]
    x += dpp_f64<0x4E>(x);   // quad_perm:[2,3,0,1]
    x += dpp_f64<0x141>(x);  // row_half_mirror
    x += dpp_f64<0x140>(x);  // row_mirror
    return (readlane_f64(x, 0) + readlane_f64(x, 16)) + (readlane_f64(x, 32) + readlane_f64(x, 48));
}

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t x)
{
    auto permuted = [](uint64_t v, auto ctrl) {
        return __builtin_bit_cast(uint64_t, dpp_f64<decltype(ctrl)::value>(__builtin_bit_cast(double, v)));
    };
    x += permuted(x, std::integral_constant<int, 0xB1>{});
    x += permuted(x, std::integral_constant<int, 0x4E>{});
    x += permuted(x, std::integral_constant<int, 0x141>{});
    x += permuted(x, std::integral_constant<int, 0x140>{});
    auto lane = [&](const int l) { return __builtin_bit_cast(uint64_t, readlane_f64(__builtin_bit_cast(double, x), l)); };
    return lane(0) + lane(16) + lane(32) + lane(48);
}

// x*x added to acc in fp64. The square of an fp32 value is exact in fp64 (24-bit significand), so
// the only rounding is the addition's, and no finite fp32 value can make the sum overflow or vanish:
// 3.4e38 squared is 1.2e77, 1.4e-45 squared 2e-90, both far inside the fp64 range.
__device__ __forceinline__ double add_square(float x, double acc)
{
    const double d = (double)x;
    return __builtin_fma(d, d, acc);
}

struct StatsPartial {
    double sumsq;
    uint64_t nonfinite;
};

// One 16-byte load = 8 sixteen-bit or 4 thirty-two-bit gradient elements. Exact path: every element
// is tested for inf/nan (exponent field all ones), counted if so, and squared in if not.
template <int GT>
__device__ __forceinline__ void stats_accumulate(u32x4 w, float pre_mult, double (&acc)[4], uint32_t& bad)
{
    if constexpr (GT == FT_F32) {
        const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const bool nf = (ws[k] & 0x7f800000u) == 0x7f800000u;
            const float x = __builtin_bit_cast(float, ws[k]) * pre_mult;
            bad += nf ? 1u : 0u;
            acc[k] = add_square(nf ? 0.0f : x, acc[k]);
        }
    } else {
        constexpr uint32_t kExp = (GT == FT_BF16) ? 0x7f80u : 0x7c00u;
        const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t lo = ws[k] & 0xffffu, hi = ws[k] >> 16;
            const bool nlo = (lo & kExp) == kExp, nhi = (hi & kExp) == kExp;
            const float xlo = half_to_float<GT>(lo) * pre_mult;
            const float xhi = half_to_float<GT>(hi) * pre_mult;
            bad += (nlo ? 1u : 0u) + (nhi ? 1u : 0u);
            acc[k] = add_square(nlo ? 0.0f : xlo, acc[k]);
            acc[k] = add_square(nhi ? 0.0f : xhi, acc[k]);
        }
    }
}

// Non-zero iff one of the elements of the load is inf or nan. For the 16-bit types both halves of a
// word are tested at once: adding one unit of the exponent field's lowest bit to the masked field
// carries into the sign position exactly when the field is all ones.
template <int GT>
__device__ __forceinline__ uint32_t nonfinite_marks(u32x4 w)
{
    constexpr uint32_t kField = (GT == FT_F32) ? 0x7f800000u : (GT == FT_BF16 ? 0x7f807f80u : 0x7c007c00u);
    constexpr uint32_t kUnit = (GT == FT_F32) ? 0x00800000u : (GT == FT_BF16 ? 0x00800080u : 0x04000400u);
    constexpr uint32_t kCarry = (GT == FT_F32) ? 0x80000000u : 0x80008000u;
    return ((((w.x & kField) + kUnit) | ((w.y & kField) + kUnit)) | (((w.z & kField) + kUnit) | ((w.w & kField) + kUnit))) & kCarry;
}

// The same sums for a load that is known to hold finite elements only: no test, no select.
template <int GT>
__device__ __forceinline__ void stats_accumulate_finite(u32x4 w, float pre_mult, double (&acc)[4])
{
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if constexpr (GT == FT_F32) {
            acc[k] = add_square(__builtin_bit_cast(float, ws[k]) * pre_mult, acc[k]);
        } else {
            acc[k] = add_square(half_to_float<GT>(ws[k] & 0xffffu) * pre_mult, acc[k]);
            acc[k] = add_square(half_to_float<GT>(ws[k] >> 16) * pre_mult, acc[k]);
        }
    }
}

// Block-level end of a statistics pass: per-lane fp64 sums and counts -> the block's totals: a
// wavefront sum each (DPP, fixed order), then the wavefronts' sums in order through LDS; valid in
// thread 0.
template <int BLOCK>
__device__ __forceinline__ void block_stats_reduce(double lane_sum, uint32_t bad, double& total, uint64_t& total_bad)
{
    __shared__ double s_sum[BLOCK / kWave];
    __shared__ uint32_t s_bad[BLOCK / kWave];
    const double ts = wave_sum_f64(lane_sum);
    const uint32_t tb = wave_sum_u32(bad);
    if ((threadIdx.x & (kWave - 1)) == 0) {
        s_sum[threadIdx.x / kWave] = ts;
        s_bad[threadIdx.x / kWave] = tb;
    }
    __syncthreads();
    total = 0.0;
    total_bad = 0;
    if (threadIdx.x == 0) {
        double t = s_sum[0];
        uint64_t b = s_bad[0];
#pragma unroll
        for (int k = 1; k < BLOCK / kWave; ++k) {
            t += s_sum[k];
            b += s_bad[k];
        }
        total = t;
        total_bad = b;
    }
}

// A block partial as it crosses from the block that made it to the block that adds them all up
// inside one launch. The compute units of MI355X sit in eight dies with a second-level cache each; a
// release fence at device scope would write back that whole cache once per block (measured: the
// statistics pass went from 66 to 85 us). The partial is therefore stored and loaded with
// device-scope atomic accesses (relaxed), which bypass the per-die caches by themselves: once such a
// store has completed (s_waitcnt), every later device-scope access on the device sees it.
// A block draws its ticket only after both words of its partial have completed, so the block that
// draws the last ticket finds every partial whole. The protocol checks itself all the same: the
// count travels with the pass's 16-bit tag in its upper bits, and the reader takes a slot only when
// it carries this pass's tag (re-reading a bounded number of times otherwise), so that a slot that
// still held an earlier pass's contents could never be added up unnoticed. A slot that never shows
// the tag -- which the coherence of device-scope accesses rules out -- is reported as kPartialLost
// non-finite elements: the step is skipped and the iteration flagged, not silently wrong.
constexpr int kPartialTagShift = 48;                      // counts stay below 2^48 elements
constexpr uint64_t kPartialCountMask = (1ull << kPartialTagShift) - 1;
constexpr uint64_t kPartialLost = 1ull << 47;
constexpr int kPartialRetries = 1 << 16;

__device__ __forceinline__ void publish_partial(StatsPartial* slot, double sum, uint64_t bad, uint32_t tag)
{
    __hip_atomic_store(reinterpret_cast<uint64_t*>(&slot->sumsq), __builtin_bit_cast(uint64_t, sum), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&slot->nonfinite, (bad & kPartialCountMask) | ((uint64_t)tag << kPartialTagShift), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // both have arrived before the ticket is drawn
}
// One slot, patiently: for a slot that did not show this pass's tag at the first look.
__device__ __forceinline__ StatsPartial reread_partial(const StatsPartial* slot, uint32_t tag)
{
    StatsPartial r;
    uint64_t word = 0;
    int tries = 0;
    do {
        word = __hip_atomic_load(&slot->nonfinite, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } while ((uint32_t)(word >> kPartialTagShift) != tag && ++tries < kPartialRetries);
    if ((uint32_t)(word >> kPartialTagShift) != tag) {
        r.sumsq = 0.0;
        r.nonfinite = kPartialLost;
        return r;
    }
    asm volatile("" ::: "memory");  // the sum is loaded after the tagged count has been seen
    r.sumsq = __builtin_bit_cast(double, __hip_atomic_load(reinterpret_cast<const uint64_t*>(&slot->sumsq), __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT));
    r.nonfinite = word & kPartialCountMask;
    return r;
}
// Thread t of 256 adds up partials t, t + 256, ... in that order. The loads of four slots are issued
// together and looked at afterwards: the block that runs this has just waited for the last partial,
// and a round trip to device-coherent memory per slot and word (four in a row for 512 partials) would
// be most of what the final sum costs.
template <bool COHERENT>
__device__ __forceinline__ void sum_partials(const StatsPartial* partials, int nparts, uint32_t tag, double& s, uint64_t& b)
{
    constexpr int kBatch = 4;
    s = 0.0;
    b = 0;
    for (int first = threadIdx.x; first < nparts; first += 256 * kBatch) {
        uint64_t word[kBatch], sum[kBatch];
#pragma unroll
        for (int k = 0; k < kBatch; ++k) {
            const int i = first + k * 256;
            word[k] = sum[k] = 0;
            if (i < nparts) {
                if constexpr (COHERENT) {
                    word[k] = __hip_atomic_load(&partials[i].nonfinite, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    sum[k] = __hip_atomic_load(reinterpret_cast<const uint64_t*>(&partials[i].sumsq), __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                } else {  // written by an earlier launch
                    word[k] = partials[i].nonfinite;
                    sum[k] = __builtin_bit_cast(uint64_t, partials[i].sumsq);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kBatch; ++k) {
            const int i = first + k * 256;
            if (i < nparts) {
                StatsPartial part;
                part.sumsq = __builtin_bit_cast(double, sum[k]);
                part.nonfinite = word[k];
                if constexpr (COHERENT) {
                    part.nonfinite = word[k] & kPartialCountMask;
                    if ((uint32_t)(word[k] >> kPartialTagShift) != tag) part = reread_partial(partials + i, tag);
                }
                s += part.sumsq;
                b += part.nonfinite;
            }
        }
    }
}

// The per-step decision from a statistics record (one thread):
//   skip = nonfinite != 0 . norm = sqrt(sumsq) (double) . clip = min(1, max_norm / (norm + 1e-6))
//   (double, then fp32; 1 when max_norm <= 0) . grad_mult = clip * inv_scale (one fp32 multiply)
__device__ __forceinline__ void write_decision(uint64_t nonfinite, double sumsq, float inv_scale, float max_norm,
                                               ft_step_control_t* ctl)
{
    const double norm = __builtin_sqrt(sumsq);
    double coef = 1.0;
    if (max_norm > 0.0f) {
        coef = (double)max_norm / (norm + 1e-6);
        if (!(coef < 1.0)) coef = 1.0;
    }
    const float clip = (float)coef;
    ctl->skip = nonfinite != 0 ? 1u : 0u;
    ctl->grad_mult = clip * inv_scale;
    // the norm of finite fp32 gradients can exceed the fp32 range (two elements of 3e38): the
    // informational copy saturates instead of turning into inf; clip is computed from the double
    ctl->grad_norm = norm < 3.4028234663852886e38 ? (float)norm : 3.4028234663852886e38f;
    ctl->clip_coef = clip;
}

// Stores (or adds to) the statistics record and, when a control record is asked for, decides from
// the record as it now stands: the last launch of a statistics pass then is the decision as well.
__device__ __forceinline__ void publish_stats(double s, uint64_t b, ft_grad_stats_t* out, int accumulate, float inv_scale,
                                              float max_norm, ft_step_control_t* ctl)
{
    if (accumulate) {
        s += out->sumsq;
        b += out->nonfinite;
    }
    out->sumsq = s;
    out->nonfinite = b;
    if (ctl) write_decision(b, s, inv_scale, max_norm, ctl);
}

// What the end of a statistics pass needs beside the block partials: the elements outside the
// vector body, where the result goes, and the decision to take from it (ctl == nullptr: none).
struct StatsFinalArgs {
    const void* g;        // the whole gradient buffer
    uint64_t head;        // elements in front of the vector body
    uint64_t tail_begin;  // first element behind it
    uint64_t n;
    ft_grad_stats_t* out;
    int accumulate;
    float inv_scale;
    float max_norm;
    ft_step_control_t* ctl;
    uint32_t* ticket;     // one-launch mode: counts the blocks that have delivered their partial; nullptr: two launches
    uint32_t tag;         // one-launch mode: 16-bit tag of this pass (differs from the previous pass on the same scratch)
};

// End of a statistics pass, run by the first 256 threads of ONE block (all threads of the block must
// call it): adds the block partials in a fixed order (strided per thread, wavefront sums, then the
// four wavefronts), then the elements before/after the vector body one by one, and writes or
// accumulates the result. The order of the additions depends on nparts only, not on which block
// runs it.
template <int GT, bool COHERENT>
__device__ __forceinline__ void stats_final_block(const StatsPartial* partials, int nparts, float pre_mult, const StatsFinalArgs& f)
{
    __shared__ double s_fsum[4];
    __shared__ uint64_t s_fbad[4];
    if (threadIdx.x < 256) {
        double s;
        uint64_t b;
        sum_partials<COHERENT>(partials, nparts, f.tag, s, b);
        s = wave_sum_f64(s);
        b = wave_sum_u64(b);
        if ((threadIdx.x & (kWave - 1)) == 0) {
            s_fsum[threadIdx.x / kWave] = s;
            s_fbad[threadIdx.x / kWave] = b;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = (s_fsum[0] + s_fsum[1]) + (s_fsum[2] + s_fsum[3]);
        uint64_t b = (s_fbad[0] + s_fbad[1]) + (s_fbad[2] + s_fbad[3]);
        for (uint64_t i = 0; i < f.n; ++i) {
            if (i == f.head) i = f.tail_begin;  // skip the vector body
            if (i >= f.n) break;
            float x;
            bool nf;
            if constexpr (GT == FT_F32) {
                const uint32_t w = reinterpret_cast<const uint32_t*>(f.g)[i];
                nf = (w & 0x7f800000u) == 0x7f800000u;
                x = __builtin_bit_cast(float, w);
            } else {
                constexpr uint32_t kExp = (GT == FT_BF16) ? 0x7f80u : 0x7c00u;
                const uint32_t w = reinterpret_cast<const uint16_t*>(f.g)[i];
                nf = (w & kExp) == kExp;
                x = half_to_float<GT>(w);
            }
            if (nf)
                b += 1;
            else
                s = add_square(x * pre_mult, s);
        }
        publish_stats(s, b, f.out, f.accumulate, f.inv_scale, f.max_norm, f.ctl);
    }
}

// Stage 1: every block writes one StatsPartial. nvec = number of 16-byte units; the caller
// handles the elements outside [0, nvec*per_unit) in grad_stats_final_kernel.
// Every square is formed and added in fp64 (four accumulators per lane), in the vector body as in
// the edges, so an element contributes the same whatever part of the call it falls into, and no
// finite gradient can overflow the sum or vanish from it. The sums are the same bits whichever of the
// two ways below a block takes: both add an element's square to the same accumulator in the same order.
// The gradients are read again by the update that follows the decision, so what of them still fits
// the memory-side cache afterwards is worth keeping there: tiles from `keep_from_tile` on (the last
// ones this pass touches) are read with ordinary loads, everything before with streaming loads that
// leave nothing behind. The update's own traffic is streaming, so the kept lines survive until it
// reaches them. Measured on the 7B-layer partition (405 MB of fp16 gradients, 256 MB cache): the
// update behind an all-streaming pass takes 0.838 ms, behind a caching pass 0.79 ms.
template <int GT, int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void grad_stats_kernel(const u32x4* __restrict__ g, uint64_t nvec,
                                                           float pre_mult, StatsPartial* partials,
                                                           uint64_t keep_from_tile, const float* scale_dev, StatsFinalArgs fin)
{
    static_assert(BLOCK >= 256, "the final sum is taken by the first 256 threads of a block");
    if (scale_dev) pre_mult = fin.inv_scale = *scale_dev;  // 1/loss_scale kept in device memory (wave-uniform load)
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    uint32_t bad = 0;
    constexpr uint64_t kTile = (uint64_t)BLOCK * UNROLL;
    const uint64_t full_tiles = nvec / kTile;
    const uint64_t stream_tiles = keep_from_tile < full_tiles ? keep_from_tile : full_tiles;
    // The optimistic pass: whole tiles only, no branch inside a loop body (a body that first screens
    // its loads and then chooses between two ways of adding them has to wait for all of a tile's loads
    // before it can start on the first, and took 4-15 us more over 405 MB than one that simply adds:
    // 62-76 against 57.5 us). Every load is added as if finite, and its inf/nan marks are collected on
    // the side; a block that has seen a mark throws its sums away and goes over its tiles again, element
    // by element (an overflow step is thrown away as a whole anyway, and costs this block its share of
    // the pass a second time).
    uint32_t marks = 0;
    uint64_t tile = blockIdx.x;
    for (; tile < stream_tiles; tile += gridDim.x) {
        const uint64_t base = tile * kTile + threadIdx.x;
        u32x4 w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) w[u] = __builtin_nontemporal_load(g + base + (uint64_t)u * BLOCK);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            marks |= nonfinite_marks<GT>(w[u]);
            stats_accumulate_finite<GT>(w[u], pre_mult, acc);
        }
    }
    for (; tile < full_tiles; tile += gridDim.x) {  // buffer loads with the default cache policy: a distinct instruction
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(g + tile * kTile), 0,
                                                                           (int)(kTile * 16), kRawBufferFlags);
        u32x4 w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            w[u] = __builtin_amdgcn_raw_buffer_load_b128(r, (int)((threadIdx.x + u * BLOCK) * 16), 0, 0);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            marks |= nonfinite_marks<GT>(w[u]);
            stats_accumulate_finite<GT>(w[u], pre_mult, acc);
        }
    }
    if (__syncthreads_or(marks != 0)) {  // rare: the same tiles in the same order, every element tested
        acc[0] = acc[1] = acc[2] = acc[3] = 0.0;
        for (tile = blockIdx.x; tile < full_tiles; tile += gridDim.x) {
            const uint64_t base = tile * kTile + threadIdx.x;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) stats_accumulate<GT>(g[base + (uint64_t)u * BLOCK], pre_mult, acc, bad);
        }
    }
    // the units behind the last whole tile go to the block whose turn that tile would have been
    if (tile == full_tiles) {
        const uint64_t base = tile * kTile + threadIdx.x;
        for (int u = 0; u < UNROLL; ++u) {
            const uint64_t i = base + (uint64_t)u * BLOCK;
            if (i >= nvec) break;
            stats_accumulate<GT>(g[i], pre_mult, acc, bad);
        }
    }
    double total;
    uint64_t total_bad;
    block_stats_reduce<BLOCK>((acc[0] + acc[1]) + (acc[2] + acc[3]), bad, total, total_bad);
    if (fin.ticket == nullptr) {  // two launches: grad_stats_final_kernel follows
        if (threadIdx.x == 0) {
            partials[blockIdx.x].sumsq = total;
            partials[blockIdx.x].nonfinite = total_bad;
        }
        return;
    }
    // One launch: every block draws a ticket once its partial has arrived where the whole device
    // sees it; the block that draws the last one adds the partials up, in the same fixed order as the
    // separate launch would, and leaves the ticket counter at zero for the next pass on this stream.
    __shared__ uint32_t s_last;
    if (threadIdx.x == 0) {
        publish_partial(partials + blockIdx.x, total, total_bad, fin.tag);
        s_last = __hip_atomic_fetch_add(fin.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1 ? 1u : 0u;
    }
    __syncthreads();
    if (s_last == 0) return;
    stats_final_block<GT, true>(partials, (int)gridDim.x, pre_mult, fin);
    if (threadIdx.x == 0) __hip_atomic_store(fin.ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The end of a statistics pass as a launch of its own (one block of 256): for a pass whose vector
// body is empty and for callers that may not share a ticket counter (a stream under graph capture).
template <int GT>
__global__ __launch_bounds__(256) void grad_stats_final_kernel(const StatsPartial* partials, int nparts, float pre_mult,
                                                               const float* scale_dev, StatsFinalArgs fin)
{
    if (scale_dev) pre_mult = fin.inv_scale = *scale_dev;
    stats_final_block<GT, false>(partials, nparts, pre_mult, fin);
}

// ---- gradient accumulation ---------------------------------------------------------------------
// acc[i] = fma((float)g[i], scale, acc[i]), rounded to acc's type (scale == 1 is a plain add of the
// widened gradient). Optionally clears g afterwards and gathers the statistics of the new acc
// (exactly what grad_stats_kernel would report for it), so that the pass over the gradients that
// accumulation needs anyway also yields the overflow flag and the norm.
template <int AT>
__device__ __forceinline__ void stats_of_stored(float value, uint32_t bits, float pre_mult, double& acc, uint32_t& bad)
{
    constexpr uint32_t kExp = (AT == FT_F32) ? 0x7f800000u : (AT == FT_BF16 ? 0x7f80u : 0x7c00u);
    const bool nf = (bits & kExp) == kExp;
    const float x = value * pre_mult;
    bad += nf ? 1u : 0u;
    acc = add_square(nf ? 0.0f : x, acc);
}

// One 64-unit tile: lane `threadIdx.x` takes unit tile*64 + lane when that is below nvec. All
// accesses are streaming: every buffer is far larger than the caches and is touched once. The
// descriptors cover only the units of this tile that exist, so lanes past nvec cannot store.
template <int AT, int GT, bool ZERO, bool STATS>
__device__ __forceinline__ void accumulate_tile(void* acc, void* g, uint64_t tile, uint64_t nvec, float scale,
                                                float pre_mult, double& sum, uint32_t& bad, bool keep, bool g_relaxed)
{
    constexpr uint32_t kAccUnit = (AT == FT_F32) ? 16 : 8, kGradUnit = (GT == FT_F32) ? 16 : 8;
    const uint64_t t0 = tile * 64;  // wave-uniform
    const uint32_t live = (nvec - t0 < 64) ? (uint32_t)(nvec - t0) : 64u;
    const __amdgpu_buffer_rsrc_t racc = tile_rsrc(static_cast<char*>(acc) + t0 * kAccUnit, live * kAccUnit);
    const uint64_t i = t0 + threadIdx.x;
    if (threadIdx.x >= live) return;

    // The gradient unit as raw bits, fetched either way before anything waits for it. g_relaxed: g's
    // tiles do not start on cache lines where acc's do (g off its vector alignment, or only off the
    // lines), so element alignment only, and a tile shares a line with its neighbour at either end:
    // read with the default cache policy (a buffer load: a distinct instruction, the compiler would
    // merge two global loads that differ in the streaming hint), so that the second reader finds the
    // line in a cache and the clearing store below meets it there.
    f32x4 g32;
    u32x2 g16;
    if constexpr (GT == FT_F32) {
        if (!g_relaxed) {
            g32 = ld<true>(reinterpret_cast<const f32x4*>(g) + i);
        } else {
            const __amdgpu_buffer_rsrc_t r = tile_rsrc(reinterpret_cast<f32x4_e*>(g) + t0, live * 16);
            g32 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(threadIdx.x * 16), 0, 0));
        }
    } else {
        if (!g_relaxed) {
            g16 = ld<true>(reinterpret_cast<const u32x2*>(g) + i);
        } else {
            const __amdgpu_buffer_rsrc_t r = tile_rsrc(reinterpret_cast<u16x4_e*>(g) + t0, live * 8);
            g16 = __builtin_amdgcn_raw_buffer_load_b64(r, (int)(threadIdx.x * 8), 0, 0);
        }
    }
    f32x4 a4;
    if constexpr (AT == FT_F32) {
        a4 = ld<true>(reinterpret_cast<const f32x4*>(acc) + i);
    } else {
        const u32x2 w = ld<true>(reinterpret_cast<const u32x2*>(acc) + i);
        a4.x = half_to_float<AT>(w.x & 0xffffu);
        a4.y = half_to_float<AT>(w.x >> 16);
        a4.z = half_to_float<AT>(w.y & 0xffffu);
        a4.w = half_to_float<AT>(w.y >> 16);
    }
    f32x4 g4;
    if constexpr (GT == FT_F32) {
        g4 = g32;
    } else {
        g4.x = half_to_float<GT>(g16.x & 0xffffu);
        g4.y = half_to_float<GT>(g16.x >> 16);
        g4.z = half_to_float<GT>(g16.y & 0xffffu);
        g4.w = half_to_float<GT>(g16.y >> 16);
    }
    f32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float x = __builtin_fmaf(g4[k], scale, a4[k]);
        asm volatile("" : "+v"(x));  // round to fp32 first; a narrowing store must see this value
        r[k] = x;
    }
    if constexpr (AT == FT_F32) {
        if (keep)
            st_keep(racc, threadIdx.x * kAccUnit, r);
        else
            st_stream(racc, threadIdx.x * kAccUnit, r);
        if constexpr (STATS) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float rk = r[k];  // a scalar copy: bit-casting the vector element itself reads lane 0
                stats_of_stored<FT_F32>(rk, __builtin_bit_cast(uint32_t, rk), pre_mult, sum, bad);
            }
        }
    } else {
        u32x2 w;
        w.x = pack2<AT>(r.x, r.y);
        w.y = pack2<AT>(r.z, r.w);
        if (keep)
            st_keep(racc, threadIdx.x * kAccUnit, w);
        else
            st_stream(racc, threadIdx.x * kAccUnit, w);
        if constexpr (STATS) {
            const uint32_t b[4] = {w.x & 0xffffu, w.x >> 16, w.y & 0xffffu, w.y >> 16};
#pragma unroll
            for (int k = 0; k < 4; ++k) stats_of_stored<AT>(half_to_float<AT>(b[k]), b[k], pre_mult, sum, bad);
        }
    }
    if constexpr (ZERO) {
        if (g_relaxed) {
            if constexpr (GT == FT_F32) {
                const f32x4_e z = {0.f, 0.f, 0.f, 0.f};
                __builtin_nontemporal_store(z, reinterpret_cast<f32x4_e*>(g) + i);
            } else {
                const u16x4_e z = {0, 0, 0, 0};
                __builtin_nontemporal_store(z, reinterpret_cast<u16x4_e*>(g) + i);
            }
            return;
        }
        const __amdgpu_buffer_rsrc_t rg = tile_rsrc(static_cast<char*>(g) + t0 * kGradUnit, live * kGradUnit);
        if constexpr (GT == FT_F32) {
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            st_stream(rg, threadIdx.x * kGradUnit, z);
        } else {
            const u32x2 z = {0u, 0u};
            st_stream(rg, threadIdx.x * kGradUnit, z);
        }
    }
}

// What one wavefront-sized workgroup of the accumulation pass reports: 16 bytes per 256 elements.
// The squares are formed and added in fp64 from the first element on (see add_square).
struct WavePartial {
    double sumsq;
    uint32_t nonfinite;
    uint32_t reserved;
};

// nvec = number of 4-element units; one 64-lane workgroup per 64 units (the loop only matters when
// the grid had to be capped). With STATS every workgroup writes wave_partials[blockIdx.x].
template <int AT, int GT, bool ZERO, bool STATS>
__global__ __launch_bounds__(64) void grad_accumulate_kernel(void* acc, void* g, uint64_t nvec, float scale,
                                                             float pre_mult, WavePartial* __restrict__ wave_partials,
                                                             uint64_t keep_from_tile, int g_relaxed)
{
    double sum = 0.0;
    uint32_t bad = 0;
    const uint64_t ntiles = (nvec + 63) / 64;
    for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x)
        accumulate_tile<AT, GT, ZERO, STATS>(acc, g, tile, nvec, scale, pre_mult, sum, bad, tile >= keep_from_tile, g_relaxed != 0);
    if constexpr (STATS) {
        const double t = wave_sum_f64(sum);
        const uint32_t tb = wave_sum_u32(bad);
        if (threadIdx.x == 0) {
            WavePartial w;
            w.sumsq = t;
            w.nonfinite = tb;
            w.reserved = 0;
            wave_partials[blockIdx.x] = w;
        }
    }
}

// Second level: block r adds the contiguous slice [r*per_block, (r+1)*per_block) of the wavefront
// partials in fp64, lanes striding the slice, then a fixed tree; one StatsPartial per block. The
// order of every addition is fixed by (count, gridDim), so the result is reproducible.
__global__ __launch_bounds__(256) void reduce_wave_partials_kernel(const WavePartial* __restrict__ wave_partials,
                                                                   uint64_t count, uint64_t per_block,
                                                                   StatsPartial* __restrict__ partials)
{
    __shared__ double s_sum[256];
    __shared__ uint64_t s_bad[256];
    const uint64_t lo = (uint64_t)blockIdx.x * per_block;
    uint64_t hi = lo + per_block;
    if (hi > count) hi = count;
    double s = 0.0;
    uint64_t b = 0;
    for (uint64_t i = lo + threadIdx.x; i < hi; i += 256) {
        const WavePartial w = wave_partials[i];
        s += w.sumsq;
        b += w.nonfinite;
    }
    s_sum[threadIdx.x] = s;
    s_bad[threadIdx.x] = b;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + w];
            s_bad[threadIdx.x] += s_bad[threadIdx.x + w];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partials[blockIdx.x].sumsq = s_sum[0];
        partials[blockIdx.x].nonfinite = s_bad[0];
    }
}

// Last launch of an accumulation pass (one block of 256): the elements outside the vector body (up
// to 255 in front of it, up to 3 behind) go one per thread and round; with STATS the block then adds
// the second-level partials and every thread's edge share in a fixed tree order and thread 0 writes
// or accumulates the result.
template <int AT, int GT, bool ZERO, bool STATS>
__global__ __launch_bounds__(256) void grad_accumulate_finish_kernel(void* acc, void* g, uint64_t head,
                                                                     uint64_t tail_begin, uint64_t n, float scale,
                                                                     float pre_mult,
                                                                     const StatsPartial* __restrict__ partials,
                                                                     int nparts, ft_grad_stats_t* out, int accumulate,
                                                                     float inv_scale, float max_norm, ft_step_control_t* ctl)
{
    double s = 0.0;
    uint64_t b = 0;
    const uint64_t edge = head + (n - tail_begin);
    for (uint64_t e = threadIdx.x; e < edge; e += 256) {
        const uint64_t i = e < head ? e : tail_begin + (e - head);
        float gi;
        if constexpr (GT == FT_F32)
            gi = reinterpret_cast<const float*>(g)[i];
        else
            gi = half_to_float<GT>(reinterpret_cast<const uint16_t*>(g)[i]);
        float ai;
        if constexpr (AT == FT_F32)
            ai = reinterpret_cast<const float*>(acc)[i];
        else
            ai = half_to_float<AT>(reinterpret_cast<const uint16_t*>(acc)[i]);
        float x = __builtin_fmaf(gi, scale, ai);
        asm volatile("" : "+v"(x));
        uint32_t bits;
        float stored;
        if constexpr (AT == FT_F32) {
            reinterpret_cast<float*>(acc)[i] = x;
            bits = __builtin_bit_cast(uint32_t, x);
            stored = x;
        } else {
            bits = pack2<AT>(x, 0.0f) & 0xffffu;
            reinterpret_cast<uint16_t*>(acc)[i] = (uint16_t)bits;
            stored = half_to_float<AT>(bits);
        }
        if constexpr (STATS) {
            uint32_t nb = 0;
            stats_of_stored<AT>(stored, bits, pre_mult, s, nb);
            b += nb;
        }
        if constexpr (ZERO) {
            if constexpr (GT == FT_F32)
                reinterpret_cast<float*>(g)[i] = 0.0f;
            else
                reinterpret_cast<uint16_t*>(g)[i] = 0;
        }
    }
    if constexpr (STATS) {
        __shared__ double s_sum[256];
        __shared__ uint64_t s_bad[256];
        double ps = s;   // this thread's edge elements, then its share of the partials
        uint64_t pb = b;
        for (int i = threadIdx.x; i < nparts; i += 256) {
            ps += partials[i].sumsq;
            pb += partials[i].nonfinite;
        }
        s_sum[threadIdx.x] = ps;
        s_bad[threadIdx.x] = pb;
        __syncthreads();
        for (int w = 128; w > 0; w >>= 1) {
            if ((int)threadIdx.x < w) {
                s_sum[threadIdx.x] += s_sum[threadIdx.x + w];
                s_bad[threadIdx.x] += s_bad[threadIdx.x + w];
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) publish_stats(s_sum[0], s_bad[0], out, accumulate, inv_scale, max_norm, ctl);
    }
}

__global__ void grad_control_kernel(const ft_grad_stats_t* stats, float inv_scale, float max_norm,
                                    ft_step_control_t* ctl)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    write_decision(stats->nonfinite, stats->sumsq, inv_scale, max_norm, ctl);
}

}  // namespace ftk
