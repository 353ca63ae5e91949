// ft_adam.hip -- resident optimizer step, gradient statistics and the registry behind the C ABI.
//
// Replaces the native half of the reference's optimizer step:
//   flextrain/ops/csrc/adam/cpu_adam.cpp:8-16        (the four exported functions)
//   flextrain/ops/csrc/adam/cpu_adam_impl.cpp:143-302 (registry, marshalling, work partition)
//   flextrain/ops/csrc/includes/cpu_adam.h:67-102     (host scalars)
// The arithmetic itself lives in ft_kernels.hpp.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <cmath>
#include <map>
#include <mutex>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "ft_internal.hpp"
#include "ft_kernels.hpp"
#include "ft_launch_plan.hpp"

// Launch shape of the update kernel, from sweeps on MI355X at 2e8 elements: one 64-lane wavefront
// per workgroup, one 4-element unit per lane, one workgroup per tile, non-temporal loads, streaming
// stores, and at most 11 workgroups resident per compute unit. More resident wavefronts put more
// requests in flight than HBM can serve in order and cost up to 8 % of the bandwidth.
#ifndef FT_ADAM_WAVES_PER_CU
#define FT_ADAM_WAVES_PER_CU 11
#endif
#ifndef FT_STATS_BLOCK
#define FT_STATS_BLOCK 256
#endif
#ifndef FT_STATS_UNROLL
#define FT_STATS_UNROLL 4
#endif
#ifndef FT_STATS_BLOCKS_PER_CU
#define FT_STATS_BLOCKS_PER_CU 2
#endif

namespace {

thread_local std::string t_last_error;

std::mutex g_mu;
std::unordered_map<int, fth::AdamObject> g_adams;
std::unordered_map<int, int> g_cu_count;      // device -> compute units
// What the library keeps per (device, stream) for the statistics passes enqueued there: a scratch
// buffer for callers that bring none (calls on different streams never share one) and a ticket
// counter for the one-launch statistics pass. Calls on one stream run in order, so they may share
// both. ft_release_stream_scratch gives them back.
struct StreamState {
    void* ptr = nullptr;  // library-owned scratch, grown on demand
    size_t bytes = 0;
    int ticket_slot = -1; // index into the device's ticket pool, -1: none assigned (yet, or pool exhausted)
    uint32_t tag = 0;     // tag of the last one-launch pass enqueued here (16 bits, never 0)
};
std::map<std::pair<int, hipStream_t>, StreamState> g_stream_state;
constexpr int kTicketSlots = 1024;
constexpr int kTicketStride = 16;  // counters 64 bytes apart: one cache line each
std::unordered_map<int, std::vector<int>> g_free_ticket_slots;  // device -> slots not in use
int g_adam_waves_per_cu = FT_ADAM_WAVES_PER_CU;
std::unordered_map<int, int> g_lds_per_cu;   // device -> bytes of LDS per compute unit
std::atomic<int> g_stats_blocks_per_cu{FT_STATS_BLOCKS_PER_CU};  // read without the lock
// How many bytes at the end of a statistics pass are read with caching loads (the size of the
// memory-side cache of MI355X: what can still be there when the update reads the gradients again).
std::atomic<size_t> g_stats_keep_bytes{static_cast<size_t>(256) << 20};
// The statistics pass as one launch (the last block takes the final sum) or as two.
std::atomic<int> g_stats_one_launch{1};
// Workgroups (of 64 lanes) one launch may hold: what the runtime allows, or less when a test asks for
// many launches of a modest amount of work (ft_set_launch_limit).
std::atomic<uint64_t> g_launch_limit{ftk::kMaxWorkgroupsPerLaunch};
inline uint64_t launch_limit() { return g_launch_limit.load(); }
inline uint64_t multi_launch_limit()
{
    const uint64_t l = launch_limit();
    return l < ftk::kMultiMaxWorkgroups ? l : ftk::kMultiMaxWorkgroups;
}

constexpr int kMaxStatsBlocks = 8192;

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline size_t elem_size(int dt) { return dt == FT_F32 ? 4 : 2; }

// True when, `head` elements in, every array of a step sits on a cache line (the 16-bit copy, which
// is only written: on half a line), or when the segment is too short for that to matter. Vector
// alignment is not all: the aligned kernels stream every array, and an array whose tiles start
// inside a line (m sixteen bytes off p, say) then costs them far more than it costs the relaxed
// kernel, which knows how to treat such an array (measured on 202 M elements with one array 4
// elements off the others: m 0.895 ms, p 1.04 ms, against 0.838 and 0.844 ms; the aligned kernel is at
// full speed with the copy 64 bytes off, 0.828 ms, and not with a state array 64 bytes off, 0.857 ms).
inline bool arrays_on_lines(size_t head, size_t n, const void* p, const void* m, const void* v, const void* g, size_t gsz,
                            const void* h, const void* out_p, const void* out_m, const void* out_v)
{
    if (head >= n || n - head < 16 * 256) return true;
    auto on = [&](const void* base, size_t esz, size_t line) { return aligned(static_cast<const char*>(base) + head * esz, line); };
    const size_t line = fth::kLineBytes;
    return on(p, 4, line) && on(m, 4, line) && on(v, 4, line) && on(g, gsz, line) && (h == nullptr || on(h, 2, line / 2)) &&
           on(out_p, 4, line) && on(out_m, 4, line) && on(out_v, 4, line);
}
inline bool valid_dtype(int dt) { return dt == FT_F32 || dt == FT_F16 || dt == FT_BF16; }

}  // namespace

namespace fth {

int fail(int code, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    t_last_error = buf;
    return code;
}

int find_adam(int id, AdamObject* out)
{
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_adams.find(id);
    if (it == g_adams.end()) return fail(FT_ENOENT, "no optimizer with id %d (ft_adam_create first)", id);
    *out = it->second;
    return FT_OK;
}

int cu_count()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_cu_count.find(dev);
    if (it != g_cu_count.end()) return it->second;
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    g_cu_count[dev] = n;
    return n;
}

// Dynamic LDS requested per 64-lane workgroup of a streaming kernel. The kernel never touches it:
// the allocation only bounds how many workgroups fit on a compute unit at once. The tuned figure
// (g_adam_waves_per_cu) is for the update with 16-bit gradients, whose lanes have 56 bytes of loads
// in flight each; what has to stay constant is the bytes in flight per compute unit, so a kernel
// that loads fewer bytes per lane gets proportionally more resident wavefronts.
unsigned throttle_lds_bytes(unsigned load_bytes_per_lane, unsigned percent)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lk(g_mu);
    int waves = (g_adam_waves_per_cu * 56 + static_cast<int>(load_bytes_per_lane) / 2) / static_cast<int>(load_bytes_per_lane);
    waves = waves * static_cast<int>(percent) / 100;
    if (waves < 1) waves = 1;
    if (waves >= 32) return 0;  // hardware limit: 32 wavefronts per CU anyway
    auto it = g_lds_per_cu.find(dev);
    int lds = 0;
    if (it != g_lds_per_cu.end()) {
        lds = it->second;
    } else {
        if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess || lds <= 0)
            lds = 160 * 1024;
        g_lds_per_cu[dev] = lds;
    }
    int per_wg = (lds / waves) / 512 * 512;
    if (per_wg > 64 * 1024) per_wg = 64 * 1024;
    return static_cast<unsigned>(per_wg);
}

ftk::AdamConsts make_consts(uint64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                            bool bias_correction, bool adamw_mode, float grad_mult)
{
    // beta^t: the reference calls std::pow(float, size_t), i.e. the double overload, and stores the
    // result in a float member (cpu_adam.h:73-74). Everything after that is float arithmetic.
    const float b1t = static_cast<float>(std::pow(static_cast<double>(beta1), static_cast<double>(step)));
    const float b2t = static_cast<float>(std::pow(static_cast<double>(beta2), static_cast<double>(step)));
    float bias1 = 1.0f, bias2 = 1.0f;
    if (bias_correction) {
        bias1 = 1.0f - b1t;
        bias2 = 1.0f / sqrtf(1.0f - b2t);
    }
    ftk::AdamConsts c;
    c.beta1 = beta1;
    c.beta2 = beta2;
    c.omb1 = 1.0f - beta1;
    c.omb2 = 1.0f - beta2;
    c.bias2 = bias2;
    c.eps = eps;
    c.step_size = (-1.0f * lr) / bias1;
    c.wd_mode = 0;
    c.wd_coef = 0.0f;
    if (weight_decay > 0.0f) {
        c.wd_mode = adamw_mode ? 1 : 2;
        c.wd_coef = adamw_mode ? (-1.0f * lr) * weight_decay : weight_decay;
    }
    c.grad_mult = grad_mult;
    return c;
}

// Elements in front of the vector body of a segment: up to 3 to bring p to a 16-byte boundary (what
// the vector accesses need) and, once the segment is long enough for it to matter, on to a 1 KiB
// boundary, so that every tile (1 KiB of each fp32 array, 512 bytes of each 16-bit one) covers
// whole cache lines. Tiles cut at an odd offset write partial lines: the 7B-layer partition
// stepped as two segments cut at a random element took 0.99 ms against 0.83 ms.
size_t segment_head(const void* p, size_t n)
{
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    size_t head = ((16 - (a & 15)) & 15) / 4;
    if (head > n) return n;
    if (n - head >= 16 * 256) head = ((1024 - (a & 1023)) & 1023) / 4;
    return head;
}

namespace {

struct OutPtrs {
    float *p, *m, *v;
};

template <int GT, int HT>
int launch_typed(const ftk::AdamConsts& c, float* p, const void* g, float* m, float* v, void* h, size_t n,
                 const ft_step_control_t* ctl, hipStream_t stream, OutPtrs out, const ftk::AdamConsts* hyper)
{
    constexpr size_t gsz = (GT == FT_F32) ? 4 : 2;
    const char* gb = reinterpret_cast<const char*>(g);
    char* mb = reinterpret_cast<char*>(m);
    char* vb = reinterpret_cast<char*>(v);
    char* hb = reinterpret_cast<char*>(h);

    // Elements before the first 16-byte boundary of p. The vector body needs every array to reach
    // its own vector alignment after the same number of elements; flat buffers sliced at a common
    // element offset (the reference's StepContext views, flextrain/param_group.py:196-199) do.
    const size_t head = segment_head(p, n);
    const bool vec_ok = aligned(mb + head * 4, 16) && aligned(vb + head * 4, 16) &&
                        aligned(gb + head * gsz, gsz * 4) && (h == nullptr || aligned(hb + head * 2, 8)) &&
                        aligned(out.p + head, 16) && aligned(out.m + head, 16) && aligned(out.v + head, 16);
    // Whole 64-unit tiles go to the tile kernel, everything else (the head and up to 255 elements
    // behind the last full tile) to the scalar kernel.
    const size_t ntiles = vec_ok ? (n - head) / 4 / ftk::kWave : 0;
    const size_t body = ntiles * ftk::kWave * 4;

    auto scalar_part = [&](size_t off, size_t cnt) -> int {
        if (cnt == 0) return FT_OK;
        ftk::AdamArgs a;
        a.p = p + off;
        a.g = gb + off * gsz;
        a.m = m + off;
        a.v = v + off;
        a.p_out = out.p + off;
        a.m_out = out.m + off;
        a.v_out = out.v + off;
        a.h = h ? hb + off * 2 : nullptr;
        a.ctl = ctl;
        a.hyper = hyper;
        a.n = cnt;
        a.c = c;
        size_t blocks = (cnt + 255) / 256;
        const size_t cap = static_cast<size_t>(cu_count()) * 16;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((ftk::adam_scalar_kernel<GT, HT>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                           stream, a);
        FT_HIP(hipGetLastError());
        return FT_OK;
    };

    // Segments whose arrays agree as vectors but not on cache lines go the relaxed way as well.
    const bool lines_ok = arrays_on_lines(head, n, p, m, v, g, gsz, h, out.p, out.m, out.v);
    if (!vec_ok || !lines_ok) {
        // Arrays whose alignments disagree: whole tiles still go through a tile kernel (one that
        // assumes element alignment only), the rest element by element. The tiles start where most
        // of the traffic is on whole cache lines (written bytes counted twice).
        const fth::ArrayPlacement place[8] = {
            {reinterpret_cast<uintptr_t>(out.p), 4, 8}, {reinterpret_cast<uintptr_t>(out.m), 4, 8},
            {reinterpret_cast<uintptr_t>(out.v), 4, 8}, {reinterpret_cast<uintptr_t>(h), 2, h ? 4u : 0u},
            {reinterpret_cast<uintptr_t>(p), 4, 4},     {reinterpret_cast<uintptr_t>(m), 4, 4},
            {reinterpret_cast<uintptr_t>(v), 4, 4},     {reinterpret_cast<uintptr_t>(g), static_cast<uint32_t>(gsz), static_cast<uint32_t>(gsz)}};
        uint32_t on_lines = 0;
        const size_t head_r = fth::plan_relaxed_head(place, 8, &on_lines);
        const size_t rhead = head_r < n ? head_r : n;
        const size_t rtiles = (n - rhead) / 4 / ftk::kWave;
        if (rtiles == 0) return scalar_part(0, n);
        // How the kernel treats each array (measured on a 202 M-element update with one array or several
        // one element off the others; fractions of 8 TB/s; the aligned kernel: 85-86 %). Outputs on
        // lines are stored write-through like the aligned kernel's. Where exactly one of the three
        // state arrays is off the lines, or none of them and the gradient is, that array is read with
        // the default cache policy and the tiles are taken in order (83-86 %; streamed and in runs of
        // eight per die: 81-83 %); a copy that alone is off is stored with the default policy, tiles in
        // order (83 %). In every other case all loads stream and tiles go in runs (two state arrays
        // off: 77-78 % against 72 % the other way; every array at another offset: 75 %).
        uint32_t flags = on_lines & (ftk::kRelaxedOnLinesP | ftk::kRelaxedOnLinesM | ftk::kRelaxedOnLinesV);
        const bool copy_off = h && !(on_lines & 8u), grad_off = !(on_lines & 128u);
        if (h && !copy_off) flags |= ftk::kRelaxedOnLinesH;
        const uint32_t state_off = (~on_lines >> 4) & 7u;  // inputs p, m, v whose tiles start inside a line
        int cached = 0;
        if (state_off == 1u || state_off == 2u || state_off == 4u) {
            cached = 1;
            flags |= (state_off == 1u ? 0u : state_off == 2u ? 1u : 2u) << ftk::kRelaxedCachedShift;
        } else if (state_off == 0u && grad_off) {
            cached = 2;
            if (copy_off) flags |= ftk::kRelaxedCopyCached;
        } else if (state_off == 0u && copy_off) {
            flags |= ftk::kRelaxedCopyCached;
        } else {
            flags |= ftk::kRelaxedRuns;
        }
        ftk::AdamArgs a;
        a.p = p + rhead;
        a.g = gb + rhead * gsz;
        a.m = m + rhead;
        a.v = v + rhead;
        a.p_out = out.p + rhead;
        a.m_out = out.m + rhead;
        a.v_out = out.v + rhead;
        a.h = h ? hb + rhead * 2 : nullptr;
        a.ctl = ctl;
        a.hyper = hyper;
        a.n = rtiles * ftk::kWave;
        a.c = c;
        const unsigned lds = throttle_lds_bytes(48 + 4 * static_cast<unsigned>(gsz));
        uint64_t tile0 = 0, blocks = 0;
        for (uint64_t piece = 0; plan_launch_piece(rtiles, launch_limit(), piece, &tile0, &blocks); ++piece) {
            auto launch = [&](auto has_ctl, auto how) {
                hipLaunchKernelGGL((ftk::adam_tile_relaxed_kernel<GT, HT, decltype(has_ctl)::value, decltype(how)::value>),
                                   dim3(static_cast<unsigned>(blocks)), dim3(ftk::kWave), lds, stream, a, static_cast<uint64_t>(tile0),
                                   flags);
            };
            auto launch_ctl = [&](auto how) {
                if (ctl)
                    launch(std::true_type{}, how);
                else
                    launch(std::false_type{}, how);
            };
            if (cached == 1)
                launch_ctl(std::integral_constant<int, 1>{});
            else if (cached == 2)
                launch_ctl(std::integral_constant<int, 2>{});
            else
                launch_ctl(std::integral_constant<int, 0>{});
            FT_HIP(hipGetLastError());
        }
        const size_t rbody = rtiles * ftk::kWave * 4;
        int rc = scalar_part(0, rhead);
        if (rc != FT_OK) return rc;
        return scalar_part(rhead + rbody, n - rhead - rbody);
    }

    // An in-place segment with edge elements is one launch of the many-segment kernel (tiles and
    // edges in the same grid) instead of up to three.
    const bool in_place = out.p == p && out.m == m && out.v == v;
    if (in_place && (head > 0 || head + body < n) && ntiles + 1 <= multi_launch_limit()) {
        ftk::AdamMultiArgs ma;
        ma.first_wg[0] = 0;
        for (int k = 1; k < ftk::kMultiMaxSegments; ++k) ma.first_wg[k] = 0xffffffffu;
        ma.ctl = ctl;
        ftk::AdamSegment& d = ma.seg[0];
        d.p = p;
        d.g = g;
        d.m = m;
        d.v = v;
        d.h = h;
        d.n = n;
        d.head = static_cast<uint32_t>(head);
        d.body_tiles = static_cast<uint32_t>(ntiles);
        d.hyper = hyper;
        d.c = c;
        return launch_adam_multi(ma, GT, h != nullptr, HT, hyper != nullptr, static_cast<unsigned>(ntiles) + 1u, stream);
    }

    if (ntiles > 0) {
        ftk::AdamArgs a;
        a.p = p + head;
        a.g = gb + head * gsz;
        a.m = m + head;
        a.v = v + head;
        a.p_out = out.p + head;
        a.m_out = out.m + head;
        a.v_out = out.v + head;
        a.h = h ? hb + head * 2 : nullptr;
        a.ctl = ctl;
        a.hyper = hyper;
        a.n = ntiles * ftk::kWave;
        a.c = c;
        const unsigned lds = throttle_lds_bytes(48 + 4 * static_cast<unsigned>(gsz));
        // one workgroup per tile; more tiles than a launch may hold workgroups are cut into several
        uint64_t tile0 = 0, blocks = 0;
        for (uint64_t piece = 0; plan_launch_piece(ntiles, launch_limit(), piece, &tile0, &blocks); ++piece) {
            auto launch = [&](auto has_ctl, auto has_hyper) {
                hipLaunchKernelGGL((ftk::adam_tile_kernel<GT, HT, decltype(has_ctl)::value, decltype(has_hyper)::value>),
                                   dim3(static_cast<unsigned>(blocks)), dim3(ftk::kWave), lds, stream, a,
                                   static_cast<uint64_t>(tile0));
            };
            if (ctl && hyper)
                launch(std::true_type{}, std::true_type{});
            else if (ctl)
                launch(std::true_type{}, std::false_type{});
            else if (hyper)
                launch(std::false_type{}, std::true_type{});
            else
                launch(std::false_type{}, std::false_type{});
            FT_HIP(hipGetLastError());
        }
    }
    int rc = scalar_part(0, head);
    if (rc != FT_OK) return rc;
    return scalar_part(head + body, n - head - body);
}

template <int GT>
int launch_g(const ftk::AdamConsts& c, float* p, const void* g, float* m, float* v, void* h, int half_dtype,
             size_t n, const ft_step_control_t* ctl, hipStream_t stream, OutPtrs out, const ftk::AdamConsts* hyper)
{
    if (h == nullptr) return launch_typed<GT, -1>(c, p, g, m, v, nullptr, n, ctl, stream, out, hyper);
    if (half_dtype == FT_F16) return launch_typed<GT, FT_F16>(c, p, g, m, v, h, n, ctl, stream, out, hyper);
    return launch_typed<GT, FT_BF16>(c, p, g, m, v, h, n, ctl, stream, out, hyper);
}

}  // namespace

int launch_adam(const ftk::AdamConsts& c, float* p, const void* g, int g_dtype, float* m, float* v,
                void* half_out, int half_dtype, size_t n, const ft_step_control_t* ctl, hipStream_t stream,
                float* p_out, float* m_out, float* v_out, const ftk::AdamConsts* hyper)
{
    if (n == 0) return FT_OK;
    if (!p || !g || !m || !v) return fail(FT_EINVAL, "params, grads, exp_avg and exp_avg_sq must not be NULL");
    if (!valid_dtype(g_dtype)) return fail(FT_EINVAL, "unknown gradient dtype code %d", g_dtype);
    if (half_out && half_dtype != FT_F16 && half_dtype != FT_BF16)
        return fail(FT_EINVAL, "low-precision copy must be FT_F16 or FT_BF16, got %d", half_dtype);
    if (!aligned(p, 4) || !aligned(m, 4) || !aligned(v, 4) || !aligned(g, elem_size(g_dtype)) ||
        (half_out && !aligned(half_out, 2)))
        return fail(FT_EALIGN, "a pointer is not aligned to its element size");
    if (ctl && !aligned(ctl, 16)) return fail(FT_EALIGN, "ft_step_control_t must be 16-byte aligned");
    if (hyper && !aligned(hyper, 16)) return fail(FT_EALIGN, "ft_adam_hyper_t must be 16-byte aligned");
    const OutPtrs out{p_out ? p_out : p, m_out ? m_out : m, v_out ? v_out : v};
    if (!aligned(out.p, 4) || !aligned(out.m, 4) || !aligned(out.v, 4))
        return fail(FT_EALIGN, "an output pointer is not aligned to its element size");
    switch (g_dtype) {
        case FT_F32: return launch_g<FT_F32>(c, p, g, m, v, half_out, half_dtype, n, ctl, stream, out, hyper);
        case FT_F16: return launch_g<FT_F16>(c, p, g, m, v, half_out, half_dtype, n, ctl, stream, out, hyper);
        default: return launch_g<FT_BF16>(c, p, g, m, v, half_out, half_dtype, n, ctl, stream, out, hyper);
    }
}

namespace {

template <int GT, int HT>
void launch_multi_typed(const ftk::AdamMultiArgs& a, bool with_hyper, unsigned workgroups, unsigned lds, hipStream_t stream)
{
    auto launch = [&](auto has_ctl, auto has_hyper) {
        hipLaunchKernelGGL((ftk::adam_multi_kernel<GT, HT, decltype(has_ctl)::value, decltype(has_hyper)::value>),
                           dim3(workgroups), dim3(ftk::kWave), lds, stream, a);
    };
    if (a.ctl && with_hyper)
        launch(std::true_type{}, std::true_type{});
    else if (a.ctl)
        launch(std::true_type{}, std::false_type{});
    else if (with_hyper)
        launch(std::false_type{}, std::true_type{});
    else
        launch(std::false_type{}, std::false_type{});
}

template <int GT>
void launch_multi_g(const ftk::AdamMultiArgs& a, bool with_half, int half_dtype, bool with_hyper, unsigned workgroups,
                    hipStream_t stream)
{
    const unsigned lds = throttle_lds_bytes(48 + 4 * (GT == FT_F32 ? 4u : 2u));
    if (!with_half) return launch_multi_typed<GT, -1>(a, with_hyper, workgroups, lds, stream);
    if (half_dtype == FT_F16) return launch_multi_typed<GT, FT_F16>(a, with_hyper, workgroups, lds, stream);
    return launch_multi_typed<GT, FT_BF16>(a, with_hyper, workgroups, lds, stream);
}

}  // namespace

// One launch over the segments collected in `a` (count of them, total workgroups). with_hyper: every
// segment's scalars are read from its device record (all of them or none: two kernel variants).
int launch_adam_multi(const ftk::AdamMultiArgs& a, int g_dtype, bool with_half, int half_dtype, bool with_hyper,
                      unsigned workgroups, hipStream_t stream)
{
    if (workgroups == 0) return FT_OK;
    switch (g_dtype) {
        case FT_F32: launch_multi_g<FT_F32>(a, with_half, half_dtype, with_hyper, workgroups, stream); break;
        case FT_F16: launch_multi_g<FT_F16>(a, with_half, half_dtype, with_hyper, workgroups, stream); break;
        default: launch_multi_g<FT_BF16>(a, with_half, half_dtype, with_hyper, workgroups, stream); break;
    }
    FT_HIP(hipGetLastError());
    return FT_OK;
}

}  // namespace fth

// ================================================================================================
// C ABI
// ================================================================================================
extern "C" size_t ft_grad_stats_workspace_bytes(void);

namespace {

// The caller's scratch if given (checked against `need` bytes), else a buffer the library owns for
// this (device, stream), grown when a call needs more than it holds (hipFree waits for the device,
// so work still using the old buffer has finished before it goes away). Calls on one stream are
// ordered, so they may share a buffer; calls on different streams get different ones.
int resolve_stats_workspace(void* workspace, size_t workspace_bytes, size_t need, hipStream_t stream, ftk::StatsPartial** out)
{
    ftk::StatsPartial* parts = static_cast<ftk::StatsPartial*>(workspace);
    if (parts) {
        if (workspace_bytes < need)
            return fth::fail(FT_EINVAL, "workspace of %zu bytes is smaller than the %zu bytes this call needs",
                             workspace_bytes, need);
        if (!aligned(parts, 16)) return fth::fail(FT_EALIGN, "workspace must be 16-byte aligned");
    } else {
        int dev = 0;
        FT_HIP(hipGetDevice(&dev));
        std::lock_guard<std::mutex> lk(g_mu);
        StreamState& own = g_stream_state[std::make_pair(dev, stream)];
        if (own.bytes < need) {
            if (own.ptr) FT_HIP(hipFree(own.ptr));
            own.ptr = nullptr;
            own.bytes = 0;
            void* w = nullptr;
            hipError_t e = hipMalloc(&w, need);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return fth::fail(FT_ENOMEM, "hipMalloc(%zu) for the statistics scratch failed: %s", need, hipGetErrorString(e));
            }
            own.ptr = w;
            own.bytes = need;
        }
        parts = static_cast<ftk::StatsPartial*>(own.ptr);
    }
    *out = parts;
    return FT_OK;
}

// Ticket counters of the one-launch statistics pass: part of the loaded code object, so zero when
// the library is loaded, and every pass leaves its counter at zero again. In host code the array's
// name is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) uint32_t g_ticket_pool[kTicketSlots * kTicketStride];
std::unordered_map<int, uint32_t*> g_ticket_pool_ptr;  // device -> that device's copy of the pool

// The ticket counter of (current device, stream), or nullptr when the pass has to take two launches:
// a stream under graph capture (the recorded kernel would be replayed on whatever stream the graph is
// launched on, beside eager passes that own this counter), or no counter left.
int stream_ticket(hipStream_t stream, uint32_t** out, uint32_t* tag)
{
    *out = nullptr;
    *tag = 0;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
        (void)hipGetLastError();
        return FT_OK;
    }
    if (capture != hipStreamCaptureStatusNone) return FT_OK;
    int dev = 0;
    FT_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_mu);
    auto pool = g_ticket_pool_ptr.find(dev);
    if (pool == g_ticket_pool_ptr.end()) {
        void* ptr = nullptr;
        FT_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_ticket_pool)));
        if (!ptr) return fth::fail(FT_EHIP, "hipGetSymbolAddress returned a null address for the ticket counters");
        pool = g_ticket_pool_ptr.emplace(dev, static_cast<uint32_t*>(ptr)).first;
        std::vector<int>& free_slots = g_free_ticket_slots[dev];
        for (int k = kTicketSlots - 1; k >= 0; --k) free_slots.push_back(k);
    }
    StreamState& st = g_stream_state[std::make_pair(dev, stream)];
    if (st.ticket_slot < 0) {
        std::vector<int>& free_slots = g_free_ticket_slots[dev];
        if (free_slots.empty()) return FT_OK;
        st.ticket_slot = free_slots.back();
        free_slots.pop_back();
    }
    *out = pool->second + static_cast<size_t>(st.ticket_slot) * kTicketStride;
    st.tag = st.tag % 0xffffu + 1;  // 1 ... 65535, a new one for every pass on this stream
    *tag = st.tag;
    return FT_OK;
}

constexpr int kReduceBlocks = 256;  // second-level blocks of the accumulation pass's statistics

// A decision to take in the last launch of a statistics pass (ctl == nullptr: none).
struct Decide {
    float inv_scale = 1.0f;
    float max_norm = 0.0f;
    ft_step_control_t* ctl = nullptr;
    const float* scale_dev = nullptr;  // 1/loss_scale in device memory: replaces pre_mult and inv_scale
};

// Statistics scratch of ft_grad_accumulate_static: block partials followed by one wavefront partial
// per 256 elements, for calls of up to FT_STATIC_MAX_ELEMS elements. It is part of the loaded code
// object, so every GPU the library runs on holds its own copy (16.1 MiB) until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress, never an address.
constexpr size_t kStaticScratchBytes =
    sizeof(ftk::StatsPartial) * kMaxStatsBlocks + (static_cast<size_t>(FT_STATIC_MAX_ELEMS) / 256 + 1) * sizeof(ftk::WavePartial);
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

std::unordered_map<int, void*> g_static_scratch_ptr;  // device -> that device's copy of the array

// The current device's address of the array; looked up once per device, with that device current.
int static_scratch(void** out)
{
    int dev = 0;
    FT_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_static_scratch_ptr.find(dev);
    if (it == g_static_scratch_ptr.end()) {
        void* ptr = nullptr;
        FT_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch)));
        if (!ptr) return fth::fail(FT_EHIP, "hipGetSymbolAddress returned a null address for the statistics scratch");
        it = g_static_scratch_ptr.emplace(dev, ptr).first;
    }
    *out = it->second;
    return FT_OK;
}

// Wavefront partials of the accumulation pass live behind the fixed block-partial area.
size_t accumulate_workspace_bytes(size_t n)
{
    const size_t waves = (n / 4 + 63) / 64;
    return ft_grad_stats_workspace_bytes() + waves * sizeof(ftk::WavePartial);
}

template <int AT, int GT, bool ZERO, bool STATS>
int launch_accumulate(void* acc, void* g, size_t n, size_t head, size_t nvec, bool g_relaxed, float scale, float pre_mult,
                      ftk::StatsPartial* parts, ft_grad_stats_t* stats_out, int stats_accumulate, const Decide& dec, hipStream_t stream)
{
    constexpr size_t asz = (AT == FT_F32) ? 4 : 2, gsz = (GT == FT_F32) ? 4 : 2;
    int reduce_blocks = 0;
    if (nvec > 0) {
        // Like the update: one tile per wavefront-sized workgroup, residency throttled through
        // dynamic LDS so that the bytes in flight per compute unit stay at the tuned level.
        // (the kernel's workgroups stride over the tiles, so a grid capped at what one launch may
        // hold still covers them all)
        size_t waves = (nvec + 63) / 64;
        if (waves > launch_limit()) waves = static_cast<size_t>(launch_limit());
        // A pass that ends in a decision is followed by the update, which reads the accumulator as
        // its gradients: the last stats_keep_bytes of it are stored with the default cache policy so
        // that the update finds them in the memory-side cache (everything else streams).
        uint64_t keep_from = ~0ull;
        if (dec.ctl) {
            const size_t tiles = (nvec + 63) / 64, keep_tiles = g_stats_keep_bytes.load() / (64 * 4 * asz);
            keep_from = tiles > keep_tiles ? tiles - keep_tiles : 0;
        }
        ftk::WavePartial* wave_parts =
            STATS ? reinterpret_cast<ftk::WavePartial*>(reinterpret_cast<char*>(parts) + ft_grad_stats_workspace_bytes())
                  : nullptr;
        // Measured on the 7B-layer partition, fp32 accumulator and 16-bit gradients: the variant that
        // also clears the source (as many bytes stored as loaded) is fastest with three quarters of the
        // wavefronts the rule gives (20 per CU: 351 us; 26: 357 us; 16: 353 us), the other variants with all.
        constexpr unsigned percent = (ZERO && !STATS && AT == FT_F32 && GT != FT_F32) ? 75u : 100u;
        hipLaunchKernelGGL((ftk::grad_accumulate_kernel<AT, GT, ZERO, STATS>), dim3(static_cast<unsigned>(waves)), dim3(64),
                           fth::throttle_lds_bytes(4 * static_cast<unsigned>(asz + gsz), percent), stream,
                           static_cast<void*>(static_cast<char*>(acc) + head * asz),
                           static_cast<void*>(static_cast<char*>(g) + head * gsz), static_cast<uint64_t>(nvec), scale,
                           pre_mult, wave_parts, keep_from, g_relaxed ? 1 : 0);
        FT_HIP(hipGetLastError());
        if (STATS) {
            reduce_blocks = waves < static_cast<size_t>(kReduceBlocks) ? static_cast<int>(waves) : kReduceBlocks;
            const uint64_t per_block = (waves + reduce_blocks - 1) / reduce_blocks;
            hipLaunchKernelGGL(ftk::reduce_wave_partials_kernel, dim3(reduce_blocks), dim3(256), 0, stream, wave_parts,
                               static_cast<uint64_t>(waves), per_block, parts);
            FT_HIP(hipGetLastError());
        }
    }
    // Edge elements and, with statistics, the sum of the second-level partials: one small launch.
    const size_t tail_begin = head + nvec * 4;
    if (STATS || head > 0 || tail_begin < n) {
        hipLaunchKernelGGL((ftk::grad_accumulate_finish_kernel<AT, GT, ZERO, STATS>), dim3(1), dim3(256), 0, stream, acc, g,
                           static_cast<uint64_t>(head), static_cast<uint64_t>(tail_begin), static_cast<uint64_t>(n),
                           scale, pre_mult, static_cast<const ftk::StatsPartial*>(parts), reduce_blocks, stats_out,
                           stats_accumulate, dec.inv_scale, dec.max_norm, dec.ctl);
        FT_HIP(hipGetLastError());
    }
    return FT_OK;
}

template <int AT, int GT>
int launch_accumulate_flags(bool zero, bool stats, void* acc, void* g, size_t n, size_t head, size_t nvec, bool g_relaxed, float scale,
                            float pre_mult, ftk::StatsPartial* parts, ft_grad_stats_t* stats_out, int stats_accumulate, const Decide& dec, hipStream_t stream)
{
    if (zero && stats) return launch_accumulate<AT, GT, true, true>(acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
    if (zero) return launch_accumulate<AT, GT, true, false>(acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
    if (stats) return launch_accumulate<AT, GT, false, true>(acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
    return launch_accumulate<AT, GT, false, false>(acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
}

template <int AT>
int launch_accumulate_g(int g_dtype, bool zero, bool stats, void* acc, void* g, size_t n, size_t head, size_t nvec, bool g_relaxed,
                        float scale, float pre_mult, ftk::StatsPartial* parts, ft_grad_stats_t* stats_out, int stats_accumulate, const Decide& dec, hipStream_t stream)
{
    switch (g_dtype) {
        case FT_F32: return launch_accumulate_flags<AT, FT_F32>(zero, stats, acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
        case FT_F16: return launch_accumulate_flags<AT, FT_F16>(zero, stats, acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
        default: return launch_accumulate_flags<AT, FT_BF16>(zero, stats, acc, g, n, head, nvec, g_relaxed, scale, pre_mult, parts, stats_out, stats_accumulate, dec, stream);
    }
}

}  // namespace

extern "C" {

const char* ft_last_error(void) { return t_last_error.c_str(); }

int ft_abi_version(void) { return 3; }

int ft_device_count(void)
{
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fth::fail(FT_EHIP, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
    }
    return n;
}

int ft_adam_create(int id, float lr, float beta1, float beta2, float eps, float weight_decay, int adamw_mode,
                   int should_log)
{
    fth::AdamObject o{lr, beta1, beta2, eps, weight_decay, adamw_mode != 0};
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_adams[id] = o;
    }
    if (should_log) {
        printf("Adam Optimizer #%d is created with gfx950 HIP arithmetic capability.\n", id);
        printf("Config: alpha=%f, betas=(%f, %f), weight_decay=%f, adam_w=%d\n", lr, beta1, beta2, weight_decay,
               adamw_mode != 0);
        fflush(stdout);
    }
    return FT_OK;
}

int ft_adam_destroy(int id)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_adams.erase(id);
    return FT_OK;
}

int ft_adam_step(int id, uint64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                 int bias_correction, float grad_mult, void* p, const void* g, int g_dtype, void* m, void* v,
                 void* half_out, int half_dtype, size_t n, const void* ctl, void* stream)
{
    fth::AdamObject o;
    int rc = fth::find_adam(id, &o);
    if (rc != FT_OK) return rc;
    const ftk::AdamConsts c =
        fth::make_consts(step, lr, beta1, beta2, eps, weight_decay, bias_correction != 0, o.adamw_mode, grad_mult);
    return fth::launch_adam(c, static_cast<float*>(p), g, g_dtype, static_cast<float*>(m), static_cast<float*>(v),
                            half_out, half_dtype, n, static_cast<const ft_step_control_t*>(ctl),
                            static_cast<hipStream_t>(stream));
}

int ft_adam_hyper_fill(int id, uint64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                       int bias_correction, float grad_mult, ft_adam_hyper_t* out)
{
    static_assert(sizeof(ftk::AdamConsts) <= sizeof(ft_adam_hyper_t), "the public record must hold the kernels' scalars");
    if (!out) return fth::fail(FT_EINVAL, "out must not be NULL");
    fth::AdamObject o;
    int rc = fth::find_adam(id, &o);
    if (rc != FT_OK) return rc;
    const ftk::AdamConsts c =
        fth::make_consts(step, lr, beta1, beta2, eps, weight_decay, bias_correction != 0, o.adamw_mode, grad_mult);
    memset(out, 0, sizeof *out);
    memcpy(out, &c, sizeof c);
    return FT_OK;
}

int ft_adam_step_hyper(int id, const void* hyper_dev, void* p, const void* g, int g_dtype, void* m, void* v, void* half_out,
                       int half_dtype, size_t n, const void* ctl, void* stream)
{
    fth::AdamObject o;
    int rc = fth::find_adam(id, &o);
    if (rc != FT_OK) return rc;
    if (!hyper_dev) return fth::fail(FT_EINVAL, "hyper_dev must not be NULL");
    ftk::AdamConsts unused{};  // every scalar comes from the device record
    return fth::launch_adam(unused, static_cast<float*>(p), g, g_dtype, static_cast<float*>(m), static_cast<float*>(v), half_out,
                            half_dtype, n, static_cast<const ft_step_control_t*>(ctl), static_cast<hipStream_t>(stream), nullptr,
                            nullptr, nullptr, static_cast<const ftk::AdamConsts*>(hyper_dev));
}

int ft_adam_step_multi(int id, const ft_adam_segment_t* segs, int n_segs, int g_dtype, int half_dtype,
                       const void* ctl_, void* stream_)
{
    fth::AdamObject o;
    int rc = fth::find_adam(id, &o);
    if (rc != FT_OK) return rc;
    if (n_segs < 0 || (n_segs > 0 && !segs)) return fth::fail(FT_EINVAL, "segs must not be NULL and n_segs not negative");
    if (!valid_dtype(g_dtype)) return fth::fail(FT_EINVAL, "unknown gradient dtype code %d", g_dtype);
    const ft_step_control_t* ctl = static_cast<const ft_step_control_t*>(ctl_);
    if (ctl && !aligned(ctl, 16)) return fth::fail(FT_EALIGN, "ft_step_control_t must be 16-byte aligned");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const size_t gsz = elem_size(g_dtype);
    // Everything is checked before anything is launched: a bad segment must not leave half a step behind.
    for (int i = 0; i < n_segs; ++i) {
        const ft_adam_segment_t& sg = segs[i];
        if (sg.n == 0) continue;
        if (!sg.p || !sg.g || !sg.m || !sg.v)
            return fth::fail(FT_EINVAL, "segment %d: params, grads, exp_avg and exp_avg_sq must not be NULL", i);
        if (sg.half_out && half_dtype != FT_F16 && half_dtype != FT_BF16)
            return fth::fail(FT_EINVAL, "low-precision copy must be FT_F16 or FT_BF16, got %d", half_dtype);
        if (!aligned(sg.p, 4) || !aligned(sg.m, 4) || !aligned(sg.v, 4) || !aligned(sg.g, gsz) ||
            (sg.half_out && !aligned(sg.half_out, 2)))
            return fth::fail(FT_EALIGN, "segment %d: a pointer is not aligned to its element size", i);
        if (sg.hyper && !aligned(sg.hyper, 16)) return fth::fail(FT_EALIGN, "segment %d: ft_adam_hyper_t must be 16-byte aligned", i);
    }
    // Four batches fill side by side (with and without a low-precision copy, scalars by value or from
    // a device record: four kernel variants); a batch is launched when it holds kMultiMaxSegments
    // segments or its grid is full.
    struct Batch {
        ftk::AdamMultiArgs a;
        int count = 0;
        unsigned workgroups = 0;
    } batch[4];
    auto flush = [&](int which) -> int {
        Batch& b = batch[which];
        if (b.count == 0) return FT_OK;
        for (int k = b.count; k < ftk::kMultiMaxSegments; ++k) b.a.first_wg[k] = 0xffffffffu;
        b.a.ctl = ctl;
        const int r = fth::launch_adam_multi(b.a, g_dtype, (which & 1) != 0, half_dtype, (which & 2) != 0, b.workgroups, stream);
        b.count = 0;
        b.workgroups = 0;
        return r;
    };
    for (int i = 0; i < n_segs; ++i) {
        const ft_adam_segment_t& sg = segs[i];
        if (sg.n == 0) continue;
        const ftk::AdamConsts c = fth::make_consts(sg.step, sg.lr, sg.beta1, sg.beta2, sg.eps, sg.weight_decay,
                                                   sg.bias_correction != 0, o.adamw_mode, sg.grad_mult);
        float* p = static_cast<float*>(sg.p);
        char* mb = static_cast<char*>(sg.m);
        char* vb = static_cast<char*>(sg.v);
        const char* gb = static_cast<const char*>(sg.g);
        char* hb = static_cast<char*>(sg.half_out);
        const size_t head = fth::segment_head(p, sg.n);
        const bool vec_ok = aligned(mb + head * 4, 16) && aligned(vb + head * 4, 16) && aligned(gb + head * gsz, gsz * 4) &&
                            (!hb || aligned(hb + head * 2, 8));
        const size_t body_tiles = (sg.n - head) / (ftk::kWave * 4);
        const bool edge = head + (sg.n - head) % (ftk::kWave * 4) > 0;
        if (!vec_ok || !arrays_on_lines(head, sg.n, p, mb, vb, gb, gsz, hb, p, mb, vb) || body_tiles + 1 > multi_launch_limit()) {
            // arrays whose alignments disagree (as vectors or on cache lines), or a segment too long
            // for one grid: the single-segment path takes it
            rc = fth::launch_adam(c, p, sg.g, g_dtype, static_cast<float*>(sg.m), static_cast<float*>(sg.v), sg.half_out,
                                  half_dtype, sg.n, ctl, stream, nullptr, nullptr, nullptr,
                                  static_cast<const ftk::AdamConsts*>(sg.hyper));
            if (rc != FT_OK) return rc;
            continue;
        }
        const int which = (sg.half_out ? 1 : 0) | (sg.hyper ? 2 : 0);
        const unsigned wgs = static_cast<unsigned>(body_tiles) + (edge ? 1u : 0u);
        if (fth::segment_batch_is_full(batch[which].count, batch[which].workgroups, wgs, ftk::kMultiMaxSegments, multi_launch_limit()))
            if ((rc = flush(which)) != FT_OK) return rc;
        Batch& b = batch[which];
        ftk::AdamSegment& d = b.a.seg[b.count];
        d.p = p;
        d.g = sg.g;
        d.m = static_cast<float*>(sg.m);
        d.v = static_cast<float*>(sg.v);
        d.h = sg.half_out;
        d.n = sg.n;
        d.head = static_cast<uint32_t>(head);
        d.body_tiles = static_cast<uint32_t>(body_tiles);
        d.hyper = static_cast<const ftk::AdamConsts*>(sg.hyper);
        d.c = c;
        b.a.first_wg[b.count] = (b.workgroups << 4) | static_cast<unsigned>(b.count);
        b.workgroups += wgs;
        ++b.count;
    }
    for (int which = 0; which < 4; ++which)
        if ((rc = flush(which)) != FT_OK) return rc;
    return FT_OK;
}

size_t ft_grad_stats_workspace_bytes(void) { return sizeof(ftk::StatsPartial) * kMaxStatsBlocks; }

size_t ft_grad_accumulate_workspace_bytes(size_t n) { return accumulate_workspace_bytes(n); }

}  // extern "C"

namespace {

int grad_stats_impl(const void* g, int g_dtype, size_t n, float pre_mult, void* out, int accumulate, void* workspace,
                    size_t workspace_bytes, const Decide& dec, void* stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!out) return fth::fail(FT_EINVAL, "out must not be NULL");
    if (!aligned(out, 16)) return fth::fail(FT_EALIGN, "ft_grad_stats_t must be 16-byte aligned");
    if (!valid_dtype(g_dtype)) return fth::fail(FT_EINVAL, "unknown gradient dtype code %d", g_dtype);
    if (n > 0 && !g) return fth::fail(FT_EINVAL, "g must not be NULL");
    if (n > 0 && !aligned(g, elem_size(g_dtype))) return fth::fail(FT_EALIGN, "g is not aligned to its element size");

    ftk::StatsPartial* parts = nullptr;
    int wrc = resolve_stats_workspace(workspace, workspace_bytes, ft_grad_stats_workspace_bytes(), stream, &parts);
    if (wrc != FT_OK) return wrc;

    const size_t esz = elem_size(g_dtype);
    const size_t per_unit = 16 / esz;
    size_t head = 0;
    if (n > 0) {
        head = ((16 - (reinterpret_cast<uintptr_t>(g) & 15)) & 15) / esz;
        if (head > n) head = n;
    }
    const size_t nvec = (n - head) / per_unit;
    const size_t tail_begin = head + nvec * per_unit;
    ftk::StatsFinalArgs fin;
    fin.g = g;
    fin.head = head;
    fin.tail_begin = tail_begin;
    fin.n = n;
    fin.out = static_cast<ft_grad_stats_t*>(out);
    fin.accumulate = accumulate;
    fin.inv_scale = dec.inv_scale;
    fin.max_norm = dec.max_norm;
    fin.ctl = dec.ctl;
    fin.ticket = nullptr;
    fin.tag = 0;
    int blocks = 0;
    if (nvec > 0) {
        constexpr size_t kTile = static_cast<size_t>(FT_STATS_BLOCK) * FT_STATS_UNROLL;
        size_t b = (nvec + kTile - 1) / kTile;
        size_t cap = static_cast<size_t>(fth::cu_count()) * static_cast<size_t>(g_stats_blocks_per_cu.load());
        if (cap > static_cast<size_t>(kMaxStatsBlocks)) cap = kMaxStatsBlocks;
        if (b > cap) b = cap;
        blocks = static_cast<int>(b);
        // One launch where the stream has a ticket counter of its own: the block that delivers the
        // last partial also takes the final sum (and the decision).
        if (g_stats_one_launch.load()) {
            int trc = stream_ticket(stream, &fin.ticket, &fin.tag);
            if (trc != FT_OK) return trc;
        }
        const ftk::u32x4* gv = reinterpret_cast<const ftk::u32x4*>(static_cast<const char*>(g) + head * esz);
        const size_t ntiles = (nvec + kTile - 1) / kTile, keep_tiles = g_stats_keep_bytes.load() / (kTile * 16);
        const uint64_t keep_from = ntiles > keep_tiles ? ntiles - keep_tiles : 0;
        switch (g_dtype) {
            case FT_F32:
                hipLaunchKernelGGL((ftk::grad_stats_kernel<FT_F32, FT_STATS_BLOCK, FT_STATS_UNROLL>), dim3(blocks),
                                   dim3(FT_STATS_BLOCK), 0, stream, gv, nvec, pre_mult, parts, keep_from, dec.scale_dev, fin);
                break;
            case FT_F16:
                hipLaunchKernelGGL((ftk::grad_stats_kernel<FT_F16, FT_STATS_BLOCK, FT_STATS_UNROLL>), dim3(blocks),
                                   dim3(FT_STATS_BLOCK), 0, stream, gv, nvec, pre_mult, parts, keep_from, dec.scale_dev, fin);
                break;
            default:
                hipLaunchKernelGGL((ftk::grad_stats_kernel<FT_BF16, FT_STATS_BLOCK, FT_STATS_UNROLL>), dim3(blocks),
                                   dim3(FT_STATS_BLOCK), 0, stream, gv, nvec, pre_mult, parts, keep_from, dec.scale_dev, fin);
                break;
        }
        FT_HIP(hipGetLastError());
        if (fin.ticket) return FT_OK;
    }
    switch (g_dtype) {
        case FT_F32:
            hipLaunchKernelGGL((ftk::grad_stats_final_kernel<FT_F32>), dim3(1), dim3(256), 0, stream, parts, blocks, pre_mult,
                               dec.scale_dev, fin);
            break;
        case FT_F16:
            hipLaunchKernelGGL((ftk::grad_stats_final_kernel<FT_F16>), dim3(1), dim3(256), 0, stream, parts, blocks, pre_mult,
                               dec.scale_dev, fin);
            break;
        default:
            hipLaunchKernelGGL((ftk::grad_stats_final_kernel<FT_BF16>), dim3(1), dim3(256), 0, stream, parts, blocks, pre_mult,
                               dec.scale_dev, fin);
            break;
    }
    FT_HIP(hipGetLastError());
    return FT_OK;
}

}  // namespace

extern "C" {

int ft_grad_stats(const void* g, int g_dtype, size_t n, float pre_mult, void* out, int accumulate, void* workspace,
                  size_t workspace_bytes, void* stream)
{
    return grad_stats_impl(g, g_dtype, n, pre_mult, out, accumulate, workspace, workspace_bytes, Decide{}, stream);
}

int ft_grad_decide(const void* g, int g_dtype, size_t n, float pre_mult, void* stats, int accumulate, float inv_scale,
                   float max_norm, void* ctl_out, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!ctl_out) return fth::fail(FT_EINVAL, "ctl_out must not be NULL");
    if (!aligned(ctl_out, 16)) return fth::fail(FT_EALIGN, "ft_step_control_t must be 16-byte aligned");
    Decide dec;
    dec.inv_scale = inv_scale;
    dec.max_norm = max_norm;
    dec.ctl = static_cast<ft_step_control_t*>(ctl_out);
    return grad_stats_impl(g, g_dtype, n, pre_mult, stats, accumulate, workspace, workspace_bytes, dec, stream);
}

int ft_grad_decide_dev(const void* g, int g_dtype, size_t n, const void* inv_scale_dev, void* stats, int accumulate,
                       float max_norm, void* ctl_out, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!ctl_out || !inv_scale_dev) return fth::fail(FT_EINVAL, "ctl_out and inv_scale_dev must not be NULL");
    if (!aligned(ctl_out, 16)) return fth::fail(FT_EALIGN, "ft_step_control_t must be 16-byte aligned");
    if (!aligned(inv_scale_dev, 4)) return fth::fail(FT_EALIGN, "inv_scale_dev must be 4-byte aligned");
    Decide dec;
    dec.max_norm = max_norm;
    dec.ctl = static_cast<ft_step_control_t*>(ctl_out);
    dec.scale_dev = static_cast<const float*>(inv_scale_dev);
    return grad_stats_impl(g, g_dtype, n, 1.0f, stats, accumulate, workspace, workspace_bytes, dec, stream);
}

}  // extern "C"

namespace {

// static_scratch_only: the statistics scratch is the library's static device array (nothing is
// allocated); otherwise the caller's workspace, or the library-owned buffer when that is NULL.
int grad_accumulate_impl(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                         float stats_pre_mult, void* stats_out, int stats_accumulate, void* workspace,
                         size_t workspace_bytes, bool static_scratch_only, const Decide& dec, void* stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!valid_dtype(acc_dtype) || !valid_dtype(g_dtype))
        return fth::fail(FT_EINVAL, "unknown dtype code (acc %d, g %d)", acc_dtype, g_dtype);
    if (stats_out && !aligned(stats_out, 16)) return fth::fail(FT_EALIGN, "ft_grad_stats_t must be 16-byte aligned");
    const bool stats = stats_out != nullptr;
    if (n > 0 && (!acc || !g)) return fth::fail(FT_EINVAL, "acc and g must not be NULL");
    const size_t asz = elem_size(acc_dtype), gsz = elem_size(g_dtype);
    size_t head = 0, nvec = 0;
    bool g_relaxed = false;
    if (n > 0) {
        if (!aligned(acc, asz) || !aligned(g, gsz)) return fth::fail(FT_EALIGN, "a pointer is not aligned to its element size");
        head = ((asz * 4 - (reinterpret_cast<uintptr_t>(acc) & (asz * 4 - 1))) & (asz * 4 - 1)) / asz;
        if (head > n) head = n;  // shorter than the way to the first boundary: edge elements only
        // g off its vector alignment where acc reaches its own: the kernel then reads (and clears) g
        // through accesses that assume element alignment only
        g_relaxed = head < n && !aligned(static_cast<char*>(g) + head * gsz, gsz * 4);
        // A long buffer: on to the first tile boundary of acc (256 elements = 1 KiB of fp32), so that
        // every tile's streaming stores cover whole cache lines (a multiple of 4 more: g stays aligned).
        if (n - head >= 16 * 256) {
            const size_t tile_bytes = 256 * asz;
            head = ((tile_bytes - (reinterpret_cast<uintptr_t>(acc) & (tile_bytes - 1))) & (tile_bytes - 1)) / asz;
            // ... and g aligned as vectors but off the cache lines there is treated like g off its
            // vector alignment: its tiles share lines with their neighbours all the same
            if (!aligned(static_cast<char*>(g) + head * gsz, fth::kLineBytes)) g_relaxed = true;
        }
        nvec = (n - head) / 4;
    }
    ftk::StatsPartial* parts = nullptr;
    if (stats && static_scratch_only) {
        void* ptr = nullptr;
        int wrc = static_scratch(&ptr);
        if (wrc != FT_OK) return wrc;
        parts = static_cast<ftk::StatsPartial*>(ptr);
    } else if (stats) {
        int wrc = resolve_stats_workspace(workspace, workspace_bytes, accumulate_workspace_bytes(n), stream, &parts);
        if (wrc != FT_OK) return wrc;
    }
    ft_grad_stats_t* out = static_cast<ft_grad_stats_t*>(stats_out);
    switch (acc_dtype) {
        case FT_F32: return launch_accumulate_g<FT_F32>(g_dtype, zero_g != 0, stats, acc, g, n, head, nvec, g_relaxed, scale, stats_pre_mult, parts, out, stats_accumulate, dec, stream);
        case FT_F16: return launch_accumulate_g<FT_F16>(g_dtype, zero_g != 0, stats, acc, g, n, head, nvec, g_relaxed, scale, stats_pre_mult, parts, out, stats_accumulate, dec, stream);
        default: return launch_accumulate_g<FT_BF16>(g_dtype, zero_g != 0, stats, acc, g, n, head, nvec, g_relaxed, scale, stats_pre_mult, parts, out, stats_accumulate, dec, stream);
    }
}

}  // namespace

extern "C" {

int ft_grad_accumulate(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                       float stats_pre_mult, void* stats_out, int stats_accumulate, void* workspace,
                       size_t workspace_bytes, void* stream)
{
    return grad_accumulate_impl(acc, acc_dtype, g, g_dtype, n, scale, zero_g, stats_pre_mult, stats_out, stats_accumulate,
                                workspace, workspace_bytes, false, Decide{}, stream);
}

int ft_grad_accumulate_decide(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                              float stats_pre_mult, void* stats, int stats_accumulate, float inv_scale, float max_norm,
                              void* ctl_out, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!stats || !ctl_out) return fth::fail(FT_EINVAL, "stats and ctl_out must not be NULL");
    if (!aligned(ctl_out, 16)) return fth::fail(FT_EALIGN, "ft_step_control_t must be 16-byte aligned");
    Decide dec;
    dec.inv_scale = inv_scale;
    dec.max_norm = max_norm;
    dec.ctl = static_cast<ft_step_control_t*>(ctl_out);
    return grad_accumulate_impl(acc, acc_dtype, g, g_dtype, n, scale, zero_g, stats_pre_mult, stats, stats_accumulate,
                                workspace, workspace_bytes, false, dec, stream);
}

int ft_grad_accumulate_static(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                              float stats_pre_mult, void* stats_out, int stats_accumulate, void* stream)
{
    if (n > static_cast<size_t>(FT_STATIC_MAX_ELEMS))
        return fth::fail(FT_EINVAL, "ft_grad_accumulate_static takes at most %llu elements per call, got %zu "
                         "(use ft_grad_accumulate with a workspace for longer buffers)",
                         static_cast<unsigned long long>(FT_STATIC_MAX_ELEMS), n);
    return grad_accumulate_impl(acc, acc_dtype, g, g_dtype, n, scale, zero_g, stats_pre_mult, stats_out, stats_accumulate,
                                nullptr, 0, true, Decide{}, stream);
}

int ft_grad_control(const void* stats, float inv_scale, float max_norm, void* ctl_out, void* stream)
{
    if (!stats || !ctl_out) return fth::fail(FT_EINVAL, "stats and ctl_out must not be NULL");
    if (!aligned(stats, 16) || !aligned(ctl_out, 16))
        return fth::fail(FT_EALIGN, "stats and ctl_out must be 16-byte aligned");
    hipLaunchKernelGGL(ftk::grad_control_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream),
                       static_cast<const ft_grad_stats_t*>(stats), inv_scale, max_norm,
                       static_cast<ft_step_control_t*>(ctl_out));
    FT_HIP(hipGetLastError());
    return FT_OK;
}

int ft_release_stream_scratch(void* stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int dev = 0;
    FT_HIP(hipGetDevice(&dev));
    FT_HIP(hipStreamSynchronize(stream));  // nothing enqueued there may still use the buffer or the counter
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_stream_state.find(std::make_pair(dev, stream));
    if (it == g_stream_state.end()) return FT_OK;
    if (it->second.ptr) FT_HIP(hipFree(it->second.ptr));
    if (it->second.ticket_slot >= 0) g_free_ticket_slots[dev].push_back(it->second.ticket_slot);
    g_stream_state.erase(it);
    return FT_OK;
}

int ft_set_launch_limit(uint64_t max_workgroups)
{
    if (max_workgroups > ftk::kMaxWorkgroupsPerLaunch)
        return fth::fail(FT_EINVAL, "a launch holds at most %llu workgroups of 64 lanes",
                         static_cast<unsigned long long>(ftk::kMaxWorkgroupsPerLaunch));
    g_launch_limit = max_workgroups == 0 ? ftk::kMaxWorkgroupsPerLaunch : max_workgroups;
    return FT_OK;
}

int ft_launch_pieces(uint64_t workgroups, uint64_t limit, uint64_t* first, uint64_t* count, int capacity)
{
    if (limit == 0) limit = g_launch_limit.load();
    const uint64_t pieces = fth::launch_piece_count(workgroups, limit);
    if (pieces > 0x7fffffffull) return fth::fail(FT_EINVAL, "more pieces than an int can count");
    for (uint64_t k = 0; k < pieces && static_cast<int64_t>(k) < capacity; ++k)
        if (!fth::plan_launch_piece(workgroups, limit, k, first + k, count + k)) return fth::fail(FT_EINVAL, "piece %llu missing", static_cast<unsigned long long>(k));
    return static_cast<int>(pieces);
}

int ft_segment_batches(const uint64_t* workgroups, int n_segs, uint64_t limit, int* batch_of)
{
    if (n_segs < 0 || (n_segs > 0 && (!workgroups || !batch_of))) return fth::fail(FT_EINVAL, "bad arguments");
    if (limit == 0) limit = multi_launch_limit();
    return fth::plan_segment_batches(workgroups, n_segs, ftk::kMultiMaxSegments, limit, batch_of);
}

int ft_relaxed_tile_start(const uint64_t* addresses, const uint32_t* elem_bytes, const uint32_t* weights, int count, uint32_t* on_lines)
{
    if (count < 1 || count > 32 || !addresses || !elem_bytes || !weights || !on_lines) return fth::fail(FT_EINVAL, "bad arguments");
    fth::ArrayPlacement place[32];
    for (int k = 0; k < count; ++k) {
        if (elem_bytes[k] != 2 && elem_bytes[k] != 4) return fth::fail(FT_EINVAL, "array %d: element size %u", k, elem_bytes[k]);
        place[k] = {addresses[k], elem_bytes[k], weights[k]};
    }
    return static_cast<int>(fth::plan_relaxed_head(place, count, on_lines));
}

int ft_set_stats_launches(int launches)
{
    if (launches != 1 && launches != 2) return fth::fail(FT_EINVAL, "a statistics pass takes 1 or 2 launches, not %d", launches);
    g_stats_one_launch = launches == 1 ? 1 : 0;
    return FT_OK;
}

int ft_set_cache_tuning(size_t stats_keep_bytes)
{
    g_stats_keep_bytes = stats_keep_bytes;
    return FT_OK;
}

int ft_set_launch_tuning(int adam_waves_per_cu, int stats_blocks_per_cu)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_adam_waves_per_cu = adam_waves_per_cu > 0 ? adam_waves_per_cu : FT_ADAM_WAVES_PER_CU;
    g_stats_blocks_per_cu = stats_blocks_per_cu > 0 ? stats_blocks_per_cu : FT_STATS_BLOCKS_PER_CU;
    return FT_OK;
}

}  // extern "C"
