// ft_ceiling -- the shipped kernels beside bare kernels of the same memory traffic.
//
// A bandwidth-bound kernel can be compared with a published peak, or with what the machine gives
// the same loads and stores when nothing else happens in the kernel. This program measures the
// second: for the update, the accumulation pass and the statistics pass on the Llama-7B decoder-layer
// partition it times the library's kernel (the same device code, compiled from the same header with
// the same flags) and a bare kernel of the same shape and traffic, in one process, on the same
// buffers, launch after launch (HIP events around every launch, fastest and median of 30), and
// prints one JSON object per line:
//   {"case": "...", "bytes": B, "bare_us": .., "shipped_us": .., "bare_median_us": .., "shipped_median_us": ..}
// No result of the library is checked here (the parity tests do that); nothing but timing.
//
//   hipcc --offload-arch=gfx950 -O3 ... -o flextrain_amd/ft_ceiling flextrain_amd/csrc/ft_ceiling.hip
//   ./flextrain_amd/ft_ceiling [elements]
#include "ft_kernels.hpp"

#include <stdio.h>
#include <stdlib.h>

#include <algorithm>
#include <vector>

using namespace ftk;

#define CK(x)                                                                  \
    do {                                                                       \
        hipError_t e_ = (x);                                                   \
        if (e_ != hipSuccess) {                                                \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));            \
            exit(1);                                                           \
        }                                                                      \
    } while (0)

namespace {

__global__ void fill_f32(float* p, uint64_t n, float scale)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = scale * (float)(((i * 2654435761u) & 1023u) + 1u) / 1024.f;
}
__global__ void fill_bf16(uint16_t* p, uint64_t n)  // finite values around 1e-3, both signs
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = (uint16_t)(0x3a80u ^ ((i * 2654435761u) & 0x807fu));
}

// ---- bare kernels: the traffic of the shipped ones and next to nothing else --------------------
// update: one 64-lane workgroup per 256-element tile; loads g (8 B per lane), p, m, v (16 B each),
// stores p, m, v and the 16-bit copy through the same streaming buffer stores
__global__ __launch_bounds__(kWave) void bare_update_kernel(float* p, const void* g, float* m, float* v, void* h)
{
    const uint64_t t0 = (uint64_t)blockIdx.x * kWave, i = t0 + threadIdx.x;
    const f32x4 gg = load_g4<FT_BF16, true>(g, i);
    f32x4 pp = ld<true>(reinterpret_cast<const f32x4*>(p) + i);
    f32x4 mm = ld<true>(reinterpret_cast<const f32x4*>(m) + i);
    f32x4 vv = ld<true>(reinterpret_cast<const f32x4*>(v) + i);
    pp += gg * 1e-3f;
    mm = mm * 0.9f + gg * 0.1f;
    vv = vv * 0.999f + gg * gg * 0.001f;
    st_stream(tile_rsrc(reinterpret_cast<f32x4*>(p) + t0, kWave * 16), threadIdx.x * 16, pp);
    st_stream(tile_rsrc(reinterpret_cast<f32x4*>(m) + t0, kWave * 16), threadIdx.x * 16, mm);
    st_stream(tile_rsrc(reinterpret_cast<f32x4*>(v) + t0, kWave * 16), threadIdx.x * 16, vv);
    u32x2 w;
    w.x = pack2<FT_BF16>(pp.x, pp.y);
    w.y = pack2<FT_BF16>(pp.z, pp.w);
    st_stream(tile_rsrc(reinterpret_cast<u32x2*>(h) + t0, kWave * 8), threadIdx.x * 8, w);
}

// accumulation: acc (fp32) += g (bf16), optionally clearing g
template <bool ZERO>
__global__ __launch_bounds__(kWave) void bare_accumulate_kernel(float* acc, void* g, float scale)
{
    const uint64_t t0 = (uint64_t)blockIdx.x * kWave, i = t0 + threadIdx.x;
    const f32x4 gg = load_g4<FT_BF16, true>(g, i);
    f32x4 a = ld<true>(reinterpret_cast<const f32x4*>(acc) + i);
    a.x = __builtin_fmaf(gg.x, scale, a.x);
    a.y = __builtin_fmaf(gg.y, scale, a.y);
    a.z = __builtin_fmaf(gg.z, scale, a.z);
    a.w = __builtin_fmaf(gg.w, scale, a.w);
    st_stream(tile_rsrc(reinterpret_cast<f32x4*>(acc) + t0, kWave * 16), threadIdx.x * 16, a);
    if constexpr (ZERO) {
        const u32x2 z = {0u, 0u};
        st_stream(tile_rsrc(reinterpret_cast<u32x2*>(g) + t0, kWave * 8), threadIdx.x * 8, z);
    }
}

// statistics: grid-stride blocks of 256 threads, 4 x 16-byte loads per lane; ARITHMETIC: squares in
// fp64 and one partial per block, else nothing but the loads
template <bool ARITHMETIC>
__global__ __launch_bounds__(256) void bare_read_kernel(const u32x4* g, uint64_t nvec, double* partials, uint32_t* sink)
{
    constexpr uint64_t kTile = 256 * 4;
    const uint64_t ntiles = nvec / kTile;
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    uint32_t seen = 0;
    for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const uint64_t base = tile * kTile + threadIdx.x;
        u32x4 w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) w[u] = __builtin_nontemporal_load(g + base + (uint64_t)u * 256);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if constexpr (ARITHMETIC)
                stats_accumulate_finite<FT_BF16>(w[u], 0.5f, acc);
            else
                seen |= w[u].x & w[u].y & w[u].z & w[u].w;
        }
    }
    if constexpr (ARITHMETIC) {
        double total;
        uint64_t bad;
        block_stats_reduce<256>((acc[0] + acc[1]) + (acc[2] + acc[3]), 0, total, bad);
        if (threadIdx.x == 0) partials[blockIdx.x] = total;
    } else {
        if (seen == 0xdeadbeefu) *sink = seen;  // never true for the data below: keeps the loads alive
    }
}

struct Timing {
    double fastest_us, median_us;
};

template <typename F>
Timing time_launches(F launch)
{
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    for (int i = 0; i < 3; ++i) launch();
    std::vector<float> t;
    for (int i = 0; i < 30; ++i) {
        CK(hipEventRecord(a));
        launch();
        CK(hipEventRecord(b));
        CK(hipEventSynchronize(b));
        float ms = 0.f;
        CK(hipEventElapsedTime(&ms, a, b));
        t.push_back(ms);
    }
    CK(hipGetLastError());
    CK(hipEventDestroy(a));
    CK(hipEventDestroy(b));
    std::sort(t.begin(), t.end());
    return {t[0] * 1e3, t[t.size() / 2] * 1e3};
}

void report(const char* name, double bytes, Timing bare, Timing shipped)
{
    printf("{\"case\": \"%s\", \"bytes\": %.0f, \"bare_us\": %.2f, \"shipped_us\": %.2f, \"bare_median_us\": %.2f, "
           "\"shipped_median_us\": %.2f, \"bare_frac_of_8TBs\": %.4f, \"shipped_frac_of_8TBs\": %.4f}\n",
           name, bytes, bare.fastest_us, shipped.fastest_us, bare.median_us, shipped.median_us,
           bytes / (bare.fastest_us * 1e-6) / 8e12, bytes / (shipped.fastest_us * 1e-6) / 8e12);
    fflush(stdout);
}

// dynamic LDS that lets `waves` 64-lane workgroups share a compute unit (what the library's
// residency throttle asks for)
unsigned lds_for_waves(int waves, int lds_per_cu)
{
    if (waves >= 32) return 0;
    int per_wg = (lds_per_cu / waves) / 512 * 512;
    if (per_wg > 64 * 1024) per_wg = 64 * 1024;
    return (unsigned)per_wg;
}

}  // namespace

int main(int argc, char** argv)
{
    // whole tiles only: 256 elements per update tile, 8192 per statistics tile
    uint64_t n = argc > 1 ? strtoull(argv[1], nullptr, 10) : 202383360ull;  // 4*4096^2 + 3*4096*11008 + 2*4096
    n = n / 8192 * 8192;
    if (n == 0) {
        fprintf(stderr, "need at least 8192 elements\n");
        return 2;
    }
    int dev = 0, lds_per_cu = 0, cus = 0;
    CK(hipGetDevice(&dev));
    CK(hipDeviceGetAttribute(&lds_per_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev));
    CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (lds_per_cu <= 0) lds_per_cu = 160 * 1024;

    // five arrays in one allocation, each 2 MiB-aligned plus a stagger of 2 KiB per array (the layout
    // flextrain_amd.memory.allocate_device_arrays gives the library's own callers)
    const size_t two_mib = (size_t)2 << 20;
    const size_t slot = (n * 4 + two_mib + two_mib - 1) / two_mib * two_mib;
    char* raw = nullptr;
    CK(hipMalloc(&raw, slot * 5 + 2 * two_mib));
    char* base = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(raw) + two_mib - 1) / two_mib * two_mib);
    float* p = reinterpret_cast<float*>(base);
    float* m = reinterpret_cast<float*>(base + slot + 2048);
    float* v = reinterpret_cast<float*>(base + 2 * slot + 4096);
    uint16_t* g = reinterpret_cast<uint16_t*>(base + 3 * slot + 6144);
    uint16_t* h = reinterpret_cast<uint16_t*>(base + 4 * slot + 8192);
    const unsigned fill_blocks = (unsigned)((n + 255) / 256);
    fill_f32<<<fill_blocks, 256>>>(p, n, 0.02f);
    fill_f32<<<fill_blocks, 256>>>(m, n, 1e-4f);
    fill_f32<<<fill_blocks, 256>>>(v, n, 1e-6f);
    fill_bf16<<<fill_blocks, 256>>>(g, n);
    CK(hipDeviceSynchronize());

    const uint64_t tiles = n / 256;
    if (tiles > kMaxWorkgroupsPerLaunch) {
        fprintf(stderr, "too many elements for one launch\n");
        return 2;
    }

    // ---- update (28 B/element), 11 resident wavefronts per CU as the library launches it ---------
    {
        AdamArgs a{};
        a.p = p; a.g = g; a.m = m; a.v = v;
        a.p_out = p; a.m_out = m; a.v_out = v; a.h = h;
        a.ctl = nullptr; a.hyper = nullptr; a.n = tiles * kWave;
        a.c.beta1 = 0.9f; a.c.beta2 = 0.999f; a.c.omb1 = 0.1f; a.c.omb2 = 0.001f; a.c.bias2 = 1.0f; a.c.eps = 1e-8f;
        a.c.step_size = -1e-4f; a.c.wd_coef = -1e-6f; a.c.grad_mult = 1.0f; a.c.wd_mode = 1;
        const unsigned lds = lds_for_waves(11, lds_per_cu);
        const Timing bare = time_launches([&] {
            hipLaunchKernelGGL(bare_update_kernel, dim3((unsigned)tiles), dim3(kWave), lds, 0, p, (const void*)g, m, v, (void*)h);
        });
        const Timing shipped = time_launches([&] {
            hipLaunchKernelGGL((adam_tile_kernel<FT_BF16, FT_BF16, false, false>), dim3((unsigned)tiles), dim3(kWave), lds, 0, a,
                               (uint64_t)0);
        });
        report("update, bf16 gradients and copy (adam_tile_kernel)", n * 28.0, bare, shipped);

        // the same update with one array one element off the others (the relaxed-alignment tiles),
        // against the same bare kernel on aligned arrays: what the odd array costs
        AdamArgs b = a;
        b.m = m + 1;  // the allocation has room behind every array
        b.m_out = m + 1;
        const uint32_t m_off = kRelaxedOnLinesP | kRelaxedOnLinesV | kRelaxedOnLinesH | (1u << kRelaxedCachedShift);
        const Timing relaxed_m = time_launches([&] {
            hipLaunchKernelGGL((adam_tile_relaxed_kernel<FT_BF16, FT_BF16, false, 1>), dim3((unsigned)tiles), dim3(kWave), lds, 0, b,
                               (uint64_t)0, m_off);
        });
        report("update, m one element off (adam_tile_relaxed_kernel, that array cached)", n * 28.0, bare, relaxed_m);
        b = a;
        b.g = g + 1;
        const uint32_t g_off = kRelaxedOnLinesP | kRelaxedOnLinesM | kRelaxedOnLinesV | kRelaxedOnLinesH;
        const Timing relaxed_g = time_launches([&] {
            hipLaunchKernelGGL((adam_tile_relaxed_kernel<FT_BF16, FT_BF16, false, 2>), dim3((unsigned)tiles), dim3(kWave), lds, 0, b,
                               (uint64_t)0, g_off);
        });
        report("update, g one element off (adam_tile_relaxed_kernel, gradient cached)", n * 28.0, bare, relaxed_g);
    }

    // ---- accumulation (10 and 12 B/element): acc = p's array, fp32; g bf16 ---------------------------
    {
        const uint64_t nvec = n / 4;
        const unsigned lds26 = lds_for_waves(26, lds_per_cu), lds20 = lds_for_waves(20, lds_per_cu);
        Timing bare = time_launches([&] {
            hipLaunchKernelGGL(bare_accumulate_kernel<false>, dim3((unsigned)tiles), dim3(kWave), lds26, 0, p, (void*)g, 1e-3f);
        });
        Timing shipped = time_launches([&] {
            hipLaunchKernelGGL((grad_accumulate_kernel<FT_F32, FT_BF16, false, false>), dim3((unsigned)tiles), dim3(kWave), lds26, 0,
                               (void*)p, (void*)g, nvec, 1e-3f, 1.0f, (WavePartial*)nullptr, ~0ull, 0);
        });
        report("accumulate (grad_accumulate_kernel)", n * 10.0, bare, shipped);
        bare = time_launches([&] {
            hipLaunchKernelGGL(bare_accumulate_kernel<true>, dim3((unsigned)tiles), dim3(kWave), lds20, 0, p, (void*)g, 1e-3f);
        });
        shipped = time_launches([&] {
            hipLaunchKernelGGL((grad_accumulate_kernel<FT_F32, FT_BF16, true, false>), dim3((unsigned)tiles), dim3(kWave), lds20, 0,
                               (void*)p, (void*)g, nvec, 1e-3f, 1.0f, (WavePartial*)nullptr, ~0ull, 0);
        });
        report("accumulate + clear (grad_accumulate_kernel)", n * 12.0, bare, shipped);
        fill_bf16<<<fill_blocks, 256>>>(g, n);  // the clearing variants left zeros
        CK(hipDeviceSynchronize());
    }

    // ---- statistics (2 B/element): 2 blocks of 256 threads per CU as the library launches it ---------
    {
        const uint64_t nvec = n / 8;
        const unsigned grid = (unsigned)cus * 2;
        double* partials = nullptr;
        StatsPartial* parts = nullptr;
        uint32_t *sink = nullptr, *ticket = nullptr;
        ft_grad_stats_t* out = nullptr;
        ft_step_control_t* ctl = nullptr;
        CK(hipMalloc(&partials, grid * sizeof(double)));
        CK(hipMalloc(&parts, grid * sizeof(StatsPartial)));
        CK(hipMalloc(&sink, 256));
        CK(hipMalloc(&ticket, 256));
        CK(hipMalloc(&out, 256));
        CK(hipMalloc(&ctl, 256));
        CK(hipMemset(ticket, 0, 256));
        CK(hipMemset(parts, 0, grid * sizeof(StatsPartial)));
        const u32x4* gv = reinterpret_cast<const u32x4*>(g);
        const Timing loads_only = time_launches([&] {
            hipLaunchKernelGGL(bare_read_kernel<false>, dim3(grid), dim3(256), 0, 0, gv, nvec, partials, sink);
        });
        const Timing bare = time_launches([&] {
            hipLaunchKernelGGL(bare_read_kernel<true>, dim3(grid), dim3(256), 0, 0, gv, nvec, partials, sink);
        });
        StatsFinalArgs fin{};
        fin.g = g; fin.head = 0; fin.tail_begin = n; fin.n = n;
        fin.out = out; fin.accumulate = 0; fin.inv_scale = 0.5f; fin.max_norm = 1.0f; fin.ctl = ctl;
        fin.ticket = nullptr; fin.tag = 0;
        const Timing partials_only = time_launches([&] {  // the first of the two launches of the older form
            hipLaunchKernelGGL((grad_stats_kernel<FT_BF16, 256, 4>), dim3(grid), dim3(256), 0, 0, gv, nvec, 0.5f, parts, ~0ull,
                               (const float*)nullptr, fin);
        });
        uint32_t tag = 0;
        fin.ticket = ticket;
        const Timing whole = time_launches([&] {  // one launch: partials, final sum, record and decision
            tag = tag % 0xffffu + 1;
            fin.tag = tag;
            hipLaunchKernelGGL((grad_stats_kernel<FT_BF16, 256, 4>), dim3(grid), dim3(256), 0, 0, gv, nvec, 0.5f, parts, ~0ull,
                               (const float*)nullptr, fin);
        });
        report("read only, no arithmetic, against the same with fp64 squares", n * 2.0, loads_only, bare);
        report("statistics, block partials only (grad_stats_kernel)", n * 2.0, bare, partials_only);
        report("statistics with final sum and decision, one launch (grad_stats_kernel)", n * 2.0, bare, whole);
    }
    CK(hipFree(raw));
    return 0;
}
