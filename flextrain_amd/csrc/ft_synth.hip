// ft_synth.hip -- seeded synthetic inputs, bit-identical on the GPU and on the host.
//
// The reference makes its benchmark inputs with torch.randn on the host
// (flextrain/optimizer.py:71-95, driven by flextrain/auto_config.py:281-317). Here an element's
// value is a pure function of (seed, substream, element index): a 64-bit counter hash, 24-bit
// uniforms, and for normals a Box-Muller transform whose logarithm, cosine and conversions are
// written out in IEEE fp32 operations (one rounding per statement, fused multiply-adds spelt out;
// the file is compiled without contraction and without fast-math). The same functions are compiled
// for the device and for the host, so a partition of billions of elements is reproduced exactly
// on any machine, in any chunking, without shipping data.
#include <thread>
#include <vector>

#include "ft_internal.hpp"

namespace {

#define FT_HD __host__ __device__ __forceinline__

FT_HD uint64_t mix64(uint64_t z)  // the splitmix64 finaliser
{
    z ^= z >> 30;
    z *= 0xbf58476d1ce4e5b9ull;
    z ^= z >> 27;
    z *= 0x94d049bb133111ebull;
    z ^= z >> 31;
    return z;
}

// 64 random bits of element `index` of `substream` under `seed`.
FT_HD uint64_t element_bits(uint64_t seed, uint32_t substream, uint64_t index)
{
    const uint64_t key = mix64(seed ^ (0x9e3779b97f4a7c15ull * (static_cast<uint64_t>(substream) + 1u)));
    return mix64(key + 0xd1342543de82ef95ull * index);
}

FT_HD float bits_as_float(uint32_t b)
{
    union {
        uint32_t u;
        float f;
    } x;
    x.u = b;
    return x.f;
}

FT_HD uint32_t float_as_bits(float f)
{
    union {
        uint32_t u;
        float f;
    } x;
    x.f = f;
    return x.u;
}

// (k + 1) * 2^-24 for a 24-bit k: uniform on (0, 1], every value exact in fp32.
FT_HD float unit_interval(uint32_t k24) { return static_cast<float>(k24 + 1u) * 5.9604644775390625e-08f; }

// Natural logarithm of u in (0, 1]: u = 2^e * t with t in [sqrt(1/2), sqrt(2)), so that u close
// to 1 gives e = 0 and no cancellation; ln t = 2 atanh((t-1)/(t+1)).
FT_HD float ln_unit(float u)
{
    const uint32_t b = float_as_bits(u);  // u >= 2^-24: a normal number
    int e = static_cast<int>(b >> 23) - 127;
    float t = bits_as_float((b & 0x007fffffu) | 0x3f800000u);  // [1, 2)
    if (t >= 1.41421356f) {
        t = t * 0.5f;  // exact
        e += 1;
    }
    const float s = (t - 1.0f) / (t + 1.0f);  // |s| <= 0.1716; t - 1 is exact
    const float s2 = s * s;
    float poly = 0.09090909f;                 // 1/11
    poly = fmaf(poly, s2, 0.11111111f);       // 1/9
    poly = fmaf(poly, s2, 0.14285715f);       // 1/7
    poly = fmaf(poly, s2, 0.2f);
    poly = fmaf(poly, s2, 0.33333334f);
    poly = fmaf(poly, s2, 1.0f);
    const float ln_t = (s + s) * poly;
    return fmaf(static_cast<float>(e), 0.69314718f, ln_t);
}

// cos(2 pi (k + 1) / 2^24) by octants: the angle inside an octant is at most pi/4, where the
// usual single-precision minimax polynomials are good to ~1e-7.
FT_HD float cos_turn(uint32_t k24)
{
    const uint32_t a = (k24 + 1u) & 0x00ffffffu;  // position on the circle in 2^-24 turns
    const uint32_t octant = a >> 21;
    const uint32_t frac = a & 0x001fffffu;        // 21 bits inside the octant
    // odd octants measure the angle back from their upper edge
    const uint32_t f = (octant & 1u) ? (0x00200000u - frac) : frac;
    const float x = static_cast<float>(f) * 3.7450702829977e-07f;  // * (pi/4) / 2^21
    const float x2 = x * x;
    float sp = -1.9515295891e-4f;
    sp = fmaf(sp, x2, 8.3321608736e-3f);
    sp = fmaf(sp, x2, -1.6666654611e-1f);
    const float sinx = fmaf(sp * x2, x, x);
    float cp = 2.443315711809948e-5f;
    cp = fmaf(cp, x2, -1.388731625493765e-3f);
    cp = fmaf(cp, x2, 4.166664568298827e-2f);
    const float cosx = fmaf(cp * x2, x2, fmaf(-0.5f, x2, 1.0f));
    // cos of the full angle from the octant: 0:c 1:s 2:-s 3:-c 4:-c 5:-s 6:s 7:c
    const uint32_t use_sin = ((octant + 1u) >> 1) & 1u;
    const uint32_t negative = ((octant + 2u) >> 2) & 1u;
    const float r = use_sin ? sinx : cosx;
    return negative ? -r : r;
}

FT_HD float synth_value(uint64_t seed, uint32_t substream, uint64_t index, int kind, float scale)
{
    const uint64_t bits = element_bits(seed, substream, index);
    const uint32_t k1 = static_cast<uint32_t>(bits >> 40);               // 24 bits
    const uint32_t k2 = static_cast<uint32_t>(bits >> 8) & 0x00ffffffu;  // 24 other bits
    if (kind == FT_SYNTH_UNIFORM) return unit_interval(k1) * scale;
    const float radius = sqrtf(-2.0f * ln_unit(unit_interval(k1)));
    return (radius * cos_turn(k2)) * scale;
}

// fp32 -> bf16 / fp16 bits, round to nearest even, written with integer operations so that the
// host and the device cannot differ. Inputs here are finite.
FT_HD uint16_t to_bf16_bits(float x)
{
    const uint32_t b = float_as_bits(x);
    return static_cast<uint16_t>((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}

FT_HD uint16_t to_f16_bits(float x)
{
    const uint32_t b = float_as_bits(x);
    const uint32_t sign = (b >> 16) & 0x8000u;
    const uint32_t mag = b & 0x7fffffffu;
    if (mag >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);  // rounds to infinity (or is inf/nan)
    if (mag < 0x38800000u) {                                               // below 2^-14: fp16 subnormal
        if (mag < 0x33000000u) return static_cast<uint16_t>(sign);         // below 2^-25: zero
        const uint32_t e = mag >> 23;
        const uint32_t m = (mag & 0x007fffffu) | 0x00800000u;
        const uint32_t shift = 126u - e;  // 14..24
        const uint32_t kept = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1u);
        const uint32_t up = (rem > half || (rem == half && (kept & 1u))) ? 1u : 0u;
        return static_cast<uint16_t>(sign | (kept + up));
    }
    const uint32_t rebased = mag - 0x38000000u;  // exponent re-biased from 127 to 15
    const uint32_t kept = rebased >> 13;
    const uint32_t rem = rebased & 0x1fffu;
    const uint32_t up = (rem > 0x1000u || (rem == 0x1000u && (kept & 1u))) ? 1u : 0u;
    return static_cast<uint16_t>(sign | (kept + up));
}

FT_HD void store_value(void* out, int dtype, size_t i, float x)
{
    if (dtype == FT_F32)
        static_cast<float*>(out)[i] = x;
    else if (dtype == FT_BF16)
        static_cast<uint16_t*>(out)[i] = to_bf16_bits(x);
    else
        static_cast<uint16_t*>(out)[i] = to_f16_bits(x);
}

__global__ void synth_fill_kernel(void* out, int dtype, size_t n, uint64_t seed, uint32_t substream, uint64_t first_index,
                                  int kind, float scale)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
        store_value(out, dtype, i, synth_value(seed, substream, first_index + i, kind, scale));
}

int check_args(const void* out, int dtype, size_t n, int kind)
{
    if (dtype != FT_F32 && dtype != FT_F16 && dtype != FT_BF16) return fth::fail(FT_EINVAL, "unknown dtype code %d", dtype);
    if (kind != FT_SYNTH_NORMAL && kind != FT_SYNTH_UNIFORM) return fth::fail(FT_EINVAL, "kind must be FT_SYNTH_NORMAL or FT_SYNTH_UNIFORM");
    if (n > 0 && !out) return fth::fail(FT_EINVAL, "out must not be NULL");
    const size_t esz = dtype == FT_F32 ? 4 : 2;
    if (reinterpret_cast<uintptr_t>(out) % esz) return fth::fail(FT_EALIGN, "out is not aligned to its element size");
    return FT_OK;
}

}  // namespace

extern "C" {

int ft_synth_fill(void* out, int dtype, size_t n, uint64_t seed, uint32_t substream, uint64_t first_index, int kind,
                  float scale, void* stream)
{
    int rc = check_args(out, dtype, n, kind);
    if (rc != FT_OK || n == 0) return rc;
    const size_t want = (n + 255) / 256;
    const size_t cap = static_cast<size_t>(fth::cu_count()) * 16;
    const unsigned grid = static_cast<unsigned>(want < cap ? want : cap);
    hipLaunchKernelGGL(synth_fill_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), out, dtype, n, seed,
                       substream, first_index, kind, scale);
    FT_HIP(hipGetLastError());
    return FT_OK;
}

int ft_synth_fill_host(void* out, int dtype, size_t n, uint64_t seed, uint32_t substream, uint64_t first_index, int kind,
                       float scale)
{
    int rc = check_args(out, dtype, n, kind);
    if (rc != FT_OK) return rc;
    auto fill_range = [=](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; ++i) store_value(out, dtype, i, synth_value(seed, substream, first_index + i, kind, scale));
    };
    // elements are independent: large fills are cut over the hardware threads (at most 16)
    unsigned workers = std::thread::hardware_concurrency();
    if (workers > 16) workers = 16;
    if (workers < 2 || n < (1u << 20)) {
        fill_range(0, n);
        return FT_OK;
    }
    const size_t share = (n + workers - 1) / workers;
    std::vector<std::thread> pool;
    for (unsigned w = 0; w < workers; ++w) {
        const size_t lo = static_cast<size_t>(w) * share;
        const size_t hi = lo + share < n ? lo + share : n;
        if (lo < hi) pool.emplace_back(fill_range, lo, hi);
    }
    for (std::thread& t : pool) t.join();
    return FT_OK;
}

}  // extern "C"
