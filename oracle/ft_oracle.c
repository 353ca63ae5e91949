/*
 * ft_oracle.c -- host scalars, dispatch, gradient statistics and conversions of the CPU checker
 * (test infrastructure, see ft_oracle.h for what follows which reference lines).
 */
#include "ft_oracle.h"

#include <math.h>
#include <omp.h>

#include "conv_inl.h"

typedef void (*range_fn)(const ft_oracle_scalars*, float, float*, const void*, int, float*, float*,
                         void*, int, size_t, size_t);

void ft_oracle_adam_range_base(const ft_oracle_scalars*, float, float*, const void*, int, float*,
                               float*, void*, int, size_t, size_t);
void ft_oracle_adam_range_avx2(const ft_oracle_scalars*, float, float*, const void*, int, float*,
                               float*, void*, int, size_t, size_t);
void ft_oracle_adam_range_avx512(const ft_oracle_scalars*, float, float*, const void*, int, float*,
                                 float*, void*, int, size_t, size_t);

int ft_oracle_best_isa(void)
{
#if defined(__x86_64__)
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
        __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512dq") &&
        __builtin_cpu_supports("fma"))
        return 2;
    if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) return 1;
#endif
    return 0;
}

int ft_oracle_max_threads(void) { return omp_get_max_threads(); }

void ft_oracle_scalars_compute(uint64_t step, float lr, float beta1, float beta2, float eps,
                               float weight_decay, int bias_correction, int adamw_mode,
                               int double_sqrt, ft_oracle_scalars* out)
{
    /* cpu_adam.h:73-74,86-87: std::pow(float, size_t) promotes both operands to double; the
     * result is stored into a float member. The cached-value branch (:75-83) keeps a value that
     * the same pow() call produced earlier, so a stateless evaluation is equivalent. */
    const float b1t = (float)pow((double)beta1, (double)step);
    const float b2t = (float)pow((double)beta2, (double)step);

    float bias1 = 1.0f, bias2 = 1.0f;
    if (bias_correction) { /* cpu_adam.h:98-101 */
        bias1 = 1.0f - b1t;
        if (double_sqrt)
            bias2 = (float)(1.0 / sqrt((double)(1.0f - b2t)));
        else
            bias2 = 1.0f / sqrtf(1.0f - b2t);
    }
    out->beta1 = beta1;
    out->beta2 = beta2;
    out->omb1 = 1.0f - beta1; /* cpu_adam.h:148-149, float arithmetic */
    out->omb2 = 1.0f - beta2;
    out->bias2 = bias2;
    out->eps = eps;
    out->step_size = (-1.0f * lr) / bias1; /* cpu_adam.h:161: -1 * _alpha / _bias_correction1 */
    if (weight_decay > 0.0f) {             /* cpu_adam.h:165-168 */
        out->wd_mode = adamw_mode ? 1 : 2;
        out->wd_coef = adamw_mode ? (-1.0f * lr) * weight_decay : weight_decay;
    } else {
        out->wd_mode = 0;
        out->wd_coef = 0.0f;
    }
    out->beta1_t = b1t;
    out->beta2_t = b2t;
    out->bias1 = bias1;
}

static range_fn pick(int isa)
{
    const int best = ft_oracle_best_isa();
    if (isa < 0) isa = best;
    if (isa > best) return 0;
    switch (isa) {
        case 0: return ft_oracle_adam_range_base;
        case 1: return ft_oracle_adam_range_avx2;
        case 2: return ft_oracle_adam_range_avx512;
        default: return 0;
    }
}

int ft_oracle_adam_step(const ft_oracle_scalars* s, float grad_mult, float* p, const void* g,
                        int g_dtype, float* m, float* v, void* half_out, int half_dtype, size_t n,
                        int isa, int threads)
{
    if (g_dtype < 0 || g_dtype > 2) return -1;
    if (half_out && half_dtype != FT_ORACLE_F16 && half_dtype != FT_ORACLE_BF16) return -1;
    range_fn fn = pick(isa);
    if (!fn) return -1;
    if (n == 0) return 0;

    const size_t grain = 1u << 16; /* elements per work item; a multiple of the tile */
    const size_t items = (n + grain - 1) / grain;
    if (threads <= 0) threads = omp_get_max_threads();
    if ((size_t)threads > items) threads = (int)items;

#pragma omp parallel for schedule(static) num_threads(threads)
    for (size_t k = 0; k < items; ++k) {
        const size_t b = k * grain;
        const size_t e = (b + grain < n) ? b + grain : n;
        fn(s, grad_mult, p, g, g_dtype, m, v, half_out, half_dtype, b, e);
    }
    return 0;
}

void ft_oracle_adam_trace(const ft_oracle_scalars* s, float grad_mult, float p, float g, float m,
                          float v, float out[11])
{
    float g32 = g * grad_mult;
    if (s->wd_mode == 2) g32 = fmaf(p, s->wd_coef, g32);
    const float m1 = m * s->beta1;
    const float mn = fmaf(g32, s->omb1, m1);
    const float v1 = v * s->beta2;
    const float g2 = g32 * g32;
    const float vn = fmaf(g2, s->omb2, v1);
    const float sq = sqrtf(vn);
    const float d = fmaf(sq, s->bias2, s->eps);
    const float u = mn / d;
    const float p1 = (s->wd_mode == 1) ? fmaf(p, s->wd_coef, p) : p;
    const float pn = fmaf(u, s->step_size, p1);
    out[0] = g32;
    out[1] = m1;
    out[2] = mn;
    out[3] = v1;
    out[4] = g2;
    out[5] = vn;
    out[6] = sq;
    out[7] = d;
    out[8] = u;
    out[9] = p1;
    out[10] = pn;
}

int ft_oracle_grad_stats(const void* g, int g_dtype, size_t n, float pre_mult,
                         uint64_t* out_nonfinite, double* out_sumsq, int threads)
{
    if (g_dtype < 0 || g_dtype > 2) return -1;
    if (threads <= 0) threads = omp_get_max_threads();
    uint64_t bad = 0;
    double acc = 0.0;
    const size_t grain = 1u << 16;
    const size_t items = (n + grain - 1) / grain;

#pragma omp parallel for schedule(static) num_threads(threads) reduction(+ : bad, acc)
    for (size_t k = 0; k < items; ++k) {
        const size_t b = k * grain;
        const size_t e = (b + grain < n) ? b + grain : n;
        double local = 0.0;
        uint64_t lbad = 0;
        for (size_t i = b; i < e; ++i) {
            float x;
            int nonfinite;
            if (g_dtype == FT_ORACLE_F32) {
                x = ((const float*)g)[i];
                nonfinite = (fto_bits(x) & 0x7f800000u) == 0x7f800000u;
            } else if (g_dtype == FT_ORACLE_BF16) {
                const uint16_t h = ((const uint16_t*)g)[i];
                x = fto_bf16_to_f32(h);
                nonfinite = (h & 0x7f80u) == 0x7f80u;
            } else {
                const uint16_t h = ((const uint16_t*)g)[i];
                x = fto_f16_to_f32(h);
                nonfinite = (h & 0x7c00u) == 0x7c00u;
            }
            if (nonfinite) {
                ++lbad;
            } else {
                const float u = x * pre_mult;
                local += (double)u * (double)u;
            }
        }
        acc += local;
        bad += lbad;
    }
    *out_nonfinite = bad;
    *out_sumsq = acc;
    return 0;
}

static float load_as_f32(const void* a, int dtype, size_t i)
{
    if (dtype == FT_ORACLE_F32) return ((const float*)a)[i];
    if (dtype == FT_ORACLE_BF16) return fto_bf16_to_f32(((const uint16_t*)a)[i]);
    return fto_f16_to_f32(((const uint16_t*)a)[i]);
}

int ft_oracle_grad_accumulate(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g)
{
    if (acc_dtype < 0 || acc_dtype > 2 || g_dtype < 0 || g_dtype > 2) return -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        const float x = fmaf(load_as_f32(g, g_dtype, i), scale, load_as_f32(acc, acc_dtype, i));
        if (acc_dtype == FT_ORACLE_F32)
            ((float*)acc)[i] = x;
        else if (acc_dtype == FT_ORACLE_BF16)
            ((uint16_t*)acc)[i] = fto_f32_to_bf16(x);
        else
            ((uint16_t*)acc)[i] = fto_f32_to_f16(x);
        if (zero_g) {
            if (g_dtype == FT_ORACLE_F32)
                ((float*)g)[i] = 0.0f;
            else
                ((uint16_t*)g)[i] = 0;
        }
    }
    return 0;
}

uint16_t ft_oracle_f32_to_f16(float x) { return fto_f32_to_f16(x); }
uint16_t ft_oracle_f32_to_bf16(float x) { return fto_f32_to_bf16(x); }
float ft_oracle_f16_to_f32(uint16_t h) { return fto_f16_to_f32(h); }
float ft_oracle_bf16_to_f32(uint16_t h) { return fto_bf16_to_f32(h); }

void ft_oracle_convert(const void* src, int src_dtype, void* dst, int dst_dtype, size_t n)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        float x;
        if (src_dtype == FT_ORACLE_F32)
            x = ((const float*)src)[i];
        else if (src_dtype == FT_ORACLE_BF16)
            x = fto_bf16_to_f32(((const uint16_t*)src)[i]);
        else
            x = fto_f16_to_f32(((const uint16_t*)src)[i]);
        if (dst_dtype == FT_ORACLE_F32)
            ((float*)dst)[i] = x;
        else if (dst_dtype == FT_ORACLE_BF16)
            ((uint16_t*)dst)[i] = fto_f32_to_bf16(x);
        else
            ((uint16_t*)dst)[i] = fto_f32_to_f16(x);
    }
}
