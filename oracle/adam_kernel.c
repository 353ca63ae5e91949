/*
 * adam_kernel.c -- element loop of the CPU checker (test infrastructure, see ft_oracle.h).
 *
 * Compiled three times (portable, AVX2, AVX-512) with FT_ISA_SUFFIX naming the variant. The
 * loop body is the reference's op sequence, flextrain/ops/csrc/includes/cpu_adam.h:188-205, one
 * IEEE-754 round-to-nearest fp32 operation per statement; products feeding an addition are
 * written as fmaf() exactly where the reference issues SIMD_FMA, and the file is compiled with
 * -ffp-contract=off so the compiler adds or removes none. Auto-vectorisation changes nothing
 * because every operation is correctly rounded lane by lane.
 */
#include <math.h>

#include "conv_inl.h"
#include "ft_oracle.h"

#ifndef FT_ISA_SUFFIX
#error "FT_ISA_SUFFIX must name the ISA variant"
#endif
#define FT_CAT2(a, b) a##b
#define FT_CAT(a, b) FT_CAT2(a, b)
#define FT_FN(name) FT_CAT(name, FT_ISA_SUFFIX)

#define FT_TILE 2048

static void load_grads(float* dst, const void* g, int g_dtype, size_t off, size_t cnt, float mult)
{
    if (g_dtype == FT_ORACLE_F32) {
        const float* s = (const float*)g + off;
        for (size_t i = 0; i < cnt; ++i) dst[i] = s[i] * mult;
    } else if (g_dtype == FT_ORACLE_BF16) {
        const uint16_t* s = (const uint16_t*)g + off;
        for (size_t i = 0; i < cnt; ++i) dst[i] = fto_float((uint32_t)s[i] << 16) * mult;
    } else {
        const uint16_t* s = (const uint16_t*)g + off;
        for (size_t i = 0; i < cnt; ++i) dst[i] = fto_f16_to_f32(s[i]) * mult;
    }
}

static void store_half(void* half_out, int half_dtype, size_t off, size_t cnt, const float* p)
{
    uint16_t* d = (uint16_t*)half_out + off;
    if (half_dtype == FT_ORACLE_BF16) {
        for (size_t i = 0; i < cnt; ++i) d[i] = fto_f32_to_bf16(p[i]);
    } else {
        for (size_t i = 0; i < cnt; ++i) d[i] = fto_f32_to_f16(p[i]);
    }
}

/* Steps elements [begin, end). */
void FT_FN(ft_oracle_adam_range)(const ft_oracle_scalars* sc, float grad_mult, float* p,
                                 const void* g, int g_dtype, float* m, float* v, void* half_out,
                                 int half_dtype, size_t begin, size_t end)
{
    const float b1 = sc->beta1, b2 = sc->beta2, omb1 = sc->omb1, omb2 = sc->omb2;
    const float bias2 = sc->bias2, eps = sc->eps, ss = sc->step_size, wdc = sc->wd_coef;
    const int wd_mode = sc->wd_mode;
    float gbuf[FT_TILE];

    for (size_t t = begin; t < end; t += FT_TILE) {
        const size_t cnt = (end - t < FT_TILE) ? (end - t) : FT_TILE;
        float* pp = p + t;
        float* mm = m + t;
        float* vv = v + t;
        load_grads(gbuf, g, g_dtype, t, cnt, grad_mult);

        if (wd_mode == 2) { /* Adam: L2 term folded into the gradient, cpu_adam.h:188-190 */
            for (size_t i = 0; i < cnt; ++i) gbuf[i] = fmaf(pp[i], wdc, gbuf[i]);
        }
        for (size_t i = 0; i < cnt; ++i) {
            const float gi = gbuf[i];
            float mi = mm[i] * b1;          /* simd_mul(momentum, momentum, betta1)        */
            mi = fmaf(gi, omb1, mi);        /* simd_fma(momentum, grad, betta1_minus1, ..) */
            float vi = vv[i] * b2;          /* simd_mul(variance, variance, betta2)        */
            const float g2 = gi * gi;       /* simd_mul(grad, grad, grad)                  */
            vi = fmaf(g2, omb2, vi);        /* simd_fma(variance, grad, betta2_minus1, ..) */
            float d = sqrtf(vi);            /* simd_sqrt(grad, variance)                   */
            d = fmaf(d, bias2, eps);        /* simd_fma(grad, grad, bias2_sqrt, eps)       */
            gbuf[i] = mi / d;               /* simd_div(grad, momentum, grad)              */
            mm[i] = mi;
            vv[i] = vi;
        }
        if (wd_mode == 1) { /* AdamW: decoupled decay on the pre-update value, :201-203 */
            for (size_t i = 0; i < cnt; ++i) pp[i] = fmaf(pp[i], wdc, pp[i]);
        }
        for (size_t i = 0; i < cnt; ++i) pp[i] = fmaf(gbuf[i], ss, pp[i]); /* :205 */

        if (half_out) store_half(half_out, half_dtype, t, cnt, pp);
    }
}
