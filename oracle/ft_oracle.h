/*
 * ft_oracle.h -- CPU checker for the optimizer-step hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. It restates, in plain C, the arithmetic of the
 * reference's CPU Adam so that the HIP kernels can be compared against it. Only the test-suite,
 * the smoke check and the CPU-baseline leg of the benchmark may load it; the shipped library
 * (libftadam.so) never links, loads or calls anything in here.
 *
 * What each function follows in the reference (paths relative to the reference checkout):
 *   ft_oracle_scalars_compute  flextrain/ops/csrc/includes/cpu_adam.h:67-102   (IncrementStep,
 *                              update_state) and :148-166 (per-call scalars of Step_AVX)
 *   ft_oracle_adam_step        flextrain/ops/csrc/includes/cpu_adam.h:176-212  (one IEEE op per
 *                              line, in that order) with the fp32->fp16 copy-out of
 *                              flextrain/ops/csrc/includes/simd.h:35-37 (vcvtps2ph, RNE)
 *   tails                      flextrain/ops/csrc/adam/cpu_adam_impl.cpp:20-67: a tail element is
 *                              stepped by the same vector ops on a padded copy, so its result is
 *                              the element-wise formula again; the restatement therefore has no
 *                              separate tail path
 *
 * Pinned by (see tests/): bit-exact agreement with the compiled reference (oracle/_ref) on
 * committed golden vectors and on fresh random inputs, closed forms at t=1 with m=v=0,
 * invariants (g=m=v=0), torch.optim.AdamW to ~1e-6, and for the conversions brute force against
 * numpy / torch casts. ft_oracle_adam_trace: every intermediate against exact rational arithmetic
 * rounded once per operation, for the three weight-decay modes, and its p', m', v' against
 * ft_oracle_adam_step. No function of the checker is without such a check.
 *
 * Extensions with NO counterpart in the reference (the reference never unscales, checks or
 * clips gradients -- flextrain/engine.py:249 multiplies the loss and nothing divides the
 * gradients): grad_mult, 16-bit gradient inputs, the bf16 copy-out, ft_oracle_grad_stats.
 * PARITY UNPINNED BY THE REFERENCE for these; they are pinned by closed forms only:
 *   g32   = (float)g16 * grad_mult              (one fp32 multiply; exact for power-of-two mult)
 *   bf16  = RNE of the upper 16 bits, NaN kept  (== torch .to(bfloat16))
 *   flag  = any element whose exponent field is all ones
 *   sumsq = sum over i of ((double)((float)g_i * pre_mult))^2, accumulated in double
 */
#ifndef FT_ORACLE_H
#define FT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { FT_ORACLE_F32 = 0, FT_ORACLE_F16 = 1, FT_ORACLE_BF16 = 2 };

/* Per-call constants of one Adam step, each exactly one float as the reference holds it. */
typedef struct ft_oracle_scalars {
    float beta1;       /* _betta1                                                    */
    float beta2;       /* _betta2                                                    */
    float omb1;        /* float(1 - _betta1)                    cpu_adam.h:148        */
    float omb2;        /* float(1 - _betta2)                    cpu_adam.h:149        */
    float bias2;       /* _bias_correction2 = 1/sqrt(1-b2^t)    cpu_adam.h:100        */
    float eps;         /* _eps                                                       */
    float step_size;   /* -1 * _alpha / _bias_correction1       cpu_adam.h:161        */
    float wd_coef;     /* AdamW: -1*_alpha*_weight_decay (:165); Adam: _weight_decay  */
    int32_t wd_mode;   /* 0: no decay, 1: AdamW (decoupled), 2: Adam (L2 into grad)   */
    float beta1_t;     /* (float)pow((double)b1,(double)t)      cpu_adam.h:73,86      */
    float beta2_t;
    float bias1;       /* _bias_correction1 = 1 - b1^t          cpu_adam.h:99         */
} ft_oracle_scalars;

/* double_sqrt != 0 evaluates 1/sqrt(1-b2^t) in double before rounding to float; it exists only
 * so that a test can show which of the two readings of the unqualified sqrt() the compiled
 * reference follows (the float one). */
void ft_oracle_scalars_compute(uint64_t step, float lr, float beta1, float beta2, float eps,
                               float weight_decay, int bias_correction, int adamw_mode,
                               int double_sqrt, ft_oracle_scalars* out);

/* One Adam/AdamW step over n elements, in place on p, m, v (fp32). g is fp32, fp16 or bf16
 * (g_dtype); half_out is NULL or an fp16/bf16 array that receives the recast of the new p.
 * isa: -1 best available, 0 portable scalar build, 1 AVX2 build, 2 AVX-512 build (all three are
 * the same source and must agree bit for bit). threads <= 0: OpenMP default. Returns 0, or -1
 * for a bad dtype / unsupported isa. */
int ft_oracle_adam_step(const ft_oracle_scalars* s, float grad_mult, float* p, const void* g,
                        int g_dtype, float* m, float* v, void* half_out, int half_dtype, size_t n,
                        int isa, int threads);

/* The same step for ONE element with every intermediate exposed (index order: g32, m1, m', v1,
 * g2, v', s, d, u, p1, p'); used by tests that check the op order against hand arithmetic. */
void ft_oracle_adam_trace(const ft_oracle_scalars* s, float grad_mult, float p, float g, float m,
                          float v, float out[11]);

/* Gradient statistics of the unscaled gradient g*pre_mult: out_nonfinite = number of elements
 * whose stored value is inf or nan (exponent all ones), out_sumsq = sum of squares in double of
 * the finite elements' fp32 products (non-finite elements contribute nothing). */
int ft_oracle_grad_stats(const void* g, int g_dtype, size_t n, float pre_mult,
                         uint64_t* out_nonfinite, double* out_sumsq, int threads);

/* Gradient accumulation: acc[i] = round_to_acc_type(fmaf((float)g[i], scale, (float)acc[i])); with
 * zero_g the gradient is cleared afterwards. No counterpart function in the reference; scale == 1
 * is the `gradacc_buffer += extra_grads` of flextrain/memory/coordinator/optimizer.py:775-777
 * (torch promotes the 16-bit operand exactly, then adds once). Pinned by numpy/torch adds and by
 * exact rational arithmetic for scale != 1. */
int ft_oracle_grad_accumulate(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g);

/* Scalar conversions (software, no hardware conversion instructions). */
uint16_t ft_oracle_f32_to_f16(float x);  /* IEEE binary16, round-to-nearest-even */
uint16_t ft_oracle_f32_to_bf16(float x); /* bfloat16, round-to-nearest-even, NaN stays NaN */
float ft_oracle_f16_to_f32(uint16_t h);
float ft_oracle_bf16_to_f32(uint16_t h);
void ft_oracle_convert(const void* src, int src_dtype, void* dst, int dst_dtype, size_t n);

/* 0 scalar, 1 AVX2, 2 AVX-512: what isa=-1 resolves to on this CPU. */
int ft_oracle_best_isa(void);
int ft_oracle_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
