// ft_cabi_check -- exercises libftadam.so through its C ABI alone, the way a binding in another
// language would: HIP runtime for memory and a stream, plain pointers and sizes into the library,
// no Python and no torch. Every result is compared bit for bit with the CPU checker
// (libftoracle.so), which is test infrastructure and linked only into this test program.
//
// Prints one line per check and exits 0 when all passed. Needs a GPU.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "ft_adam.h"
#include "ft_oracle.h"

namespace {

int g_failures = 0;

void check(bool ok, const char* what)
{
    std::printf("%s  %s\n", ok ? "ok  " : "FAIL", what);
    std::fflush(stdout);
    if (!ok) ++g_failures;
}

#define HIP_OK(expr)                                                                       \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            std::printf("FAIL  %s: %s\n", #expr, hipGetErrorString(e_));                   \
            std::exit(2);                                                                  \
        }                                                                                  \
    } while (0)

#define FT_OK_OR_DIE(expr)                                                                 \
    do {                                                                                   \
        int rc_ = (expr);                                                                  \
        if (rc_ != FT_OK) {                                                                \
            std::printf("FAIL  %s -> %d: %s\n", #expr, rc_, ft_last_error());              \
            std::exit(2);                                                                  \
        }                                                                                  \
    } while (0)

// splitmix64 -> uniform in (0, 1)
struct Rng {
    uint64_t s;
    double uniform()
    {
        uint64_t z = (s += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        z ^= z >> 31;
        return ((z >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    }
    float normal(float std) { return std * (float)(std::sqrt(-2.0 * std::log(uniform())) * std::cos(6.283185307179586 * uniform())); }
};

template <typename T>
T* dev_copy(const std::vector<T>& h)
{
    T* d = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d), h.size() * sizeof(T) + 16));
    HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

template <typename T>
bool same_bits(const T* dev, const std::vector<T>& want)
{
    std::vector<T> got(want.size());
    HIP_OK(hipMemcpy(got.data(), dev, want.size() * sizeof(T), hipMemcpyDeviceToHost));
    return std::memcmp(got.data(), want.data(), want.size() * sizeof(T)) == 0;
}

const float LR = 1e-4f, B1 = 0.9f, B2 = 0.999f, EPS = 1e-8f, WD = 0.01f;

void resident_mixed_precision_step(hipStream_t stream)
{
    const size_t n = 1000003;  // odd: head/tail paths
    const float loss_scale = 1024.f;
    const uint64_t t = 3;
    Rng rng{42};
    std::vector<float> p(n), m(n), v(n);
    std::vector<uint16_t> g(n), h(n, 0);
    for (size_t i = 0; i < n; ++i) {
        p[i] = rng.normal(0.02f);
        m[i] = rng.normal(1e-4f);
        v[i] = (float)(rng.uniform() * 1e-6);
        g[i] = ft_oracle_f32_to_f16(rng.normal(5e-3f) * loss_scale);
    }
    float *dp = dev_copy(p), *dm = dev_copy(m), *dv = dev_copy(v);
    uint16_t *dg = dev_copy(g), *dh = dev_copy(h);
    void* ws = nullptr;
    char* rec = nullptr;  // ft_grad_stats_t followed by ft_step_control_t
    HIP_OK(hipMalloc(&ws, ft_grad_stats_workspace_bytes()));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&rec), 32));

    FT_OK_OR_DIE(ft_adam_create(7, LR, B1, B2, EPS, WD, 1, 0));
    FT_OK_OR_DIE(ft_grad_stats(dg, FT_F16, n, 1.f / loss_scale, rec, 0, ws, ft_grad_stats_workspace_bytes(), stream));
    FT_OK_OR_DIE(ft_grad_control(rec, 1.f / loss_scale, 1.0f, rec + 16, stream));
    FT_OK_OR_DIE(ft_adam_step(7, t, LR, B1, B2, EPS, WD, 1, 1.0f, dp, dg, FT_F16, dm, dv, dh, FT_BF16, n, rec + 16, stream));
    HIP_OK(hipStreamSynchronize(stream));

    ft_grad_stats_t stats;
    ft_step_control_t ctl;
    HIP_OK(hipMemcpy(&stats, rec, 16, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(&ctl, rec + 16, 16, hipMemcpyDeviceToHost));
    uint64_t bad = 0;
    double sumsq = 0;
    ft_oracle_grad_stats(g.data(), FT_ORACLE_F16, n, 1.f / loss_scale, &bad, &sumsq, 0);
    check(stats.nonfinite == 0 && bad == 0 && ctl.skip == 0, "statistics: no inf/nan, step not skipped");
    check(std::fabs(std::sqrt(stats.sumsq) - std::sqrt(sumsq)) <= 1e-6 * std::sqrt(sumsq), "statistics: norm within 1e-6 of the fp64 sum");
    const float clip = (float)std::fmin(1.0, 1.0 / (std::sqrt(stats.sumsq) + 1e-6));
    check(ctl.clip_coef == clip && ctl.grad_mult == clip * (1.f / loss_scale) && clip < 1.f, "decision: clip and multiplier follow the closed form");

    ft_oracle_scalars s;
    ft_oracle_scalars_compute(t, LR, B1, B2, EPS, WD, 1, 1, 0, &s);
    ft_oracle_adam_step(&s, ctl.grad_mult, p.data(), g.data(), FT_ORACLE_F16, m.data(), v.data(), h.data(), FT_ORACLE_BF16, n, -1, 0);
    check(same_bits(dp, p) && same_bits(dm, m) && same_bits(dv, v), "update: p, m, v bit-identical to the CPU checker");
    check(same_bits(dh, h), "update: bf16 copy bit-identical");

    // an overflow: the device-side decision must leave everything untouched
    const uint16_t inf16 = 0x7c00;
    HIP_OK(hipMemcpy(dg + 12345, &inf16, 2, hipMemcpyHostToDevice));
    FT_OK_OR_DIE(ft_grad_stats(dg, FT_F16, n, 1.f / loss_scale, rec, 0, ws, ft_grad_stats_workspace_bytes(), stream));
    FT_OK_OR_DIE(ft_grad_control(rec, 1.f / loss_scale, 1.0f, rec + 16, stream));
    FT_OK_OR_DIE(ft_adam_step(7, t + 1, LR, B1, B2, EPS, WD, 1, 1.0f, dp, dg, FT_F16, dm, dv, dh, FT_BF16, n, rec + 16, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(&stats, rec, 16, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(&ctl, rec + 16, 16, hipMemcpyDeviceToHost));
    check(stats.nonfinite == 1 && ctl.skip == 1, "overflow: one inf counted, skip set");
    check(same_bits(dp, p) && same_bits(dm, m) && same_bits(dv, v) && same_bits(dh, h), "overflow: state untouched");

    // error behaviour
    check(ft_adam_step(99, 1, LR, B1, B2, EPS, WD, 1, 1.f, dp, dg, FT_F16, dm, dv, nullptr, FT_BF16, n, nullptr, stream) == FT_ENOENT &&
              std::strstr(ft_last_error(), "99") != nullptr,
          "unknown optimizer id is FT_ENOENT with a message");
    check(ft_adam_step(7, 1, LR, B1, B2, EPS, WD, 1, 1.f, reinterpret_cast<char*>(dp) + 2, dg, FT_F16, dm, dv, nullptr, FT_BF16, 8, nullptr,
                       stream) == FT_EALIGN,
          "pointer not aligned to its element is FT_EALIGN");
    check(ft_adam_step(7, 1, LR, B1, B2, EPS, WD, 1, 1.f, dp, dg, 9, dm, dv, nullptr, FT_BF16, 8, nullptr, stream) == FT_EINVAL,
          "unknown dtype code is FT_EINVAL");
    check(ft_adam_step(7, 1, LR, B1, B2, EPS, WD, 1, 1.f, nullptr, nullptr, FT_F32, nullptr, nullptr, nullptr, FT_BF16, 0, nullptr, stream) == FT_OK,
          "zero elements is a no-op");
    FT_OK_OR_DIE(ft_adam_destroy(7));
    // like the reference's erase of a missing key (cpu_adam_impl.cpp:297-302)
    check(ft_adam_destroy(7) == FT_OK, "destroying an id twice is a harmless no-op");
    check(ft_adam_step(7, 1, LR, B1, B2, EPS, WD, 1, 1.f, dp, dg, FT_F16, dm, dv, nullptr, FT_BF16, 8, nullptr, stream) == FT_ENOENT,
          "a destroyed id is unknown afterwards");
    HIP_OK(hipFree(dp)); HIP_OK(hipFree(dm)); HIP_OK(hipFree(dv)); HIP_OK(hipFree(dg)); HIP_OK(hipFree(dh));
    HIP_OK(hipFree(ws)); HIP_OK(hipFree(rec));
}

void accumulate_pass(hipStream_t stream)
{
    const size_t n = 300007;
    Rng rng{7};
    std::vector<float> acc(n);
    std::vector<uint16_t> g(n);
    for (size_t i = 0; i < n; ++i) {
        acc[i] = rng.normal(1.f);
        g[i] = ft_oracle_f32_to_bf16(rng.normal(0.1f));
    }
    float* dacc = dev_copy(acc);
    uint16_t* dg = dev_copy(g);
    void* ws = nullptr;
    char* rec = nullptr;
    HIP_OK(hipMalloc(&ws, ft_grad_accumulate_workspace_bytes(n)));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&rec), 16));
    FT_OK_OR_DIE(ft_grad_accumulate(dacc, FT_F32, dg, FT_BF16, n, 0.25f, 1, 1.0f, rec, 0, ws, ft_grad_accumulate_workspace_bytes(n), stream));
    HIP_OK(hipStreamSynchronize(stream));
    ft_oracle_grad_accumulate(acc.data(), FT_ORACLE_F32, g.data(), FT_ORACLE_BF16, n, 0.25f, 1);
    check(same_bits(dacc, acc), "accumulate: acc bit-identical to the CPU checker");
    check(same_bits(dg, g), "accumulate: source cleared");
    ft_grad_stats_t stats;
    HIP_OK(hipMemcpy(&stats, rec, 16, hipMemcpyDeviceToHost));
    uint64_t bad = 0;
    double sumsq = 0;
    ft_oracle_grad_stats(acc.data(), FT_ORACLE_F32, n, 1.0f, &bad, &sumsq, 0);
    check(stats.nonfinite == 0 && std::fabs(stats.sumsq - sumsq) <= 2e-6 * sumsq, "accumulate: fused statistics match");
    HIP_OK(hipFree(dacc)); HIP_OK(hipFree(dg)); HIP_OK(hipFree(ws)); HIP_OK(hipFree(rec));
}

// Many step contexts in one call: three ragged segments of two "parameter groups" (different
// learning rate, decay and step) cut out of flat buffers at odd element offsets, statistics and
// decision in one fused call (ft_grad_decide) over the whole gradient buffer.
void many_segments_one_launch(hipStream_t stream)
{
    const size_t total = 700011;
    const size_t lo[3] = {1, 200002, 200007}, len[3] = {200000, 5, 500001};
    const float lr[3] = {LR, 3e-4f, LR}, wd[3] = {WD, 0.f, WD};
    const uint64_t step[3] = {10, 4, 10};
    Rng rng{5};
    std::vector<float> p(total), m(total), v(total);
    std::vector<uint16_t> g(total), h(total, 0x4111);
    for (size_t i = 0; i < total; ++i) {
        p[i] = rng.normal(0.02f);
        m[i] = rng.normal(1e-4f);
        v[i] = (float)(rng.uniform() * 1e-6);
        g[i] = ft_oracle_f32_to_bf16(rng.normal(1e-3f) * 8.f);
    }
    float *dp = dev_copy(p), *dm = dev_copy(m), *dv = dev_copy(v);
    uint16_t *dg = dev_copy(g), *dh = dev_copy(h);
    void* ws = nullptr;
    char* rec = nullptr;
    HIP_OK(hipMalloc(&ws, ft_grad_stats_workspace_bytes()));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&rec), 32));
    FT_OK_OR_DIE(ft_adam_create(9, LR, B1, B2, EPS, WD, 1, 0));
    FT_OK_OR_DIE(ft_grad_decide(dg, FT_BF16, total, 1.f / 8.f, rec, 0, 1.f / 8.f, 0.f, rec + 16, ws, ft_grad_stats_workspace_bytes(), stream));
    ft_adam_segment_t segs[3];
    std::memset(segs, 0, sizeof segs);
    for (int k = 0; k < 3; ++k) {
        segs[k].p = dp + lo[k];
        segs[k].g = dg + lo[k];
        segs[k].m = dm + lo[k];
        segs[k].v = dv + lo[k];
        segs[k].half_out = dh + lo[k];
        segs[k].n = len[k];
        segs[k].step = step[k];
        segs[k].lr = lr[k];
        segs[k].beta1 = B1;
        segs[k].beta2 = B2;
        segs[k].eps = EPS;
        segs[k].weight_decay = wd[k];
        segs[k].bias_correction = 1;
        segs[k].grad_mult = 123.f;  // overridden by the control record
    }
    FT_OK_OR_DIE(ft_adam_step_multi(9, segs, 3, FT_BF16, FT_BF16, rec + 16, stream));
    HIP_OK(hipStreamSynchronize(stream));
    ft_step_control_t ctl;
    HIP_OK(hipMemcpy(&ctl, rec + 16, 16, hipMemcpyDeviceToHost));
    check(ctl.skip == 0 && ctl.grad_mult == 1.f / 8.f && ctl.clip_coef == 1.f, "fused statistics + decision: unscale only");
    for (int k = 0; k < 3; ++k) {
        ft_oracle_scalars s;
        ft_oracle_scalars_compute(step[k], lr[k], B1, B2, EPS, wd[k], 1, 1, 0, &s);
        ft_oracle_adam_step(&s, ctl.grad_mult, p.data() + lo[k], g.data() + lo[k], FT_ORACLE_BF16, m.data() + lo[k], v.data() + lo[k],
                            h.data() + lo[k], FT_ORACLE_BF16, len[k], -1, 0);
    }
    check(same_bits(dp, p) && same_bits(dm, m) && same_bits(dv, v) && same_bits(dh, h),
          "many segments: every segment bit-identical to the CPU checker, nothing outside them touched");
    // the same step with every scalar read from device memory: a second copy of the state must end up identical
    {
        std::vector<float> p2(p), m2(m), v2(v);  // the state after the first step: step it once more, both ways
        std::vector<uint16_t> h2(h);
        float *ep = dev_copy(p2), *em = dev_copy(m2), *ev = dev_copy(v2);
        uint16_t* eh = dev_copy(h2);
        ft_adam_hyper_t host_rec[3];
        ft_adam_hyper_t* dev_rec = nullptr;
        HIP_OK(hipMalloc(reinterpret_cast<void**>(&dev_rec), sizeof host_rec));
        ft_adam_segment_t by_value[3], by_record[3];
        for (int k = 0; k < 3; ++k) {
            FT_OK_OR_DIE(ft_adam_hyper_fill(9, step[k] + 1, lr[k], B1, B2, EPS, wd[k], 1, 0.5f, &host_rec[k]));
            by_value[k] = segs[k];
            by_value[k].step = step[k] + 1;
            by_value[k].grad_mult = 0.5f;
            by_record[k] = segs[k];
            by_record[k].p = ep + lo[k];
            by_record[k].m = em + lo[k];
            by_record[k].v = ev + lo[k];
            by_record[k].half_out = eh + lo[k];
            by_record[k].step = 999;       // ignored: the record decides
            by_record[k].lr = 123.f;
            by_record[k].hyper = dev_rec + k;
        }
        HIP_OK(hipMemcpyAsync(dev_rec, host_rec, sizeof host_rec, hipMemcpyHostToDevice, stream));
        FT_OK_OR_DIE(ft_adam_step_multi(9, by_value, 3, FT_BF16, FT_BF16, nullptr, stream));
        FT_OK_OR_DIE(ft_adam_step_multi(9, by_record, 2, FT_BF16, FT_BF16, nullptr, stream));
        FT_OK_OR_DIE(ft_adam_step_hyper(9, dev_rec + 2, ep + lo[2], dg + lo[2], FT_BF16, em + lo[2], ev + lo[2], eh + lo[2], FT_BF16, len[2],
                                        nullptr, stream));
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(p2.data(), dp, total * 4, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(m2.data(), dm, total * 4, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(v2.data(), dv, total * 4, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(h2.data(), dh, total * 2, hipMemcpyDeviceToHost));
        check(same_bits(ep, p2) && same_bits(em, m2) && same_bits(ev, v2) && same_bits(eh, h2),
              "scalars from device memory: the same bits as by value (many segments and single call)");
        HIP_OK(hipMemcpy(dp, p.data(), total * 4, hipMemcpyHostToDevice));  // back to the state the checks below expect
        HIP_OK(hipMemcpy(dm, m.data(), total * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dv, v.data(), total * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dh, h.data(), total * 2, hipMemcpyHostToDevice));
        HIP_OK(hipFree(ep)); HIP_OK(hipFree(em)); HIP_OK(hipFree(ev)); HIP_OK(hipFree(eh)); HIP_OK(hipFree(dev_rec));
    }
    segs[1].m = nullptr;
    check(ft_adam_step_multi(9, segs, 3, FT_BF16, FT_BF16, nullptr, stream) == FT_EINVAL, "many segments: a NULL array is refused");
    HIP_OK(hipStreamSynchronize(stream));
    check(same_bits(dp, p), "many segments: a refused call launched nothing");
    FT_OK_OR_DIE(ft_adam_destroy(9));
    HIP_OK(hipFree(dp)); HIP_OK(hipFree(dm)); HIP_OK(hipFree(dv)); HIP_OK(hipFree(dg)); HIP_OK(hipFree(dh)); HIP_OK(hipFree(ws)); HIP_OK(hipFree(rec));
}

// The accumulation pass without any workspace: the library's static scratch.
void accumulate_without_allocating(hipStream_t stream)
{
    const size_t n = 400003;
    Rng rng{11};
    std::vector<float> acc(n);
    std::vector<uint16_t> g(n);
    for (size_t i = 0; i < n; ++i) {
        acc[i] = rng.normal(1.f);
        g[i] = ft_oracle_f32_to_f16(rng.normal(0.1f));
    }
    float* dacc = dev_copy(acc);
    uint16_t* dg = dev_copy(g);
    char* rec = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&rec), 16));
    size_t free_before = 0, free_after = 0, total = 0;
    FT_OK_OR_DIE(ft_grad_accumulate_static(dacc, FT_F32, dg, FT_F16, 16, 1.0f, 0, 1.0f, rec, 0, stream));  // first use on this device
    HIP_OK(hipStreamSynchronize(stream));
    ft_oracle_grad_accumulate(acc.data(), FT_ORACLE_F32, g.data(), FT_ORACLE_F16, 16, 1.0f, 0);
    HIP_OK(hipMemGetInfo(&free_before, &total));
    FT_OK_OR_DIE(ft_grad_accumulate_static(dacc, FT_F32, dg, FT_F16, n, 0.5f, 0, 1.0f, rec, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemGetInfo(&free_after, &total));
    ft_oracle_grad_accumulate(acc.data(), FT_ORACLE_F32, g.data(), FT_ORACLE_F16, n, 0.5f, 0);
    check(same_bits(dacc, acc), "static scratch: acc bit-identical to the CPU checker");
    ft_grad_stats_t stats;
    HIP_OK(hipMemcpy(&stats, rec, 16, hipMemcpyDeviceToHost));
    uint64_t bad = 0;
    double sumsq = 0;
    ft_oracle_grad_stats(acc.data(), FT_ORACLE_F32, n, 1.0f, &bad, &sumsq, 0);
    check(stats.nonfinite == 0 && std::fabs(stats.sumsq - sumsq) <= 2e-6 * sumsq, "static scratch: fused statistics match");
    check(free_before == free_after, "static scratch: the call changed nothing about device memory");
    check(ft_grad_accumulate_static(dacc, FT_F32, dg, FT_F16, (size_t)FT_STATIC_MAX_ELEMS + 1, 1.f, 0, 1.f, rec, 0, stream) == FT_EINVAL,
          "static scratch: more than the maximum is refused");
    HIP_OK(hipFree(dacc)); HIP_OK(hipFree(dg)); HIP_OK(hipFree(rec));
}

void launch_plan_and_stream_state(hipStream_t stream)
{
    // how work is cut into launches: plain arithmetic behind the ABI
    uint64_t first[8], count[8];
    check(ft_launch_pieces(10, 4, first, count, 8) == 3 && first[2] == 8 && count[2] == 2 && count[0] == 4,
          "launch plan: 10 workgroups under a limit of 4 are pieces of 4, 4 and 2");
    check(ft_launch_pieces((1ull << 26), 0, first, count, 8) == 2 && count[0] == (0xffffffffull / 64) && count[1] == 1,
          "launch plan: the default limit is (2^32 - 1) / 64 workgroups");
    const uint64_t wgs[5] = {3, 3, 3, 9, 1};
    int batch_of[5];
    check(ft_segment_batches(wgs, 5, 9, batch_of) == 3 && batch_of[2] == 0 && batch_of[3] == 1 && batch_of[4] == 2,
          "segment batches: a launch of at most 9 workgroups");
    check(ft_set_launch_limit(0xffffffffull) == FT_EINVAL && ft_set_launch_limit(0) == FT_OK, "launch limit: above the runtime's is refused");
    // a statistics pass as one launch and as two give the same record; the stream's state can be given back
    const size_t n = 1'000'003;
    std::vector<uint16_t> g(n);
    for (size_t i = 0; i < n; ++i) g[i] = static_cast<uint16_t>(0x3c00 + (i * 2654435761u >> 22));  // fp16 values in [1, 2)
    uint16_t* dg = nullptr;
    unsigned char* rec = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dg), n * 2));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&rec), 64));
    HIP_OK(hipMemcpy(dg, g.data(), n * 2, hipMemcpyHostToDevice));
    unsigned char one[32], two[32];
    FT_OK_OR_DIE(ft_grad_decide(dg, FT_F16, n, 0.5f, rec, 0, 0.5f, 1.0f, rec + 16, nullptr, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(one, rec, 32, hipMemcpyDeviceToHost));
    FT_OK_OR_DIE(ft_set_stats_launches(2));
    FT_OK_OR_DIE(ft_grad_decide(dg, FT_F16, n, 0.5f, rec + 32, 0, 0.5f, 1.0f, rec + 48, nullptr, 0, stream));
    FT_OK_OR_DIE(ft_set_stats_launches(1));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(two, rec + 32, 32, hipMemcpyDeviceToHost));
    check(!std::memcmp(one, two, 32), "statistics pass: one launch and two launches give the same 32 bytes");
    check(ft_set_stats_launches(3) == FT_EINVAL, "statistics pass: 1 or 2 launches");
    FT_OK_OR_DIE(ft_release_stream_scratch(stream));
    FT_OK_OR_DIE(ft_grad_decide(dg, FT_F16, n, 0.5f, rec + 32, 0, 0.5f, 1.0f, rec + 48, nullptr, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(two, rec + 32, 32, hipMemcpyDeviceToHost));
    check(!std::memcmp(one, two, 32), "statistics pass: the same after the stream's scratch was released");
    FT_OK_OR_DIE(ft_release_stream_scratch(stream));
    HIP_OK(hipFree(dg)); HIP_OK(hipFree(rec));
}

void link_probe()
{
    ft_link_probe_t r;
    FT_OK_OR_DIE(ft_link_probe(64u << 20, 2, &r));
    std::printf("link: copies %.1f / %.1f / %.1f GB/s, copy kernel %.1f / %.1f / %.1f GB/s (H2D / D2H / both), "
                "copies in + kernel out %.1f, kernel in + copies out %.1f\n", r.h2d_copy, r.d2h_copy,
                r.both_copy, r.h2d_kernel, r.d2h_kernel, r.both_kernel, r.both_copy_in_kernel_out, r.both_kernel_in_copy_out);
    check(r.h2d_copy > 1 && r.d2h_copy > 1 && r.both_copy > 1 && r.h2d_kernel > 1 && r.d2h_kernel > 1 && r.both_kernel > 1 &&
              r.both_copy_in_kernel_out > 1 && r.both_kernel_in_copy_out > 1,
          "link probe: eight figures, all positive");
}

void offloaded_step(hipStream_t stream)
{
    const size_t n = 3 * (1u << 18) + 1001;  // four chunks, the last one partial
    Rng rng{99};
    float *p = nullptr, *m = nullptr, *v = nullptr;
    FT_OK_OR_DIE(ft_pinned_alloc(n * 4, reinterpret_cast<void**>(&p)));
    FT_OK_OR_DIE(ft_pinned_alloc(n * 4, reinterpret_cast<void**>(&m)));
    FT_OK_OR_DIE(ft_pinned_alloc(n * 4, reinterpret_cast<void**>(&v)));
    std::vector<float> rp(n), rm(n), rv(n);
    std::vector<uint16_t> g(n), rh(n, 0);
    for (size_t i = 0; i < n; ++i) {
        p[i] = rp[i] = rng.normal(0.02f);
        m[i] = rm[i] = rng.normal(1e-4f);
        v[i] = rv[i] = (float)(rng.uniform() * 1e-6);
        g[i] = ft_oracle_f32_to_bf16(rng.normal(1e-3f));
    }
    uint16_t *dg = dev_copy(g), *dh = dev_copy(rh);
    FT_OK_OR_DIE(ft_adam_create(8, LR, B1, B2, EPS, WD, 1, 0));
    ft_oracle_scalars s;
    const int modes[] = {FT_OFFLOAD_STAGED, FT_OFFLOAD_DIRECT, FT_OFFLOAD_AUTO};
    void* eng = nullptr;
    FT_OK_OR_DIE(ft_offload_create(1u << 18, 3, &eng));
    for (int k = 0; k < 3; ++k) {
        const uint64_t t = 10 + k;
        FT_OK_OR_DIE(ft_offload_set_mode(eng, modes[k]));
        FT_OK_OR_DIE(ft_offload_step(eng, 8, t, LR, B1, B2, EPS, WD, 1, 1.0f, p, dg, FT_BF16, 0, m, v, dh, FT_BF16, 0, n, nullptr, stream));
        FT_OK_OR_DIE(ft_offload_wait(eng));
        ft_oracle_scalars_compute(t, LR, B1, B2, EPS, WD, 1, 1, 0, &s);
        ft_oracle_adam_step(&s, 1.0f, rp.data(), g.data(), FT_ORACLE_BF16, rm.data(), rv.data(), rh.data(), FT_ORACLE_BF16, n, -1, 0);
        const bool host_ok = !std::memcmp(p, rp.data(), n * 4) && !std::memcmp(m, rm.data(), n * 4) && !std::memcmp(v, rv.data(), n * 4);
        char what[96];
        std::snprintf(what, sizeof what, "offloaded step, mode %d: host p, m, v and device bf16 copy bit-identical", modes[k]);
        check(host_ok && same_bits(dh, rh), what);
    }
    float ms = -1.f;
    FT_OK_OR_DIE(ft_offload_elapsed_ms(eng, &ms));
    check(ms > 0.f, "offloaded step reports its device time");
    FT_OK_OR_DIE(ft_offload_destroy(eng));
    FT_OK_OR_DIE(ft_adam_destroy(8));
    FT_OK_OR_DIE(ft_pinned_free(p));
    FT_OK_OR_DIE(ft_pinned_free(m));
    FT_OK_OR_DIE(ft_pinned_free(v));
    HIP_OK(hipFree(dg)); HIP_OK(hipFree(dh));
}

// The seeded input generator: the kernel and the host loop must give the same bits.
void synthetic_inputs(hipStream_t stream)
{
    const size_t n = 100003;
    const uint64_t first = (1ull << 33) + 5;
    for (int dtype : {FT_F32, FT_F16, FT_BF16}) {
        const size_t esz = dtype == FT_F32 ? 4 : 2;
        std::vector<unsigned char> host(n * esz), back(n * esz);
        void* dev = nullptr;
        HIP_OK(hipMalloc(&dev, n * esz));
        for (int kind : {FT_SYNTH_NORMAL, FT_SYNTH_UNIFORM}) {
            FT_OK_OR_DIE(ft_synth_fill(dev, dtype, n, 0, 3, first, kind, 1e-3f, stream));
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipMemcpy(back.data(), dev, n * esz, hipMemcpyDeviceToHost));
            FT_OK_OR_DIE(ft_synth_fill_host(host.data(), dtype, n, 0, 3, first, kind, 1e-3f));
            char what[96];
            std::snprintf(what, sizeof what, "synthetic inputs, dtype %d kind %d: device fill == host fill", dtype, kind);
            check(!std::memcmp(host.data(), back.data(), n * esz), what);
        }
        HIP_OK(hipFree(dev));
    }
    check(ft_synth_fill(nullptr, FT_F32, 4, 0, 0, 0, FT_SYNTH_NORMAL, 1.f, stream) == FT_EINVAL, "synthetic fill rejects a NULL target");
}

}  // namespace

int main()
{
    std::printf("ft_abi_version %d, devices %d\n", ft_abi_version(), ft_device_count());
    if (ft_device_count() < 1) {
        std::printf("FAIL  no GPU visible\n");
        return 2;
    }
    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    resident_mixed_precision_step(stream);
    accumulate_pass(stream);
    many_segments_one_launch(stream);
    accumulate_without_allocating(stream);
    launch_plan_and_stream_state(stream);
    offloaded_step(stream);
    link_probe();
    synthetic_inputs(stream);
    HIP_OK(hipStreamDestroy(stream));
    std::printf("%s (%d failed)\n", g_failures ? "FAILED" : "ALL PASSED", g_failures);
    return g_failures ? 1 : 0;
}
