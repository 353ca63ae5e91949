// ft_offload.hip -- pinned host memory, the chunked host<->HBM optimizer pipeline and the link probe.
//
// Replaces, for state that lives in pinned host DRAM, the reference's arrangement of
//   flextrain/memory/__init__.py:240-248  RotateContainer (rotating buffer sets)
//   flextrain/memory/__init__.py:366-395  FlexTrainDataStream (one side stream, device-wide waits)
//   flextrain/optimizer.py:244-263        copy grads down, step on the host, copy params up
// with a three-stage pipeline on three HIP streams. Buffer slots are handed from stage to stage
// with events, so a copy in one direction, a copy in the other and a kernel run at the same time.
#include <string.h>

#include <chrono>
#include <deque>
#include <mutex>
#include <vector>

#include "ft_internal.hpp"

namespace {

struct Slot {
    float* p = nullptr;
    float* m = nullptr;
    float* v = nullptr;
    void* g = nullptr;  // staging for host-resident gradients (chunk * 4 bytes), lazily allocated
    void* h = nullptr;  // staging for a host-resident low-precision copy (chunk * 2 bytes), lazy
    hipEvent_t h2d_done = nullptr, k_done = nullptr, d2h_done = nullptr;
    hipEvent_t free_ev = nullptr;  // whichever of the above marks the slot's last use
    bool used = false;
};

// Host memory a step writes back to, and the event that marks its last D2H.
struct Pending {
    uintptr_t lo[4], hi[4];
    int ranges = 0;
    hipEvent_t done = nullptr;
    bool overlaps(const Pending& o) const
    {
        for (int i = 0; i < ranges; ++i)
            for (int j = 0; j < o.ranges; ++j)
                if (lo[i] < o.hi[j] && o.lo[j] < hi[i]) return true;
        return false;
    }
};

constexpr size_t kMaxPending = 8;

// A window keeps the whole state of one unit on the device between ft_offload_window_open and
// ft_offload_window_close: one large H2D per array when it opens (in pieces of up to 1 GiB, each
// with its own event), any number of steps on sub-ranges that run as plain kernels on the device
// copy, and the way back either as one large D2H per array when it closes or -- write_through -- by
// the step kernels themselves, which then write their results straight to the host arrays (each
// element may then be stepped once per window). Measured on the 24-layer schedule with 16 shares
// per unit (each way, concurrently): per-share direct 43.4 GB/s; write-through windows 43.7 GB/s;
// copy-back windows 47.2 GB/s, every iteration alike. Few, large copies matter: with 256 MiB pieces
// (24 copies per unit, 576 per iteration) one iteration in six ran at half speed, the same
// degradation of long bursts of copies that kMaxChunksPerStep guards against.
constexpr size_t kWindowPieceElems = 256u * 1024u * 1024u;  // about 1 GiB per array and copy
constexpr int kMaxWindows = 4;

struct Window {
    float* dev[3] = {nullptr, nullptr, nullptr};
    size_t cap = 0;                  // elements each device array can hold
    uintptr_t host[3] = {0, 0, 0};   // host arrays this window mirrors while open
    size_t n = 0;
    bool open = false;
    bool used = false;               // d2h_done has been recorded at least once
    bool write_through = false;      // steps write their results to the host arrays themselves
    size_t piece = 0;                // elements per copy: n cut into equal pieces, never a small tail
    uint64_t closed_at = 0;          // order of closing: the window closed longest ago is reused first
    std::vector<hipEvent_t> piece_done;
    // Copy-back as pieces complete: elements of piece k stepped since it was last written back, and
    // whether the host already holds what the device copy of piece k holds.
    std::vector<size_t> piece_stepped;
    std::vector<char> piece_clean;
    hipEvent_t k_done = nullptr, d2h_done = nullptr, piece_stepped_ev = nullptr;
};

// Automatic choice of the transfer mode. Measured on MI355X / PCIe Gen5 x16: SDMA copies through
// staging slots move 48-49 GB/s each way when every copy is at least ~128 MiB, but a run of many
// smaller copies ends up with both directions on one SDMA engine and drops to 15 GB/s; the kernel
// reading and writing pinned host memory itself holds 45 GB/s each way at any size.
constexpr size_t kStagedMinElems = 32u * 1024u * 1024u;

// One step is cut into at most this many chunks; a longer one makes the engine grow its chunk (and
// its device buffers) first. Measured with 16 Mi-element chunks over 58 GB of state: 97 chunks in
// one burst run at 49 GB/s each way, 290 chunks at 27-36 GB/s, whatever the host does about it.
constexpr size_t kMaxChunksPerStep = 96;

// A long step ramps in and out: its first and its last chunk's worth of elements go as quarter
// chunks, so that the part of the pipeline that cannot overlap (the first copy in, the last copy
// out) is a quarter of a chunk each instead of a whole one. That costs kRampExtraChunks more chunks
// per step and is done for steps of at least kRampMinChunks chunks only.
constexpr size_t kRampMinChunks = 8;
constexpr size_t kRampExtraChunks = 6;

struct Engine {
    uint32_t magic = 0x46544f45;  // "FTOE"
    std::mutex mu;                // one call at a time per handle; different handles are independent
    int device = 0;
    size_t chunk = 0;
    std::vector<Slot> slots;
    hipStream_t s_h2d = nullptr, s_k = nullptr, s_d2h = nullptr;
    hipEvent_t ev_user = nullptr;   // producer stream -> pipeline
    hipEvent_t ev_begin = nullptr;  // first H2D of the last step
    hipEvent_t ev_end = nullptr;    // last D2H of the last step
    hipEvent_t ev_kernels = nullptr;  // last kernel of the last step
    bool stepped = false;
    bool end_recorded = false;  // ev_begin / ev_end have been recorded at least once
    size_t cursor = 0;  // chunks enqueued so far; slots are taken round-robin across steps
    int mode = FT_OFFLOAD_AUTO;
    size_t burst_chunks = 0;  // staged chunks enqueued since the pipeline was last seen idle
    std::deque<Pending> recent;        // steps whose write-back may still be in flight, oldest first
    std::vector<hipEvent_t> free_events;
    Window windows[kMaxWindows];
    uint64_t window_closes = 0;
    size_t window_piece_elems = kWindowPieceElems;  // ft_offload_set_window_piece
};

Engine* as_engine(void* h)
{
    Engine* e = static_cast<Engine*>(h);
    return (e && e->magic == 0x46544f45) ? e : nullptr;
}

int require_pinned(const void* ptr, const char* what)
{
    hipPointerAttribute_t attr;
    hipError_t err = hipPointerGetAttributes(&attr, ptr);
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return fth::fail(FT_EINVAL, "%s is not pinned host memory (hipPointerGetAttributes: %s)", what,
                         hipGetErrorString(err));
    }
    if (attr.type != hipMemoryTypeHost)
        return fth::fail(FT_EINVAL, "%s must be pinned host memory (memory type %d)", what, (int)attr.type);
    return FT_OK;
}

void destroy_engine(Engine* e)
{
    for (Slot& s : e->slots) {
        if (s.p) (void)hipFree(s.p);
        if (s.m) (void)hipFree(s.m);
        if (s.v) (void)hipFree(s.v);
        if (s.g) (void)hipFree(s.g);
        if (s.h) (void)hipFree(s.h);
        if (s.h2d_done) (void)hipEventDestroy(s.h2d_done);
        if (s.k_done) (void)hipEventDestroy(s.k_done);
        if (s.d2h_done) (void)hipEventDestroy(s.d2h_done);
    }
    if (e->s_h2d) (void)hipStreamDestroy(e->s_h2d);
    if (e->s_k) (void)hipStreamDestroy(e->s_k);
    if (e->s_d2h) (void)hipStreamDestroy(e->s_d2h);
    if (e->ev_user) (void)hipEventDestroy(e->ev_user);
    if (e->ev_begin) (void)hipEventDestroy(e->ev_begin);
    if (e->ev_end) (void)hipEventDestroy(e->ev_end);
    if (e->ev_kernels) (void)hipEventDestroy(e->ev_kernels);
    for (Pending& pd : e->recent)
        if (pd.done) (void)hipEventDestroy(pd.done);
    for (hipEvent_t ev : e->free_events) (void)hipEventDestroy(ev);
    for (Window& w : e->windows) {
        for (float* d : w.dev)
            if (d) (void)hipFree(d);
        for (hipEvent_t ev : w.piece_done) (void)hipEventDestroy(ev);
        if (w.k_done) (void)hipEventDestroy(w.k_done);
        if (w.d2h_done) (void)hipEventDestroy(w.d2h_done);
        if (w.piece_stepped_ev) (void)hipEventDestroy(w.piece_stepped_ev);
    }
    e->magic = 0;
    delete e;
}

// Re-creates the slots' device buffers for `chunk_elems` per chunk. Waits for the pipeline first.
// If the device has no room for them the slots are left without buffers (and the chunk as it was):
// the next staged step tries again at that size, direct steps and windows are not affected.
int resize_slots(Engine* e, size_t chunk_elems)
{
    FT_HIP(hipStreamSynchronize(e->s_h2d));
    FT_HIP(hipStreamSynchronize(e->s_k));
    FT_HIP(hipStreamSynchronize(e->s_d2h));
    for (Slot& s : e->slots) {
        void** bufs[5] = {reinterpret_cast<void**>(&s.p), reinterpret_cast<void**>(&s.m), reinterpret_cast<void**>(&s.v), &s.g, &s.h};
        for (void** b : bufs) {
            if (*b) FT_HIP(hipFree(*b));
            *b = nullptr;
        }
        s.used = false;
    }
    for (Slot& s : e->slots) {
        float** arrays[3] = {&s.p, &s.m, &s.v};
        for (float** a : arrays) {
            const hipError_t err = hipMalloc(reinterpret_cast<void**>(a), chunk_elems * 4);
            if (err != hipSuccess) {
                (void)hipGetLastError();
                for (Slot& t : e->slots) {
                    float** held[3] = {&t.p, &t.m, &t.v};
                    for (float** h : held) {
                        if (*h) (void)hipFree(*h);
                        *h = nullptr;
                    }
                }
                return fth::fail(FT_ENOMEM, "hipMalloc(%zu) for the staging slots failed: %s", chunk_elems * 4, hipGetErrorString(err));
            }
        }
    }
    e->chunk = chunk_elems;
    return FT_OK;
}

// Orders the H2D and kernel streams behind the newest earlier write-back that touched any of the
// host ranges in `mine` (the D2H stream is in order, so that one event covers all older ones).
int wait_for_overlapping_writebacks(Engine* e, const Pending& mine, bool h2d_too = true)
{
    for (auto it = e->recent.rbegin(); it != e->recent.rend(); ++it) {
        if (it->overlaps(mine)) {
            if (h2d_too) FT_HIP(hipStreamWaitEvent(e->s_h2d, it->done, 0));
            FT_HIP(hipStreamWaitEvent(e->s_k, it->done, 0));
            break;
        }
    }
    return FT_OK;
}

// Remembers a write-back whose last D2H is the newest work on the D2H stream. When the list is
// full the oldest entry is retired; every later H2D is then ordered behind it, which costs
// nothing once it has long finished.
int remember_writeback(Engine* e, Pending mine)
{
    if (e->free_events.empty()) {
        Pending& old = e->recent.front();
        FT_HIP(hipStreamWaitEvent(e->s_h2d, old.done, 0));
        FT_HIP(hipStreamWaitEvent(e->s_k, old.done, 0));
        e->free_events.push_back(old.done);
        e->recent.pop_front();
    }
    mine.done = e->free_events.back();
    e->free_events.pop_back();
    FT_HIP(hipEventRecord(mine.done, e->s_d2h));
    e->recent.push_back(mine);
    return FT_OK;
}

// The open window that holds [host_p, host_p + n) and the matching ranges of m and v, if any.
// Returns FT_OK with *out = nullptr when no window is involved, an error for a partial overlap.
int find_window(Engine* e, const void* host_p, const void* host_m, const void* host_v, size_t n, Window** out, size_t* off)
{
    *out = nullptr;
    const uintptr_t lo = reinterpret_cast<uintptr_t>(host_p), hi = lo + n * 4;
    for (Window& w : e->windows) {
        if (!w.open) continue;
        const uintptr_t wlo = w.host[0], whi = w.host[0] + w.n * 4;
        if (hi <= wlo || whi <= lo) continue;
        if (lo < wlo || hi > whi)
            return fth::fail(FT_EINVAL, "a step must lie entirely inside or entirely outside an open window");
        const size_t o = (lo - wlo) / 4;
        if (reinterpret_cast<uintptr_t>(host_m) != w.host[1] + o * 4 || reinterpret_cast<uintptr_t>(host_v) != w.host[2] + o * 4)
            return fth::fail(FT_EINVAL, "exp_avg / exp_avg_sq are not at the params' offset inside the open window");
        *out = &w;
        *off = o;
        return FT_OK;
    }
    return FT_OK;
}

// ---- link probe --------------------------------------------------------------------------------
// What the host link can carry, measured the way a ceiling should be: every figure is the best of
// one and of two transfers in flight per direction (each on a stream of its own, queued back to
// back so the link never waits for the host), once with the runtime's copies and once with a plain
// copy kernel that reads or writes the pinned host memory itself, each direction alone and both at
// once.
typedef uint32_t link_u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void link_copy_kernel(const link_u32x4* __restrict__ src, link_u32x4* __restrict__ dst, size_t n16)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

struct LinkProbe {
    static constexpr int kLanes = 2;  // transfers in flight per direction
    size_t bytes = 0;                 // per transfer
    void* host[2][kLanes] = {};       // [direction][lane]
    void* dev[2][kLanes] = {};
    hipStream_t stream[2][kLanes] = {};

    int init(size_t total_bytes)
    {
        bytes = total_bytes / kLanes & ~static_cast<size_t>(255);
        for (int d = 0; d < 2; ++d)
            for (int l = 0; l < kLanes; ++l) {
                hipError_t e = hipStreamCreateWithFlags(&stream[d][l], hipStreamNonBlocking);
                if (e == hipSuccess) e = hipHostMalloc(&host[d][l], bytes, hipHostMallocDefault);
                if (e == hipSuccess) e = hipMalloc(&dev[d][l], bytes);
                if (e != hipSuccess) {
                    (void)hipGetLastError();
                    return fth::fail(e == hipErrorOutOfMemory ? FT_ENOMEM : FT_EHIP, "link probe set-up failed: %s", hipGetErrorString(e));
                }
                memset(host[d][l], 1, bytes);  // touch the pages
                link_copy_kernel<<<1024, 256, 0, stream[d][l]>>>(static_cast<const link_u32x4*>(dev[d][l]), static_cast<link_u32x4*>(dev[d][l]), 0);
                e = hipMemcpyAsync(dev[d][l], host[d][l], bytes, hipMemcpyHostToDevice, stream[d][l]);
                if (e == hipSuccess) e = hipStreamSynchronize(stream[d][l]);
                if (e != hipSuccess) {
                    (void)hipGetLastError();
                    return fth::fail(FT_EHIP, "link probe set-up failed: %s", hipGetErrorString(e));
                }
            }
        return FT_OK;
    }

    void release()
    {
        for (int d = 0; d < 2; ++d)
            for (int l = 0; l < kLanes; ++l) {
                if (stream[d][l]) (void)hipStreamDestroy(stream[d][l]);
                if (host[d][l]) (void)hipHostFree(host[d][l]);
                if (dev[d][l]) (void)hipFree(dev[d][l]);
            }
    }

    // One transfer of direction d (0 = host to device, 1 = device to host) on lane l.
    hipError_t transfer(int d, int l, bool kernel)
    {
        void* src = d == 0 ? host[d][l] : dev[d][l];
        void* dst = d == 0 ? dev[d][l] : host[d][l];
        if (!kernel) return hipMemcpyAsync(dst, src, bytes, d == 0 ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost, stream[d][l]);
        link_copy_kernel<<<2048, 256, 0, stream[d][l]>>>(static_cast<const link_u32x4*>(src), static_cast<link_u32x4*>(dst), bytes / 16);
        return hipGetLastError();
    }

    // GB/s (1e9 bytes/s) summed over the directions in `mask` (bit 0: H2D, bit 1: D2H), direction d
    // carried by a copy kernel when kernel[d], by the runtime's copies otherwise: the better of
    // one and of two transfers in flight per direction (on this platform two in flight help a single
    // direction a little and hurt both directions at once a lot: 70 against 97 GB/s).
    int measure(int mask, bool kernel_h2d, bool kernel_d2h, int iters, double* gbps)
    {
        const bool kernel[2] = {kernel_h2d, kernel_d2h};
        *gbps = 0.0;
        for (int lanes = 1; lanes <= kLanes; ++lanes)
            for (int timed = 0; timed < 2; ++timed) {  // the first pass warms up
                const int reps = timed == 0 ? 1 : iters * (kLanes / lanes);
                const auto t0 = std::chrono::steady_clock::now();
                for (int i = 0; i < reps; ++i)
                    for (int l = 0; l < lanes; ++l)
                        for (int d = 0; d < 2; ++d)
                            if (mask & (1 << d)) FT_HIP(transfer(d, l, kernel[d]));
                for (int d = 0; d < 2; ++d)
                    for (int l = 0; l < kLanes; ++l) FT_HIP(hipStreamSynchronize(stream[d][l]));
                const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
                const int dirs = (mask & 1) + ((mask >> 1) & 1);
                const double rate = static_cast<double>(bytes) * lanes * reps * dirs / sec / 1e9;
                if (timed == 1 && rate > *gbps) *gbps = rate;
            }
        return FT_OK;
    }

    int run(int iters, ft_link_probe_t* out)
    {
        int rc;
        if ((rc = measure(1, false, false, iters, &out->h2d_copy)) != FT_OK) return rc;
        if ((rc = measure(2, false, false, iters, &out->d2h_copy)) != FT_OK) return rc;
        if ((rc = measure(3, false, false, iters, &out->both_copy)) != FT_OK) return rc;
        if ((rc = measure(1, true, true, iters, &out->h2d_kernel)) != FT_OK) return rc;
        if ((rc = measure(2, true, true, iters, &out->d2h_kernel)) != FT_OK) return rc;
        if ((rc = measure(3, true, true, iters, &out->both_kernel)) != FT_OK) return rc;
        // the two mixed pairings: one direction by the runtime's copies, the other by a copy kernel
        if ((rc = measure(3, false, true, iters, &out->both_copy_in_kernel_out)) != FT_OK) return rc;
        return measure(3, true, false, iters, &out->both_kernel_in_copy_out);
    }
};

}  // namespace

extern "C" {

int ft_pinned_alloc(size_t bytes, void** out)
{
    if (!out) return fth::fail(FT_EINVAL, "out must not be NULL");
    *out = nullptr;
    if (bytes == 0) return FT_OK;
    void* p = nullptr;
    hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fth::fail(FT_ENOMEM, "hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    *out = p;
    return FT_OK;
}

int ft_pinned_free(void* ptr)
{
    if (!ptr) return FT_OK;
    FT_HIP(hipHostFree(ptr));
    return FT_OK;
}

int ft_offload_create(size_t chunk_elems, int n_slots, void** out_handle)
{
    if (!out_handle) return fth::fail(FT_EINVAL, "out_handle must not be NULL");
    *out_handle = nullptr;
    if (chunk_elems == 0 || (chunk_elems & 3) != 0)
        return fth::fail(FT_EINVAL, "chunk_elems must be a positive multiple of 4, got %zu", chunk_elems);
    if (n_slots < 2 || n_slots > 16) return fth::fail(FT_EINVAL, "n_slots must be in [2, 16], got %d", n_slots);

    Engine* e = new Engine();
    e->chunk = chunk_elems;
    e->slots.resize(n_slots);
    auto bail = [&](hipError_t err, const char* what) {
        (void)hipGetLastError();
        destroy_engine(e);
        return fth::fail(err == hipErrorOutOfMemory ? FT_ENOMEM : FT_EHIP, "%s failed: %s", what,
                         hipGetErrorString(err));
    };
    hipError_t err;
    if ((err = hipGetDevice(&e->device)) != hipSuccess) return bail(err, "hipGetDevice");
    if ((err = hipStreamCreateWithFlags(&e->s_h2d, hipStreamNonBlocking)) != hipSuccess) return bail(err, "hipStreamCreate");
    if ((err = hipStreamCreateWithFlags(&e->s_k, hipStreamNonBlocking)) != hipSuccess) return bail(err, "hipStreamCreate");
    if ((err = hipStreamCreateWithFlags(&e->s_d2h, hipStreamNonBlocking)) != hipSuccess) return bail(err, "hipStreamCreate");
    if ((err = hipEventCreateWithFlags(&e->ev_user, hipEventDisableTiming)) != hipSuccess) return bail(err, "hipEventCreate");
    if ((err = hipEventCreate(&e->ev_begin)) != hipSuccess) return bail(err, "hipEventCreate");
    if ((err = hipEventCreate(&e->ev_end)) != hipSuccess) return bail(err, "hipEventCreate");
    if ((err = hipEventCreate(&e->ev_kernels)) != hipSuccess) return bail(err, "hipEventCreate");
    for (size_t i = 0; i < kMaxPending; ++i) {
        hipEvent_t ev = nullptr;
        if ((err = hipEventCreateWithFlags(&ev, hipEventDisableTiming)) != hipSuccess) return bail(err, "hipEventCreate");
        e->free_events.push_back(ev);
    }
    for (Slot& s : e->slots) {
        if ((err = hipMalloc(reinterpret_cast<void**>(&s.p), chunk_elems * 4)) != hipSuccess) return bail(err, "hipMalloc");
        if ((err = hipMalloc(reinterpret_cast<void**>(&s.m), chunk_elems * 4)) != hipSuccess) return bail(err, "hipMalloc");
        if ((err = hipMalloc(reinterpret_cast<void**>(&s.v), chunk_elems * 4)) != hipSuccess) return bail(err, "hipMalloc");
        if ((err = hipEventCreateWithFlags(&s.h2d_done, hipEventDisableTiming)) != hipSuccess) return bail(err, "hipEventCreate");
        if ((err = hipEventCreateWithFlags(&s.k_done, hipEventDisableTiming)) != hipSuccess) return bail(err, "hipEventCreate");
        if ((err = hipEventCreateWithFlags(&s.d2h_done, hipEventDisableTiming)) != hipSuccess) return bail(err, "hipEventCreate");
    }
    *out_handle = e;
    return FT_OK;
}

int ft_offload_destroy(void* handle)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    (void)hipStreamSynchronize(e->s_h2d);
    (void)hipStreamSynchronize(e->s_k);
    (void)hipStreamSynchronize(e->s_d2h);
    destroy_engine(e);
    return FT_OK;
}

int ft_offload_step(void* handle, int id, uint64_t step, float lr, float beta1, float beta2, float eps,
                    float weight_decay, int bias_correction, float grad_mult, void* host_p, const void* g,
                    int g_dtype, int g_on_host, void* host_m, void* host_v, void* half_out, int half_dtype,
                    int half_on_host, size_t n, const void* ctl, void* stream)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    fth::AdamObject o;
    int rc = fth::find_adam(id, &o);
    if (rc != FT_OK) return rc;
    if (n == 0) return FT_OK;
    if (!host_p || !host_m || !host_v || !g) return fth::fail(FT_EINVAL, "p, m, v and g must not be NULL");
    if (g_dtype != FT_F32 && g_dtype != FT_F16 && g_dtype != FT_BF16)
        return fth::fail(FT_EINVAL, "unknown gradient dtype code %d", g_dtype);
    if (half_out && half_dtype != FT_F16 && half_dtype != FT_BF16)
        return fth::fail(FT_EINVAL, "low-precision copy must be FT_F16 or FT_BF16, got %d", half_dtype);
    if ((rc = require_pinned(host_p, "params")) != FT_OK) return rc;
    if ((rc = require_pinned(host_m, "exp_avg")) != FT_OK) return rc;
    if ((rc = require_pinned(host_v, "exp_avg_sq")) != FT_OK) return rc;
    if (g_on_host && (rc = require_pinned(g, "grads")) != FT_OK) return rc;
    if (half_out && half_on_host && (rc = require_pinned(half_out, "low-precision copy")) != FT_OK) return rc;

    Window* window = nullptr;
    size_t window_off = 0;
    if ((rc = find_window(e, host_p, host_m, host_v, n, &window, &window_off)) != FT_OK) return rc;

    const size_t gsz = g_dtype == FT_F32 ? 4 : 2;
    const ftk::AdamConsts c =
        fth::make_consts(step, lr, beta1, beta2, eps, weight_decay, bias_correction != 0, o.adamw_mode, grad_mult);
    hipStream_t user = static_cast<hipStream_t>(stream);

    // Host ranges this step writes back to. A later step that touches any of them must not start
    // reading before this step's last D2H; steps on disjoint memory (other units, other parameter
    // groups) are free to overlap with it.
    Pending mine;
    auto add_range = [&](const void* ptr, size_t bytes) {
        mine.lo[mine.ranges] = reinterpret_cast<uintptr_t>(ptr);
        mine.hi[mine.ranges] = reinterpret_cast<uintptr_t>(ptr) + bytes;
        ++mine.ranges;
    };
    add_range(host_p, n * 4);
    add_range(host_m, n * 4);
    add_range(host_v, n * 4);
    if (half_out && half_on_host) add_range(half_out, n * 2);

    // How the state crosses the link (see ft_offload_set_mode). Staged = SDMA copy through a device
    // buffer slot; direct = the update kernel itself reads or writes the pinned host arrays.
    // Automatic: staged for large steps, but only while the burst of chunks enqueued since the
    // pipeline was last idle stays short (see kMaxChunksPerStep: the same limit holds across calls;
    // 24 units x 4 staged steps run at 49 GB/s each way, x 6 at 25 GB/s); direct otherwise.
    int mode = e->mode;
    if (e->burst_chunks > 0 && hipStreamQuery(e->s_d2h) == hipSuccess && hipStreamQuery(e->s_k) == hipSuccess &&
        hipStreamQuery(e->s_h2d) == hipSuccess)
        e->burst_chunks = 0;
    (void)hipGetLastError();  // hipErrorNotReady from the queries is not an error
    if (mode == FT_OFFLOAD_AUTO) {
        const size_t chunks = (n + e->chunk - 1) / e->chunk;
        const bool fits = chunks > kMaxChunksPerStep || e->burst_chunks + chunks <= kMaxChunksPerStep;
        mode = (n >= kStagedMinElems && fits) ? FT_OFFLOAD_STAGED : FT_OFFLOAD_DIRECT;
    }
    const bool in_staged = mode == FT_OFFLOAD_STAGED || mode == FT_OFFLOAD_STAGED_IN;
    const bool out_staged = mode == FT_OFFLOAD_STAGED || mode == FT_OFFLOAD_STAGED_OUT;

    // Everything that can refuse the step is settled before anything is enqueued: what the update
    // launches check per chunk (alignment of every array to its element size, of the records to 16
    // bytes) and every allocation the step needs (larger slots for a long step, staging for
    // host-resident gradients or copy). An error therefore leaves the handle as it was, with nothing
    // of the step in flight.
    auto misaligned = [](const void* ptr, size_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) != 0; };
    if (misaligned(host_p, 4) || misaligned(host_m, 4) || misaligned(host_v, 4) || misaligned(g, gsz) ||
        (half_out && misaligned(half_out, 2)))
        return fth::fail(FT_EALIGN, "a pointer is not aligned to its element size");
    if (ctl && misaligned(ctl, 16)) return fth::fail(FT_EALIGN, "ft_step_control_t must be 16-byte aligned");
    const bool stage_g = g_on_host && in_staged;
    // With a control record the step may turn out to be a no-op, and a skipped kernel writes no
    // low-precision copy: a staged copy-back would then carry whatever the slot held before. The
    // kernel therefore writes a host-resident copy itself, over the link, and on a skip the host
    // array keeps its contents. (p, m and v need no such care: a skipped kernel whose outputs are
    // not its inputs copies the old state through.)
    const bool stage_h = half_out && half_on_host && out_staged && !ctl;
    if (!window && (in_staged || out_staged)) {
        if ((n + e->chunk - 1) / e->chunk + kRampExtraChunks > kMaxChunksPerStep) {
            const size_t mi = 1u << 20, full = kMaxChunksPerStep - kRampExtraChunks;
            const size_t grown = ((n + full - 1) / full + mi - 1) / mi * mi;
            if ((rc = resize_slots(e, grown)) != FT_OK) return rc;
        }
        if (!e->slots.back().v && (rc = resize_slots(e, e->chunk)) != FT_OK) return rc;
        for (Slot& s : e->slots) {
            if (stage_g && !s.g) {
                const hipError_t err = hipMalloc(&s.g, e->chunk * 4);
                if (err != hipSuccess) {
                    (void)hipGetLastError();
                    s.g = nullptr;
                    return fth::fail(FT_ENOMEM, "hipMalloc(%zu) for the gradient staging failed: %s", e->chunk * 4, hipGetErrorString(err));
                }
            }
            if (stage_h && !s.h) {
                const hipError_t err = hipMalloc(&s.h, e->chunk * 2);
                if (err != hipSuccess) {
                    (void)hipGetLastError();
                    s.h = nullptr;
                    return fth::fail(FT_ENOMEM, "hipMalloc(%zu) for the copy's staging failed: %s", e->chunk * 2, hipGetErrorString(err));
                }
            }
        }
    }
    // The pipeline starts after the producer of g/ctl on the caller's stream ...
    // (a step that copies nothing in -- inside a window, or with the kernel reading host memory
    // itself -- leaves the H2D stream alone)
    FT_HIP(hipEventRecord(e->ev_user, user));
    if (!window && in_staged) FT_HIP(hipStreamWaitEvent(e->s_h2d, e->ev_user, 0));
    FT_HIP(hipStreamWaitEvent(e->s_k, e->ev_user, 0));
    // ... and after the newest earlier step that wrote to the same host memory (the D2H stream is
    // in order, so that one event covers all older ones).
    if (!window && (rc = wait_for_overlapping_writebacks(e, mine, in_staged)) != FT_OK) return rc;

    // State held in an open window: the step is one in-place kernel on the device copy; nothing
    // crosses the link until the window closes.
    if (window) {
        const size_t last_piece = (window_off + n - 1) / window->piece;
        FT_HIP(hipStreamWaitEvent(e->s_k, window->piece_done[last_piece], 0));
        float* out[3] = {nullptr, nullptr, nullptr};  // nullptr = in place on the device copy
        if (window->write_through) {
            out[0] = static_cast<float*>(host_p);
            out[1] = static_cast<float*>(host_m);
            out[2] = static_cast<float*>(host_v);
        }
        rc = fth::launch_adam(c, window->dev[0] + window_off, g, g_dtype, window->dev[1] + window_off,
                              window->dev[2] + window_off, half_out, half_dtype, n,
                              static_cast<const ft_step_control_t*>(ctl), e->s_k, out[0], out[1], out[2]);
        if (rc != FT_OK) return rc;
        // Only the kernel stream is touched by most steps: the copy streams carry the windows' large
        // copies and nothing else (hundreds of small steps per iteration would otherwise add as many
        // markers to the D2H stream). The step that completes a piece -- every element of it
        // stepped since the piece was last written back -- sends that piece on its way back, so
        // that the write-back of a window runs one piece, not one window, behind its steps.
        FT_HIP(hipEventRecord(e->ev_kernels, e->s_k));
        e->stepped = true;
        if (!window->write_through) {
            Window& w = *window;
            const size_t first_piece = window_off / w.piece;
            bool waited = false;
            for (size_t k = first_piece; k <= last_piece; ++k) {
                const size_t lo = k * w.piece, hi = (lo + w.piece < w.n) ? lo + w.piece : w.n;
                const size_t a = window_off > lo ? window_off : lo, b = (window_off + n < hi) ? window_off + n : hi;
                if (w.piece_clean[k]) {  // stepped again after its write-back: that copy is stale
                    w.piece_clean[k] = 0;
                    w.piece_stepped[k] = 0;
                }
                w.piece_stepped[k] += b - a;
                if (w.piece_stepped[k] < hi - lo) continue;
                if (!waited) {
                    FT_HIP(hipEventRecord(w.piece_stepped_ev, e->s_k));
                    FT_HIP(hipStreamWaitEvent(e->s_d2h, w.piece_stepped_ev, 0));
                    waited = true;
                }
                for (int arr = 0; arr < 3; ++arr)
                    FT_HIP(hipMemcpyAsync(reinterpret_cast<float*>(w.host[arr]) + lo, w.dev[arr] + lo, (hi - lo) * 4,
                                          hipMemcpyDeviceToHost, e->s_d2h));
                w.piece_clean[k] = 1;
                w.piece_stepped[k] = 0;
            }
        }
        return FT_OK;
    }
    FT_HIP(hipEventRecord(e->ev_begin, in_staged ? e->s_h2d : e->s_k));

    float* hp = static_cast<float*>(host_p);
    float* hm = static_cast<float*>(host_m);
    float* hv = static_cast<float*>(host_v);
    const char* gb = static_cast<const char*>(g);
    char* hb = static_cast<char*>(half_out);

    const size_t chunk = e->chunk;

    // Chunk sizes of this step. Every chunk but the last starts and ends on a multiple of 256
    // elements (whole tiles at 1 KiB boundaries) whenever the chunk size itself is one.
    const size_t quarter = (chunk / 4) & ~static_cast<size_t>(255);
    const bool ramp = (in_staged || out_staged) && quarter > 0 && n / chunk >= kRampMinChunks;
    std::vector<size_t> sizes;
    if (ramp) {
        const size_t body_end = (n - 4 * quarter) & ~static_cast<size_t>(255);
        for (int k = 0; k < 4; ++k) sizes.push_back(quarter);
        for (size_t off = 4 * quarter; off < body_end; off += chunk) sizes.push_back(body_end - off < chunk ? body_end - off : chunk);
        for (int k = 0; k < 3; ++k) sizes.push_back(quarter);
        sizes.push_back(n - body_end - 3 * quarter);
    } else {
        for (size_t off = 0; off < n; off += chunk) sizes.push_back(n - off < chunk ? n - off : chunk);
    }
    size_t off = 0;
    for (size_t index = 0; index < sizes.size(); off += sizes[index], ++index) {
        const size_t cnt = sizes[index];
        float *kp = hp + off, *km = hm + off, *kv = hv + off;          // kernel inputs
        float *op = hp + off, *om = hm + off, *ov = hv + off;          // kernel outputs
        const void* kg = gb + off * gsz;
        void* kh = half_out ? static_cast<void*>(hb + off * 2) : nullptr;
        Slot* slot = nullptr;
        if (in_staged || out_staged) {
            ++e->burst_chunks;
            // Round-robin over all steps, not per step: a step that is a single chunk (one share
            // of a unit) must not queue behind the previous step's last use of the same slot.
            slot = &e->slots[e->cursor++ % e->slots.size()];
            if (slot->used) FT_HIP(hipStreamWaitEvent(in_staged ? e->s_h2d : e->s_k, slot->free_ev, 0));
        }
        if (in_staged) {
            FT_HIP(hipMemcpyAsync(slot->p, hp + off, cnt * 4, hipMemcpyHostToDevice, e->s_h2d));
            FT_HIP(hipMemcpyAsync(slot->m, hm + off, cnt * 4, hipMemcpyHostToDevice, e->s_h2d));
            FT_HIP(hipMemcpyAsync(slot->v, hv + off, cnt * 4, hipMemcpyHostToDevice, e->s_h2d));
            if (stage_g) {
                FT_HIP(hipMemcpyAsync(slot->g, gb + off * gsz, cnt * gsz, hipMemcpyHostToDevice, e->s_h2d));
                kg = slot->g;
            }
            FT_HIP(hipEventRecord(slot->h2d_done, e->s_h2d));
            FT_HIP(hipStreamWaitEvent(e->s_k, slot->h2d_done, 0));
            kp = slot->p;
            km = slot->m;
            kv = slot->v;
        }
        if (out_staged) {
            op = slot->p;
            om = slot->m;
            ov = slot->v;
            if (stage_h) kh = slot->h;
        }
        rc = fth::launch_adam(c, kp, kg, g_dtype, km, kv, kh, half_dtype, cnt,
                              static_cast<const ft_step_control_t*>(ctl), e->s_k, op, om, ov);
        if (rc != FT_OK) return rc;
        if (slot) {
            FT_HIP(hipEventRecord(slot->k_done, e->s_k));
            slot->free_ev = slot->k_done;
            slot->used = true;
        }
        if (out_staged) {
            FT_HIP(hipStreamWaitEvent(e->s_d2h, slot->k_done, 0));
            FT_HIP(hipMemcpyAsync(hp + off, slot->p, cnt * 4, hipMemcpyDeviceToHost, e->s_d2h));
            FT_HIP(hipMemcpyAsync(hm + off, slot->m, cnt * 4, hipMemcpyDeviceToHost, e->s_d2h));
            FT_HIP(hipMemcpyAsync(hv + off, slot->v, cnt * 4, hipMemcpyDeviceToHost, e->s_d2h));
            if (stage_h) FT_HIP(hipMemcpyAsync(hb + off * 2, slot->h, cnt * 2, hipMemcpyDeviceToHost, e->s_d2h));
            FT_HIP(hipEventRecord(slot->d2h_done, e->s_d2h));
            slot->free_ev = slot->d2h_done;
        }
    }
    FT_HIP(hipEventRecord(e->ev_kernels, e->s_k));
    // the write-back is complete when the D2H stream is, and (direct output) when the kernels are
    FT_HIP(hipStreamWaitEvent(e->s_d2h, e->ev_kernels, 0));
    FT_HIP(hipEventRecord(e->ev_end, e->s_d2h));
    e->stepped = true;
    e->end_recorded = true;

    return remember_writeback(e, mine);
}

int ft_offload_window_open(void* handle, void* host_p, void* host_m, void* host_v, size_t n, int write_through,
                           int* out_window)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (!out_window) return fth::fail(FT_EINVAL, "out_window must not be NULL");
    *out_window = -1;
    if (n == 0 || !host_p || !host_m || !host_v) return fth::fail(FT_EINVAL, "p, m, v must not be NULL and n must be positive");
    int rc;
    if ((rc = require_pinned(host_p, "params")) != FT_OK) return rc;
    if ((rc = require_pinned(host_m, "exp_avg")) != FT_OK) return rc;
    if ((rc = require_pinned(host_v, "exp_avg_sq")) != FT_OK) return rc;
    void* host[3] = {host_p, host_m, host_v};
    Pending mine;
    for (int a = 0; a < 3; ++a) {
        mine.lo[a] = reinterpret_cast<uintptr_t>(host[a]);
        mine.hi[a] = mine.lo[a] + n * 4;
    }
    mine.ranges = 3;
    for (Window& w : e->windows) {
        if (!w.open) continue;
        for (int a = 0; a < 3; ++a)
            for (int b = 0; b < 3; ++b)
                if (mine.lo[a] < w.host[b] + w.n * 4 && w.host[b] < mine.hi[a])
                    return fth::fail(FT_EBUSY, "this host memory already belongs to an open window");
    }
    // The window that was closed longest ago (its write-back has had the most time to finish, and
    // the new copies must wait for it); never-used ones first.
    int pick = -1;
    for (int i = 0; i < kMaxWindows; ++i) {
        const Window& w = e->windows[i];
        if (w.open) continue;
        if (pick < 0 || w.closed_at < e->windows[pick].closed_at) pick = i;
    }
    if (pick < 0) return fth::fail(FT_EBUSY, "all %d windows are open", kMaxWindows);
    Window& w = e->windows[pick];
    if (!w.k_done) FT_HIP(hipEventCreateWithFlags(&w.k_done, hipEventDisableTiming));
    if (!w.d2h_done) FT_HIP(hipEventCreateWithFlags(&w.d2h_done, hipEventDisableTiming));
    if (!w.piece_stepped_ev) FT_HIP(hipEventCreateWithFlags(&w.piece_stepped_ev, hipEventDisableTiming));
    if (w.cap < n) {
        if (w.used) FT_HIP(hipEventSynchronize(w.d2h_done));  // its last write-back still reads the old arrays
        for (float*& d : w.dev) {
            if (d) FT_HIP(hipFree(d));
            d = nullptr;
        }
        w.cap = 0;
        for (float*& d : w.dev) {
            hipError_t err = hipMalloc(reinterpret_cast<void**>(&d), n * 4);
            if (err != hipSuccess) {
                (void)hipGetLastError();
                return fth::fail(FT_ENOMEM, "hipMalloc(%zu) for a window failed: %s", n * 4, hipGetErrorString(err));
            }
        }
        w.cap = n;
    }
    // Equal pieces of about kWindowPieceElems: a short last copy would be one of the small copies
    // that make the copy engines share (see kStagedMinElems).
    const size_t piece_elems = e->window_piece_elems;
    size_t pieces = (n + piece_elems / 2) / piece_elems;
    if (pieces == 0) pieces = 1;
    const size_t piece = ((n + pieces - 1) / pieces + 3) / 4 * 4;
    pieces = (n + piece - 1) / piece;
    while (w.piece_done.size() < pieces) {
        hipEvent_t ev = nullptr;
        FT_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        w.piece_done.push_back(ev);
    }
    // The copies read host memory: behind any write-back to it that is still in flight, and behind
    // the window's own previous write-back, which still reads the device arrays.
    if ((rc = wait_for_overlapping_writebacks(e, mine)) != FT_OK) return rc;
    if (w.used) FT_HIP(hipStreamWaitEvent(e->s_h2d, w.d2h_done, 0));
    for (size_t k = 0; k < pieces; ++k) {
        const size_t off = k * piece;
        const size_t cnt = (n - off < piece) ? (n - off) : piece;
        for (int a = 0; a < 3; ++a)
            FT_HIP(hipMemcpyAsync(w.dev[a] + off, static_cast<float*>(host[a]) + off, cnt * 4, hipMemcpyHostToDevice, e->s_h2d));
        FT_HIP(hipEventRecord(w.piece_done[k], e->s_h2d));
    }
    for (int a = 0; a < 3; ++a) w.host[a] = reinterpret_cast<uintptr_t>(host[a]);
    w.n = n;
    w.piece = piece;
    w.piece_stepped.assign(pieces, 0);
    w.piece_clean.assign(pieces, 0);  // nothing stepped yet, but a close without steps still copies back (as before)
    w.write_through = write_through != 0;
    w.open = true;
    *out_window = pick;
    return FT_OK;
}

int ft_offload_window_close(void* handle, int window)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (window < 0 || window >= kMaxWindows || !e->windows[window].open)
        return fth::fail(FT_ENOENT, "window %d is not open", window);
    Window& w = e->windows[window];
    // Everything the kernel stream holds so far includes every step on this window.
    FT_HIP(hipEventRecord(w.k_done, e->s_k));
    FT_HIP(hipStreamWaitEvent(e->s_d2h, w.k_done, 0));
    // A window nobody stepped in still has its copies in flight; they must land before the way back.
    const size_t pieces = (w.n + w.piece - 1) / w.piece;
    FT_HIP(hipStreamWaitEvent(e->s_d2h, w.piece_done[pieces - 1], 0));
    Pending mine;
    for (size_t k = 0; k < pieces && !w.write_through; ++k) {
        if (w.piece_clean[k]) continue;  // written back when its last element was stepped
        const size_t off = k * w.piece;
        const size_t cnt = (w.n - off < w.piece) ? (w.n - off) : w.piece;
        for (int a = 0; a < 3; ++a)
            FT_HIP(hipMemcpyAsync(reinterpret_cast<float*>(w.host[a]) + off, w.dev[a] + off, cnt * 4, hipMemcpyDeviceToHost, e->s_d2h));
    }
    FT_HIP(hipEventRecord(w.d2h_done, e->s_d2h));
    FT_HIP(hipEventRecord(e->ev_end, e->s_d2h));
    e->stepped = true;
    e->end_recorded = true;
    for (int a = 0; a < 3; ++a) {
        mine.lo[a] = w.host[a];
        mine.hi[a] = w.host[a] + w.n * 4;
    }
    mine.ranges = 3;
    w.open = false;
    w.used = true;
    w.closed_at = ++e->window_closes;
    return remember_writeback(e, mine);
}

int ft_offload_set_window_piece(void* handle, size_t elems)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (elems != 0 && elems < (1u << 20)) return fth::fail(FT_EINVAL, "window pieces of fewer than 1 Mi elements are refused");
    e->window_piece_elems = elems ? elems : kWindowPieceElems;
    return FT_OK;
}

int ft_offload_set_mode(void* handle, int mode)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (mode < FT_OFFLOAD_AUTO || mode > FT_OFFLOAD_STAGED_OUT) return fth::fail(FT_EINVAL, "unknown offload mode %d", mode);
    e->mode = mode;
    return FT_OK;
}

int ft_offload_stream_wait(void* handle, void* stream, int what)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (what != 0 && what != 1) return fth::fail(FT_EINVAL, "what must be 0 (kernels) or 1 (write-back)");
    if (!e->stepped) return FT_OK;
    // the write-back is over when the D2H stream has passed the last step that used it and the
    // kernels (which write host memory themselves in the direct and write-through forms) are done
    if (what == 1 && e->end_recorded) FT_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), e->ev_end, 0));
    FT_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), e->ev_kernels, 0));
    return FT_OK;
}

int ft_offload_wait(void* handle)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (!e->stepped) return FT_OK;
    if (e->end_recorded) FT_HIP(hipEventSynchronize(e->ev_end));
    FT_HIP(hipEventSynchronize(e->ev_kernels));
    // everything enqueued so far has finished: nothing is pending any more
    for (Pending& pd : e->recent) e->free_events.push_back(pd.done);
    e->recent.clear();
    e->burst_chunks = 0;
    return FT_OK;
}

int ft_offload_elapsed_ms(void* handle, float* out_ms)
{
    Engine* e = as_engine(handle);
    if (!e) return fth::fail(FT_ENOENT, "not an offload handle");
    std::lock_guard<std::mutex> lock(e->mu);
    if (!out_ms) return fth::fail(FT_EINVAL, "out_ms must not be NULL");
    if (!e->end_recorded) return fth::fail(FT_EINVAL, "no step that moves data has been enqueued on this handle");
    FT_HIP(hipEventSynchronize(e->ev_end));
    FT_HIP(hipEventElapsedTime(out_ms, e->ev_begin, e->ev_end));
    return FT_OK;
}

int ft_link_probe(size_t bytes, int iters, ft_link_probe_t* out)
{
    if (!out) return fth::fail(FT_EINVAL, "out must not be NULL");
    if (bytes < (1u << 20) || iters <= 0) return fth::fail(FT_EINVAL, "need bytes >= 1 MiB and iters > 0");
    bytes &= ~static_cast<size_t>(255);
    LinkProbe probe;
    int rc = probe.init(bytes);
    if (rc == FT_OK) rc = probe.run(iters, out);
    probe.release();
    return rc;
}

int ft_link_bandwidth(size_t bytes, int iters, int direction, double* out_gbps)
{
    if (!out_gbps) return fth::fail(FT_EINVAL, "out_gbps must not be NULL");
    if (direction < 0 || direction > 2) return fth::fail(FT_EINVAL, "direction must be 0, 1 or 2");
    ft_link_probe_t r;
    int rc = ft_link_probe(bytes, iters, &r);
    if (rc != FT_OK) return rc;
    const double copy[3] = {r.h2d_copy, r.d2h_copy, r.both_copy}, kernel[3] = {r.h2d_kernel, r.d2h_kernel, r.both_kernel};
    double best = copy[direction] > kernel[direction] ? copy[direction] : kernel[direction];
    if (direction == 2) {
        if (r.both_copy_in_kernel_out > best) best = r.both_copy_in_kernel_out;
        if (r.both_kernel_in_copy_out > best) best = r.both_kernel_in_copy_out;
    }
    *out_gbps = best;
    return FT_OK;
}

}  // extern "C"
