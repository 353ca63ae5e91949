/*
 * ft_adam.h -- C ABI of libftadam.so: the optimizer-step hot path on one MI355X (gfx950).
 *
 * Every entry point takes plain pointers and sizes; no framework types cross this boundary.
 * Device pointers are HIP device (or device-accessible pinned host) addresses owned by the
 * caller and only borrowed for the call. `stream` is a hipStream_t passed as void* (NULL = the
 * null stream); all work is enqueued on it and the call returns without waiting unless stated.
 *
 * Return value: 0 on success, a negative FT_E* code on failure; ft_last_error() then gives a
 * human-readable reason for the calling thread.
 *
 * Each declaration cites the interface of the reference it replaces (paths relative to the
 * reference checkout, npz7yyk/FlexTrain 0.1.0+e829f0c).
 */
#ifndef FT_ADAM_H
#define FT_ADAM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of gradient inputs and of the low-precision parameter copy */
enum { FT_F32 = 0, FT_F16 = 1, FT_BF16 = 2 };

enum {
    FT_OK = 0,
    FT_EINVAL = -1,   /* bad argument (NULL, dtype code, size)                       */
    FT_EALIGN = -2,   /* pointer not aligned to its element size                     */
    FT_ENOENT = -3,   /* unknown optimizer id / handle                               */
    FT_EHIP = -4,     /* a HIP runtime call failed; message carries hipGetErrorString */
    FT_ENOMEM = -5,   /* allocation failed                                           */
    FT_EBUSY = -6     /* handle still has work in flight                             */
};

/* Result of the gradient statistics pass (device memory, 16 bytes, 16-byte aligned). */
typedef struct ft_grad_stats_t {
    uint64_t nonfinite; /* number of inf/nan gradient elements                        */
    double sumsq;       /* sum of squares of the finite unscaled gradient elements    */
} ft_grad_stats_t;

/* Per-step decision consumed by the update kernel on the device (16 bytes, 16-byte aligned). */
typedef struct ft_step_control_t {
    uint32_t skip;   /* non-zero: leave p, m, v and the low-precision copy untouched    */
    float grad_mult; /* g32 = (float)g * grad_mult  (= clip_coef * 1/loss_scale)        */
    float grad_norm; /* L2 norm of the unscaled gradient, for the caller's information  */
                     /* (saturates at FLT_MAX; the decision uses the fp64 value)        */
    float clip_coef; /* min(1, max_norm / (norm + 1e-6)), 1 when clipping is off        */
} ft_step_control_t;

const char* ft_last_error(void);
int ft_abi_version(void);

/* Number of HIP devices visible, or a negative code. Never initialises a context beyond what
 * hipGetDeviceCount does. */
int ft_device_count(void);

/* ---- optimizer registry ---------------------------------------------------------------
 * Replaces create_adam / destroy_adam of the reference's pybind module
 * (flextrain/ops/csrc/adam/cpu_adam.cpp:8-16, bodies cpu_adam_impl.cpp:143-181,297-302).
 * The object holds the default hyper-parameters and adamw_mode; an unknown id is an error
 * (FT_ENOENT) instead of the reference's null-pointer dereference (cpu_adam_impl.cpp:235-237).
 */
int ft_adam_create(int id, float lr, float beta1, float beta2, float eps, float weight_decay,
                   int adamw_mode, int should_log);
int ft_adam_destroy(int id);

/* ---- resident update --------------------------------------------------------------------
 * Replaces adam_update and adam_update_copy (ds_adam_step / ds_adam_step_plus_copy,
 * flextrain/ops/csrc/adam/cpu_adam_impl.cpp:212-295; arithmetic cpu_adam.h:130-216; host
 * scalars cpu_adam.h:67-102). Same argument order and meaning for
 * (id, step, lr, beta1, beta2, eps, weight_decay, bias_correction, params, grads, exp_avg,
 * exp_avg_sq[, device_params]); additions:
 *   grad_mult   the gradient is multiplied by this fp32 factor on load (1.0f = reference)
 *   g_dtype     gradients may be fp32 (as the reference requires), fp16 or bf16
 *   half_out    NULL (= adam_update) or the low-precision copy (= adam_update_copy);
 *   half_dtype  FT_F16 reproduces the reference's copy-out (simd.h:35-37); FT_BF16 writes
 *               round-to-nearest-even bfloat16
 *   ctl         NULL, or a device ft_step_control_t read by the kernel: it overrides
 *               grad_mult and can turn the whole call into a no-op (skip)
 * p, m, v: fp32, n elements, updated in place. Pointers must be aligned to their element size.
 * The vector path needs every array to reach its vector alignment (16 bytes; 8 for the 16-bit
 * arrays) after the same number of elements, which views cut at a common element offset of aligned
 * flat buffers (the reference's StepContext views) always do; the call then steps the elements in
 * front of the first 1 KiB boundary of p and behind the last whole 256-element tile separately
 * (same launch for an in-place update) so that every tile covers whole cache lines. Arrays whose
 * alignments disagree (a 16-bit copy cut at an odd element, a state array one element off) are still
 * stepped tile by tile, through accesses that assume element alignment only; the tiles then start
 * where most of the traffic falls on whole cache lines (written bytes counted twice), see
 * ft_relaxed_tile_start. The same results, at 82-85 % of the memory bandwidth instead of 85-86 %
 * (measured with one array of a 202 M-element update one element off the others; 75 % with
 * every array at another offset).
 */
int ft_adam_step(int id, uint64_t step, float lr, float beta1, float beta2, float eps,
                 float weight_decay, int bias_correction, float grad_mult, void* p, const void* g,
                 int g_dtype, void* m, void* v, void* half_out, int half_dtype, size_t n,
                 const void* ctl, void* stream);

/* ---- the step's scalars in device memory ----------------------------------------------------
 * ft_adam_step passes step, lr, the bias corrections ... to the kernel by value, as the reference
 * does per call (cpu_adam_impl.cpp:212-295); a HIP graph that records such a launch replays those
 * values. For callers that record the step once and replay it every iteration, the scalars can
 * live in device memory instead: ft_adam_hyper_fill computes the record on the HOST exactly as
 * ft_adam_step would (cpu_adam.h:67-102,148-166), the caller copies its 48 bytes to device memory
 * (a copy recorded in the graph re-reads the host staging at every replay), and ft_adam_step_hyper /
 * ft_adam_segment_t.hyper make the kernel read it from there. Same results as by value. */
typedef struct ft_adam_hyper_t {
    uint32_t words[12]; /* opaque */
} ft_adam_hyper_t;
int ft_adam_hyper_fill(int id, uint64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                       int bias_correction, float grad_mult, ft_adam_hyper_t* host_out);
int ft_adam_step_hyper(int id, const void* hyper_dev, void* p, const void* g, int g_dtype, void* m, void* v, void* half_out,
                       int half_dtype, size_t n, const void* ctl, void* stream);

/* ---- many resident updates in one launch -------------------------------------------------------
 * Replaces the loop of flextrain/optimizer.py:44-69 (one adam_update[_copy] call per StepContext;
 * flextrain/param_group.py:365-477 cuts a unit's share into one context per parameter group and
 * buffer piece, each with its own hyper-parameters and step count): every segment is what one
 * ft_adam_step call would take, and up to 16 of them run as ONE kernel launch (more segments, or
 * segments with and without a low-precision copy, are spread over a few launches). Results are
 * those of ft_adam_step segment by segment, bit for bit. Segments must not overlap one another.
 * A segment whose arrays do not share their alignment is stepped by launches of its own (see
 * ft_adam_step). In place, resident arrays only; g_dtype, half_dtype and ctl apply to all segments.
 * Nothing is allocated, copied or synchronised: the segment table travels with the launch. */
typedef struct ft_adam_segment_t {
    void* p;            /* fp32 master parameters, updated in place                       */
    const void* g;      /* gradients (g_dtype)                                             */
    void* m;            /* exp_avg                                                         */
    void* v;            /* exp_avg_sq                                                      */
    void* half_out;     /* NULL or the low-precision copy (half_dtype)                     */
    size_t n;           /* elements; 0 = nothing to do                                     */
    uint64_t step;
    float lr, beta1, beta2, eps, weight_decay;
    int32_t bias_correction;
    float grad_mult;
    int32_t reserved;   /* 0 */
    const void* hyper;  /* NULL, or a device ft_adam_hyper_t: it replaces step ... grad_mult above */
} ft_adam_segment_t;
int ft_adam_step_multi(int id, const ft_adam_segment_t* segs, int n_segs, int g_dtype, int half_dtype,
                       const void* ctl, void* stream);

/* ---- gradient statistics and the skip / clip decision -----------------------------------
 * No counterpart in the reference: it scales the loss (flextrain/engine.py:249) but never
 * unscales, checks or clips gradients, and nothing calls DynamicLossScaler.update_scale
 * (flextrain/loss_scaler.py:134-179). These entry points supply what that state machine needs.
 *
 * ft_grad_stats: one pass over g; writes (accumulate == 0) or adds (accumulate != 0) the count
 * of inf/nan elements and the sum of squares of (float)g * pre_mult into *out (device).
 * workspace: device scratch of at least ft_grad_stats_workspace_bytes() bytes, or NULL to use a
 * buffer the library keeps per (device, stream): it is allocated on first use and re-allocated when
 * a call needs a larger one (so a NULL-workspace call may allocate and wait for the device; bring
 * a workspace, or use ft_grad_accumulate_static, where that is not acceptable). Calls on different
 * streams never share a library-owned buffer.
 * The pass is ONE kernel launch: the block that delivers the last partial sum also adds them up (in
 * an order that depends on the grid only) and takes the decision, if one is asked for. It counts
 * blocks in a counter the library keeps per (device, stream) -- calls on one stream run in order and
 * share it, calls on different streams never do. A stream under graph capture gets the two-launch
 * form instead (a recorded launch may be replayed on any stream), with the same results bit for bit.
 *
 * ft_release_stream_scratch: gives back what the library keeps for `stream` on the current device
 * (the scratch buffer of NULL-workspace calls, the block counter). Waits for the stream first. Call
 * it before destroying a stream that made statistics calls; a stream that is simply used again
 * gets a new buffer and counter on its next call.
 */
size_t ft_grad_stats_workspace_bytes(void);
int ft_grad_stats(const void* g, int g_dtype, size_t n, float pre_mult, void* out, int accumulate,
                  void* workspace, size_t workspace_bytes, void* stream);
int ft_release_stream_scratch(void* stream);

/* ft_grad_accumulate: acc[i] = fma((float)g[i], scale, acc[i]) rounded to acc's type, in place;
 * scale == 1 is the plain accumulation the reference performs after every micro-batch when
 * gradients are accumulated in a wider type than they are produced in
 * (flextrain/memory/coordinator/optimizer.py:771-777), other values fold in the averaging of
 * flextrain/optimizer.py:250. zero_g != 0 also clears g, replacing the separate zeroing of the
 * receive buffer (coordinator/optimizer.py:743). With stats_out != NULL the pass also produces the
 * statistics ft_grad_stats would report for the new acc (pre-multiplied by stats_pre_mult), so
 * the last accumulation of a step makes the separate statistics pass unnecessary.
 * acc and g should start at the same element offset of their buffers (then both are moved with
 * aligned vector accesses and every tile covers whole cache lines of both); a g that does not is
 * read (through the caches rather than streamed) and cleared through accesses that assume element
 * alignment only, with the same results, 1-3 % slower. With statistics the
 * workspace must hold ft_grad_accumulate_workspace_bytes(n) bytes (16 bytes per 256 elements on
 * top of the fixed part), or be NULL for the library's own buffer. */
size_t ft_grad_accumulate_workspace_bytes(size_t n);
int ft_grad_accumulate(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                       float stats_pre_mult, void* stats_out, int stats_accumulate, void* workspace,
                       size_t workspace_bytes, void* stream);

/* ft_grad_decide / ft_grad_accumulate_decide: ft_grad_stats / ft_grad_accumulate (with statistics)
 * followed by ft_grad_control on the record as it then stands, without the extra launch: the last
 * kernel of the statistics pass writes the decision too. For the pass that completes a step's
 * statistics (the last gradient buffer, the last micro-batch). Same results as the two calls.
 * Both leave the end of what the update will read next (the last stats_keep_bytes of g, of acc: see
 * ft_set_cache_tuning) in the memory-side cache. */
int ft_grad_decide(const void* g, int g_dtype, size_t n, float pre_mult, void* stats, int accumulate, float inv_scale,
                   float max_norm, void* ctl_out, void* workspace, size_t workspace_bytes, void* stream);
int ft_grad_accumulate_decide(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                              float stats_pre_mult, void* stats, int stats_accumulate, float inv_scale, float max_norm,
                              void* ctl_out, void* workspace, size_t workspace_bytes, void* stream);

/* ft_grad_decide_dev: ft_grad_decide with 1/loss_scale read from device memory (one float, used both
 * as pre_mult and as inv_scale), for a recorded step whose loss scale changes between replays. */
int ft_grad_decide_dev(const void* g, int g_dtype, size_t n, const void* inv_scale_dev, void* stats, int accumulate,
                       float max_norm, void* ctl_out, void* workspace, size_t workspace_bytes, void* stream);

/* ft_grad_accumulate_static: ft_grad_accumulate for callers that cannot allocate (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc). No counterpart in the
 * reference. Same arguments, results and kernels as ft_grad_accumulate, without the workspace: the
 * statistics scratch is a static device array inside the library (about 16.1 MiB on every GPU the
 * library runs on, held until the process ends), so the call allocates and frees nothing, whatever
 * the size of earlier calls. At most FT_STATIC_MAX_ELEMS elements per call (FT_EINVAL beyond).
 * All calls on one GPU share that array: calls that overlap in time on one GPU (two streams, two
 * threads) race on it and must be ordered by the caller. The first call on a device looks the
 * array's address up (hipGetSymbolAddress): make that call before a graph capture begins. */
#define FT_STATIC_MAX_ELEMS (1ull << 28)
int ft_grad_accumulate_static(void* acc, int acc_dtype, void* g, int g_dtype, size_t n, float scale, int zero_g,
                              float stats_pre_mult, void* stats_out, int stats_accumulate, void* stream);

/* ft_grad_control: turns statistics into the per-step decision, on the device:
 *   skip      = stats->nonfinite != 0
 *   norm      = sqrt(stats->sumsq)                                (double)
 *   clip_coef = max_norm > 0 ? min(1, max_norm / (norm + 1e-6)) : 1   (double, then fp32)
 *   grad_mult = clip_coef * inv_scale                             (one fp32 multiply)
 */
int ft_grad_control(const void* stats, float inv_scale, float max_norm, void* ctl_out, void* stream);

/* ---- pinned host memory -------------------------------------------------------------------
 * Replaces the pinned allocations of flextrain/memory/__init__.py:255-277 and
 * flextrain/memory/pin_memory.py:100-171 (torch pin_memory, power-of-two rounded): exact-size,
 * page-aligned, device-accessible host memory from hipHostMalloc. */
int ft_pinned_alloc(size_t bytes, void** out);
int ft_pinned_free(void* ptr);

/* ---- offloaded (streamed) update --------------------------------------------------------
 * Replaces the reference's "state lives in pinned host memory, step runs where the state is"
 * arrangement (flextrain/optimizer.py:244-263; flextrain/memory/__init__.py:240-248,366-395:
 * RotateContainer double buffering and the single side stream with device-wide synchronisation)
 * by a pipeline that brings the state to the GPU in chunks: for every chunk, H2D of p/m/v
 * (+ g when it lives on the host) on one stream, the update kernel on a second, D2H of p/m/v
 * (+ the low-precision copy when it lives on the host) on a third, ordered per buffer slot by
 * events, never by a device-wide wait.
 *
 * ft_offload_create: chunk_elems elements per chunk, n_slots (>= 2) device buffer sets. A step of
 *                    more than 96 chunks makes the engine grow its chunk (and its buffers) so that
 *                    96 suffice: longer bursts of copies run markedly slower on this platform.
 * ft_offload_step:   enqueues one full step over n elements and returns; host_p/m/v are pinned
 *                    host arrays; g and half_out are device pointers when *_on_host == 0 and
 *                    pinned host pointers otherwise (half_out may be NULL). The step starts
 *                    after the work already enqueued on `stream` (the producer of g and ctl).
 *                    Steps on the same host memory run in the order they were enqueued; steps on
 *                    disjoint host memory (other units, other parameter groups) overlap.
 * ft_offload_stream_wait: makes `stream` wait, on the device, for the last enqueued step:
 *                    what == 0 for its kernels (g may then be overwritten and a device-resident
 *                    half_out read), what == 1 for its write-back to host memory.
 * ft_offload_wait:   blocks the calling thread until everything enqueued so far has finished.
 * ft_offload_elapsed_ms: device time between the first H2D and the last D2H of the last
 *                    enqueued step that ran through the pipeline (waits for it; a step inside a
 *                    window is a bare kernel and leaves this figure alone).
 */
enum {
    FT_OFFLOAD_AUTO = 0,       /* staged for steps of at least 32 Mi elements, direct for shorter ones */
    FT_OFFLOAD_STAGED = 1,     /* SDMA H2D into a slot, kernel in place on the slot, SDMA D2H            */
    FT_OFFLOAD_DIRECT = 2,     /* no copies: the kernel reads and writes the pinned host arrays itself   */
    FT_OFFLOAD_STAGED_IN = 3,  /* SDMA H2D into a slot, the kernel writes its results to host memory     */
    FT_OFFLOAD_STAGED_OUT = 4  /* the kernel reads host memory, results leave through a slot and SDMA D2H */
};
int ft_offload_create(size_t chunk_elems, int n_slots, void** out_handle);
/* How the state crosses the host link; results are identical in every mode. */
int ft_offload_set_mode(void* handle, int mode);
int ft_offload_destroy(void* handle);
int ft_offload_step(void* handle, int id, uint64_t step, float lr, float beta1, float beta2,
                    float eps, float weight_decay, int bias_correction, float grad_mult,
                    void* host_p, const void* g, int g_dtype, int g_on_host, void* host_m,
                    void* host_v, void* half_out, int half_dtype, int half_on_host, size_t n,
                    const void* ctl, void* stream);
/* Windows: where a caller steps one unit's state in many small pieces (the per-(unit, micro-batch)
 * calls of flextrain/memory/coordinator/optimizer.py:684-696), copies of a few tens of MB each use
 * the link badly. ft_offload_window_open brings the whole p, m, v of the unit (n elements each) to
 * the device with large copies and returns at once; until ft_offload_window_close, every
 * ft_offload_step whose p/m/v lie inside those arrays (same element offset in all three) runs as
 * a kernel on the device copy. write_through == 0: the kernels work in place on the device copy,
 * the host arrays are stale until the close (a piece of them may be written back earlier, when the
 * steps have covered it; the close writes back whatever is left).
 * write_through != 0: the kernels write their results straight to the host arrays (no copy back;
 * each element may be stepped at most once per window). A step may not straddle a window's edge.
 * At most 4 windows are open at a time (FT_EBUSY beyond). The reference has no counterpart: its
 * state never leaves the host. */
int ft_offload_window_open(void* handle, void* host_p, void* host_m, void* host_v, size_t n, int write_through,
                           int* out_window);
int ft_offload_window_close(void* handle, int window);
/* Windows cross the link in equal pieces of about `elems` elements per array (0 = the default,
 * 256 Mi: about 1 GiB per copy). A window of copy-back kind sends a piece on its way back as soon as
 * every element of it has been stepped, so its write-back runs one piece behind its steps; what is
 * left goes at the close. Smaller pieces shorten that lag and make more, smaller copies -- which is
 * not free. Measured on a schedule of 24 units of 202 M elements: two pieces per unit gained 1.5-2.7 %
 * with 4 to 32 steps per unit; four pieces gained 3.5 % with 8 and 16 steps per unit and halved the
 * throughput with 32, as eight pieces did with 16 (the runtime then carries both directions on one
 * copy engine). Measure before changing it. Applies to windows this handle opens afterwards. */
int ft_offload_set_window_piece(void* handle, size_t elems);
int ft_offload_stream_wait(void* handle, void* stream, int what);
int ft_offload_wait(void* handle);
int ft_offload_elapsed_ms(void* handle, float* out_ms);

/* Host-link probe used to put the offloaded step next to what the link can do. The method follows
 * the reference's own probe (flextrain/auto_config.py:184-215: timed copies between pinned host and
 * device memory), hardened into a ceiling: `bytes` are moved per direction and iteration, every
 * figure the better of one and of two transfers in flight, once with the runtime's copies (*_copy) and once with a copy
 * kernel that reads or writes the pinned memory itself (*_kernel), host-to-device alone,
 * device-to-host alone, and both at once (both_*: the SUM of the two directions), the latter also in
 * the two mixed pairings (both_copy_in_kernel_out: the runtime's copies host-to-device while a copy
 * kernel writes device-to-host; both_kernel_in_copy_out: the reverse). GB/s = 1e9 bytes/s.
 * ft_link_bandwidth returns the best of the methods for one direction code
 * (0 = host-to-device, 1 = device-to-host, 2 = both at once, summed). */
typedef struct ft_link_probe_t {
    double h2d_copy, d2h_copy, both_copy;
    double h2d_kernel, d2h_kernel, both_kernel;
    double both_copy_in_kernel_out, both_kernel_in_copy_out; /* since ABI version 3 */
} ft_link_probe_t;
int ft_link_probe(size_t bytes, int iters, ft_link_probe_t* out);
int ft_link_bandwidth(size_t bytes, int iters, int direction, double* out_gbps);

/* ---- synthetic inputs ----------------------------------------------------------------------
 * Seeded benchmark / test inputs whose element i is a pure function of (seed, substream,
 * first_index + i): 64-bit counter hash -> 24-bit uniforms -> (FT_SYNTH_NORMAL) Box-Muller with the
 * logarithm, cosine and 16-bit conversions written out in IEEE fp32 / integer operations, so the
 * device fill and the host fill give the same bits on any machine and for any chunking of a large
 * array. The reference draws its probe inputs with torch.randn on the host
 * (flextrain/optimizer.py:71-95 via flextrain/auto_config.py:281-317), which cannot be reproduced
 * elsewhere without shipping the data.
 * FT_SYNTH_NORMAL: mean 0, standard deviation `scale`; FT_SYNTH_UNIFORM: (0, scale].
 * ft_synth_fill writes device (or pinned host) memory from a kernel on `stream`;
 * ft_synth_fill_host writes host memory from the calling thread and needs no GPU. */
#define FT_SYNTH_NORMAL 0
#define FT_SYNTH_UNIFORM 1
int ft_synth_fill(void* out, int dtype, size_t n, uint64_t seed, uint32_t substream, uint64_t first_index,
                  int kind, float scale, void* stream);
int ft_synth_fill_host(void* out, int dtype, size_t n, uint64_t seed, uint32_t substream, uint64_t first_index,
                       int kind, float scale);

/* ---- launch tuning ------------------------------------------------------------------------
 * adam_waves_per_cu: how many 64-lane workgroups of the update kernel (16-bit gradients: 56 bytes
 * of loads in flight per lane) may be resident on one compute unit; kernels with fewer bytes per
 * lane (fp32 gradients more, the accumulation pass fewer) are scaled to the same bytes in flight.
 * 32 or more = no throttle. stats_blocks_per_cu: grid size of the statistics kernel in 256-thread
 * blocks per compute unit (this one changes the order of the fp64 additions, so the sum of
 * squares may move in its last bits, within the documented tolerance). A value <= 0 restores the
 * default. Otherwise speed only, never results. */
int ft_set_launch_tuning(int adam_waves_per_cu, int stats_blocks_per_cu);
/* stats_keep_bytes: how many bytes at the END of a statistics pass (ft_grad_stats, ft_grad_decide)
 * are read with caching loads, so that the update that reads the same gradients next finds them in
 * the memory-side cache; everything before is read with streaming loads. Default 256 MiB (the
 * cache of MI355X); 0 = stream everything, SIZE_MAX = cache everything. Speed only. */
int ft_set_cache_tuning(size_t stats_keep_bytes);
/* How work is cut into launches. The runtime refuses a launch of more than 2^32 - 1 work-items in
 * x, i.e. more than 67,108,863 workgroups of the 64 lanes these kernels use; an update or an
 * accumulation pass over more tiles than that (above about 1.7e10 elements) is cut into several
 * launches, and so is a many-segment call whose segments need more workgroups together.
 * ft_set_launch_limit lowers the limit (0 restores it), so that the cutting can be exercised with
 * ordinary sizes; results never depend on it. ft_launch_pieces reports how `workgroups` workgroups
 * are cut under `limit` (0 = the current one): first[k], count[k] for piece k, at most `capacity`
 * of them; returns the number of pieces. ft_segment_batches reports which launch each of n_segs
 * segments (workgroups[i] workgroups each) of a many-segment call falls into.
 * ft_relaxed_tile_start reports where ft_adam_step starts its 256-element tiles when the arrays of
 * a step do not reach their vector alignment together: given each array's address, element size (2
 * or 4) and weight (bytes moved per element, written bytes twice), the number of elements (below 64)
 * left in front of the first tile so that as much of the traffic as possible is on whole 128-byte
 * lines, and in *on_lines the arrays (bit k: array k) whose tiles then start on lines. None of the
 * three touches a GPU. */
int ft_set_launch_limit(uint64_t max_workgroups);
int ft_launch_pieces(uint64_t workgroups, uint64_t limit, uint64_t* first, uint64_t* count, int capacity);
int ft_segment_batches(const uint64_t* workgroups, int n_segs, uint64_t limit, int* batch_of);
int ft_relaxed_tile_start(const uint64_t* addresses, const uint32_t* elem_bytes, const uint32_t* weights, int count,
                          uint32_t* on_lines);
/* launches: 1 (default) = the statistics pass as one kernel launch, 2 = the partial sums and the
 * final sum as two launches (what a stream under graph capture always gets). Same results. */
int ft_set_stats_launches(int launches);

#ifdef __cplusplus
}
#endif
#endif
