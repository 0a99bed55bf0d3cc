/*
 * C ABI of the MI355X (gfx950) stochastic-rounding AdamW library.
 *
 * Plain C types only: pointers, sizes, enums-as-int.  Every entry point
 * returns 0 on success or a negative RT_E* code; rt_last_error() then holds a
 * message (with the hipError_t text where one was involved).  No exception or
 * torch type crosses this boundary.  The caller owns every tensor pointer it
 * passes in; the library owns only its handle's private workspace.
 *
 * The reference is pure Python on torch and has no FFI of its own; each entry
 * point cites the reference code whose work it takes over.
 */
#ifndef RAMTORCH_SR_ADAMW_H
#define RAMTORCH_SR_ADAMW_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RT_ABI_VERSION 4

/* error codes */
#define RT_OK 0
#define RT_EINVAL (-1)   /* bad argument (null pointer, unknown dtype, bad offset ...) */
#define RT_EHIP (-2)     /* a HIP runtime call failed; see rt_last_error() */
#define RT_ENOMEM (-3)   /* workspace allocation failed */
#define RT_EUNSUPPORTED (-4) /* valid request the kernels do not implement */

/* element types */
#define RT_DT_BF16 0
#define RT_DT_F32 1
#define RT_DT_F16 2
#define RT_DT_F64 3 /* params and states only */

/* where the rounding noise comes from */
#define RT_NOISE_PHILOX 0   /* Philox4x32-10 keyed by seed; counter from (step, tensor, element) */
#define RT_NOISE_EXPLICIT 1 /* caller-supplied int16/uint16 noise per element and array */

/* rt_tensor_desc.host_mask bits: array lives in host memory (streamed entry point only) */
#define RT_HOST_P 1u
#define RT_HOST_G 2u
#define RT_HOST_M 4u
#define RT_HOST_V 8u
/* Host arrays of this tensor may still be written by work queued on the caller's stream: uploads wait for
 * that work.  Implied for a gradient in pinned host memory; see rt_step_streamed. */
#define RT_HOST_ORDERED 16u

/*
 * Per-(param group, step) constants: the Python doubles of
 * ramtorch/stochastic_optimizers/adamw.py:173-188, each already rounded to
 * float32 exactly where an ATen call of adamw.py:190-200 would round it.
 */
typedef struct rt_scalars {
    float beta1;          /* float32(beta1)                      adamw.py:190 */
    float one_m_beta1;    /* float32(1 - beta1)                  adamw.py:190 */
    float beta2;          /* float32(beta2)                      adamw.py:191 */
    float one_m_beta2;    /* float32(1 - beta2)                  adamw.py:191 */
    float inv_bcs;        /* float32(1.0 / sqrt(1 - beta2^t))    adamw.py:187,193 */
    float eps;            /* float32(eps)                        adamw.py:194 */
    float decay;          /* float32(1 - (lr/bc) * wd)           adamw.py:188,198 */
    float neg_step_size;  /* float32(-(lr/bc))                   adamw.py:188,200 */
    float inv_loss_scale; /* grads are multiplied by this first; 1.0f = off (not in the reference) */
    float centralization; /* float32(centralization)             adamw.py:176-184; 0 = off */
    int32_t apply_decay;  /* weight_decay != 0                   adamw.py:197 */
    int32_t reserved;
} rt_scalars;

/*
 * One parameter tensor (or one contiguous piece of one).  p/m/v are updated in
 * place.  For rt_step_multi every pointer is a device address; for
 * rt_step_streamed the arrays named in host_mask are host addresses.
 */
typedef struct rt_tensor_desc {
    void* p;               /* parameter            adamw.py:168-170, 204-214 */
    const void* g;         /* gradient             adamw.py:117, 167 */
    void* m;               /* state["ema"]         adamw.py:160, 215-222 */
    void* v;               /* state["ema_squared"] adamw.py:163, 215-222 */
    const void* noise_p;   /* RT_NOISE_EXPLICIT: numel 16-bit noises per bf16 array, else NULL */
    const void* noise_m;
    const void* noise_v;
    float* dbg_p;          /* optional device fp32[numel]: values before rounding (tests) */
    float* dbg_m;
    float* dbg_v;
    const float* row_mean; /* centralization != 0: device fp32[numel/row_len] row means of g (of the unscaled,
                              unclipped gradient: a clip coefficient is applied to the mean as to the gradient).
                              NULL with row_len set (rt_step_multi only): the update kernel takes the row means
                              itself -- same summation, same bits as rt_row_means -- which saves the separate pass
                              over g; for whole tensors (elem_offset 0, numel a multiple of row_len) of 16-bit
                              arrays, 16-byte aligned, Philox noise, no debug outputs, row_len a multiple of 8
                              in [512, 32768]; RT_EINVAL otherwise */
    uint64_t numel;
    uint64_t elem_offset;  /* index of element 0 inside the logical tensor; multiple of 8 */
    uint64_t row_len;      /* elements per row (dim 0 slice) when centralization != 0 */
    uint32_t tensor_id;    /* < 2^30; part of the Philox counter */
    uint32_t step;         /* state["step"] after the increment (adamw.py:177), mod 2^32 */
    uint32_t scalars_idx;  /* index into the rt_scalars array */
    uint8_t p_dtype;       /* RT_DT_BF16 (stochastic rounding); RT_DT_F32 / F16 / F64 (plain copy_, round to nearest) */
    uint8_t g_dtype;       /* RT_DT_BF16, RT_DT_F32 or RT_DT_F16 */
    uint8_t m_dtype;       /* as p_dtype */
    uint8_t v_dtype;       /* as p_dtype */
    uint32_t host_mask;    /* RT_HOST_* bits; must be 0 for rt_step_multi */
    uint32_t reserved;
} rt_tensor_desc;

typedef struct rt_handle rt_handle;

/* ABI version of the loaded library (RT_ABI_VERSION it was built with). */
int rt_version(void);

/* Message of the calling thread's most recent failure ("" if none). */
const char* rt_last_error(void);

/*
 * Workspace for one device: table staging, reduction scratch and, on first
 * streamed use, three streams plus double-buffered device staging.
 * Replaces nothing in the reference (it allocates temporaries per tensor,
 * adamw.py:160-170); a handle is not re-entrant, distinct handles are independent.
 */
int rt_create(int device, rt_handle** out);
int rt_destroy(rt_handle* h);

/*
 * The fused step over n device-resident tensors in one launch per dtype
 * combination: replaces the per-tensor loop body of AdamW.step,
 * adamw.py:160-222 (upcast, EMA updates, denominator, decoupled decay,
 * addcdiv, three copy_stochastic_ write-backs) and the syncs of :227-232.
 * Enqueues on `stream` (a hipStream_t; NULL = default stream) and returns
 * without synchronising.
 *   d_clip_coef: optional device float; when non-NULL grads are multiplied by
 *                *d_clip_coef after unscaling (global-norm clip, not in the reference)
 *   d_skip:      optional device uint32; when non-NULL and *d_skip != 0 the
 *                launch leaves every tensor untouched (non-finite grad norm)
 */
int rt_step_multi(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                  uint32_t n_scalars, uint64_t seed, int noise_mode, const float* d_clip_coef,
                  const uint32_t* d_skip, void* stream);

/*
 * Same update for tensors whose p/m/v (and optionally g) live in pinned host
 * memory: the CPU-resident flow of adamw.py:152-170 (H2D of ema, ema_squared,
 * grad, p) and :204-222 (D2H write-back), restructured as chunks of
 * `chunk_elems` elements moved H2D / updated / moved D2H on three streams with
 * two staging buffers per array.  Waits for work already queued on `stream`
 * (grads ready) and returns after the last D2H has completed, so host memory
 * is final on return (the post-condition of the sync at adamw.py:232).
 * Results are bit-identical to rt_step_multi on the same data.
 * d_clip_coef / d_skip: as for rt_step_multi (device pointers, may be NULL);
 * they must be final for work queued on `stream` before the call.
 * Ordering against `stream`: the update kernels always wait for the work queued
 * on it.  This call, which returns only when everything is done, also waits
 * for `stream` on the host before it uploads anything (unless an asynchronous
 * call on the handle is still running), so whatever that work writes into host
 * arrays -- a gradient copied down with grad.to("cpu", non_blocking=True), a
 * parameter refreshed with p.copy_(gpu_tensor, non_blocking=True) -- is final.
 * rt_step_streamed_async cannot wait on the host: there the uploads wait for
 * `stream` only for tensors whose gradient lies in pinned host memory or that
 * carry RT_HOST_ORDERED, and host-resident p / m / v are otherwise taken to be
 * final in host memory when the call is made.
 * Host arrays need not be pinned (plain CPU tensors, adamw.py:152-170; the
 * gradients that ramtorch's Linear.backward leaves in ordinary CPU memory,
 * linear.py:416-427, shipped up at adamw.py:167): on the way up they are
 * copied into pinned bounce buffers of the handle (4 per array, one chunk
 * each) by a few host threads while earlier chunks are on the link, on the way
 * down (updated p / m / v, adamw.py:204-222) they land in such buffers and the
 * threads copy them out, and the call hands the pipeline one chunk at a time.
 * RT_STREAM_BOUNCE_THREADS in the environment sets the number of threads
 * (default 8; 0 leaves such copies to the runtime, which stages them while the
 * calling thread waits).
 */
int rt_step_streamed(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                     uint32_t n_scalars, uint64_t seed, int noise_mode, uint64_t chunk_elems,
                     const float* d_clip_coef, const uint32_t* d_skip, void* stream);

/*
 * rt_step_streamed without the final wait, for callers that update one tensor
 * at a time while other GPU work is still being queued (for instance from the
 * post-accumulate-grad hook that ramtorch/modules/linear.py:97-111 invokes
 * inside backward, instead of the D2H + H2D round trip of the gradient in
 * linear.py:416-427 / adamw.py:167).  Returns as soon as everything is
 * enqueued (a call of more than 64 chunks is queued in batches of 64 and
 * sleeps between them until the previous batch has left the pipeline);
 * *ticket (optional) identifies the call.  Until the ticket has
 * completed the caller must keep every array of the call alive and must not
 * touch p / m / v.  Calls on one handle run in order and share the staging
 * buffers, so consecutive calls overlap like the chunks of one call.
 *   rt_streamed_completed: highest ticket whose copies have all landed (non-blocking)
 *   rt_streamed_wait:      blocks until everything enqueued so far has finished
 */
int rt_step_streamed_async(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                           uint32_t n_scalars, uint64_t seed, int noise_mode, uint64_t chunk_elems,
                           const float* d_clip_coef, const uint32_t* d_skip, void* stream, uint64_t* ticket);
int rt_streamed_wait(rt_handle* h);
int rt_streamed_completed(rt_handle* h, uint64_t* ticket_done);

/*
 * The chunk schedule rt_step_streamed would use, without touching a GPU: one
 * row of five uint64 per piece: chunk index, tensor index, first element inside
 * the tensor, element count, element offset inside the staging buffers.
 * *n_out receives the number of pieces; at most `cap` rows are written to
 * `out` (may be NULL).  Uses only numel of each desc.
 */
int rt_streamed_plan(const rt_tensor_desc* descs, uint32_t n, uint64_t chunk_elems, uint64_t* out, uint32_t cap,
                     uint32_t* n_out);

/*
 * The order of operations of a streamed call, without touching a GPU: what the
 * library itself executes for a call over n_chunks chunks, one rt_sched_op per
 * operation in the order the host issues them.  The reference keeps its own
 * staging buffers apart with ping-pong buffers and events
 * (ramtorch/modules/linear.py:163-197, 267-308) and full-device syncs
 * (adamw.py:227-232); here the discipline is this list, and it can be replayed
 * on a CPU under any interleaving of the three streams to check that no
 * staging or bounce buffer is written while something still reads it.
 *   seq0:         chunks the handle has processed before this call (chunk c
 *                 uses staging buffer (seq0 + c) % 2 and bounce slot (seq0 + c) % 4)
 *   used_mask:    bit b set: staging buffer b holds a chunk of an earlier call
 *                 whose download the first upload into it must await
 *   paced_up:     some uploaded host array is not pinned (goes up through bounce slots)
 *   paced_down:   some updated host array is not pinned (comes down through bounce slots)
 *   batch_chunks: chunks queued at once when nothing is paced (0 = all)
 * *n_out receives the number of operations; at most `cap` are written to `out`
 * (may be NULL).
 */
enum {
    RT_OP_HOST_WAIT_BACK = 0, /* host sleeps until `value` chunks have come back (a counter published behind each) */
    RT_OP_HOST_FILL = 1,      /* host threads start copying chunk's unpinned arrays into upload bounce slot `bounce` */
    RT_OP_HOST_WAIT_FILL = 2, /* host waits until those copies are done */
    RT_OP_HOST_DRAIN = 3,     /* host threads start copying chunk's results out of download bounce slot `bounce` */
    RT_OP_HOST_WAIT_DRAIN = 4,/* host waits until those copies are done */
    RT_OP_H2D = 5,            /* upload stream: host arrays (or upload slot `bounce`) -> staging buffer `stage` */
    RT_OP_KERNEL = 6,         /* compute stream: update in staging buffer `stage` */
    RT_OP_D2H = 7,            /* download stream: staging buffer `stage` -> host arrays (or download slot `bounce`) */
    RT_OP_PUBLISH = 8,        /* download stream: the chunk counter becomes `value` */
    RT_OP_TICKET = 9,         /* download stream: the call's ticket is published */
    RT_OP_HOST_WAIT_IDLE = 10 /* host waits until every earlier call on the handle has finished (a paced call starts
                                 with it: the bounce slots and the chunk counter are shared with those calls) */
};
enum { RT_EV_H2D_DONE = 0, RT_EV_COMP_DONE = 2, RT_EV_D2H_DONE = 4 }; /* + staging buffer index */
#define RT_SCHED_NONE 0xFFFFFFFFu
typedef struct rt_sched_op {
    uint32_t kind;         /* RT_OP_* */
    uint32_t chunk;        /* chunk of the call the operation belongs to */
    uint32_t stage;        /* staging buffer, or RT_SCHED_NONE */
    uint32_t bounce;       /* bounce slot, or RT_SCHED_NONE */
    uint32_t wait_event;   /* stream operations: event waited for before it starts, or RT_SCHED_NONE */
    uint32_t record_event; /* stream operations: event recorded behind it, or RT_SCHED_NONE */
    uint64_t value;        /* RT_OP_HOST_WAIT_BACK, RT_OP_PUBLISH */
} rt_sched_op;
int rt_streamed_schedule(uint32_t n_chunks, uint64_t seq0, uint32_t used_mask, int paced_up, int paced_down,
                         uint64_t batch_chunks, rt_sched_op* out, uint32_t cap, uint32_t* n_out);

/*
 * Global gradient norm over n device tensors (uses g, g_dtype, numel of each
 * desc), for the optional clip / skip check; not in the reference.  Writes to
 * d_out (device, 16-byte aligned):
 *   float  d_out[0] = total L2 norm of g * inv_loss_scale
 *   float  d_out[1] = min(1, max_norm / (total + 1e-6))   (torch clip_grad_norm_ semantics)
 *   uint32 d_out[2] = 1 if the norm is not finite, else 0
 * Two deterministic passes (per-workgroup partials, then one reducing
 * workgroup); no atomics, so the result is reproducible run to run.
 */
int rt_grad_norm(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, float inv_loss_scale,
                 float max_norm, void* d_out, void* stream);

/*
 * rt_grad_norm for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  Same arguments, same result bit for bit,
 * but the per-workgroup partial sums and the gradient table live in a fixed
 * 144 KiB device array that is part of the library's code object (one copy per
 * GPU, held until the process ends), the table travels there as kernel
 * arguments, and the call performs no hipMalloc / hipFree / hipHostMalloc.
 * Limit: at most 4096 gradients with numel != 0 per call; more returns
 * RT_EUNSUPPORTED.  Every call on one GPU uses that GPU's one array.  Outside
 * stream capture the calls take turns on the GPU, whichever handle or stream
 * they come from: each waits for an event recorded behind the previous one
 * (the event exists since rt_create; nothing is allocated per call).  Under
 * stream capture no event is used, and replays of graphs that contain such
 * calls race if they overlap on a GPU: their owner has to order them.
 */
int rt_grad_norm_static(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, float inv_loss_scale,
                        float max_norm, void* d_out, void* stream);

/*
 * Row means of g over all dims but the first, for gradient centralization
 * (adamw.py:179-184): d_row_mean[r] = mean(g[r, ...]) in fp32.
 */
int rt_row_means(rt_handle* h, const void* g, int g_dtype, uint64_t rows, uint64_t row_len,
                 float inv_loss_scale, float* d_row_mean, void* stream);

/*
 * The same for many gradients in one launch: for every tensor with a non-NULL
 * row_mean, row_mean[r] = mean of row r of g (numel / row_len rows of row_len
 * elements, numel a multiple of row_len; row_mean is written, not read).  Only
 * g, g_dtype, numel, row_len and row_mean of a descriptor are used.  Same
 * summation, and so the same bits, as rt_row_means.
 */
int rt_row_means_multi(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, float inv_loss_scale, void* stream);

/*
 * copy_stochastic_(target, source, seed) of adamw.py:6-30: fp32 device source
 * -> bf16 device target.  noise == NULL: Philox keyed by seed; else explicit
 * 16-bit noise per element.
 */
int rt_sr_copy(void* target_bf16, const float* source, uint64_t numel, const void* noise,
               uint64_t seed, void* stream);

/*
 * Timing of rt_step_multi launches on this handle, measured with HIP events
 * attached to the update kernels' own dispatches on the launch stream (start
 * of the first kernel of a call, end of its last; a pair per call, nothing is
 * read or waited for while launches are being queued).
 * Measurement only; nothing in the reference corresponds to it.
 *   rt_set_timing(h, 1): start recording (and forget earlier launches); (h, 0): stop
 *   rt_last_kernel_ms:   duration of the most recent timed launch; blocks until it has finished
 *   rt_kernel_ms_history: durations of the min(cap, 256, launches since rt_set_timing) most
 *                        recent timed launches, oldest first; blocks until they have finished
 */
int rt_set_timing(rt_handle* h, int enabled);
int rt_last_kernel_ms(rt_handle* h, float* ms);
int rt_kernel_ms_history(rt_handle* h, float* out_ms, uint32_t cap, uint32_t* n_out);

/*
 * Diagnostic, not in the reference: runs the memory traffic of the all-bf16
 * update (read p, g, m, v; write p, m, v in place; 14 bytes per element, same
 * chunking) without the arithmetic, `reps` times after one warm-up, and
 * returns the mean milliseconds per pass.  14 * numel / time is the rate this
 * access pattern can reach on the device: the practical ceiling the update
 * kernel is compared with.  The arrays are bf16-sized scratch of `numel`
 * elements (a multiple of 8192), 16-byte aligned; p, m, v are overwritten
 * (each with itself xor g, so arrays of zeros stay zeros).  Blocks until done.
 * The rate depends on where the four arrays lie in HBM (about 5.7 TB/s on
 * MI355X with all of them in one region, 6.4 TB/s with one written array in
 * another); callers that own their allocations can use this to choose a
 * placement, as the Python optimizer does for its states.
 */
int rt_stream_probe(rt_handle* h, void* p, const void* g, void* m, void* v, uint64_t numel, int reps,
                    float* ms_out, void* stream);

/*
 * Measurement only, nothing in the reference corresponds to it: what the host
 * link gives plain pinned copies of `bytes` bytes, on the handle's own copy
 * streams: out[0] = GB/s host to device, out[1] = GB/s device to host, each
 * alone; out[2] = GB/s each way with both directions running at once (what the
 * streamed pipeline does in steady state).  `reps` copies per figure after one
 * warm-up copy.  Allocates and frees its own buffers; blocks until done.
 */
int rt_host_link_probe(rt_handle* h, uint64_t bytes, int reps, double out[3]);

/*
 * Device memory that is only held, not used: the state-placement search of the
 * Python optimizer occupies memory with such blocks so that its next
 * allocation lands further on in physical address order (see rt_stream_probe),
 * without going through -- and leaving blocks behind in -- the caller's own
 * caching allocator.  Nothing in the reference corresponds to it.
 * rt_dev_hold returns RT_ENOMEM when the device has no such block left.
 * rt_dev_release accepts h == NULL (the block's device is found by its address).
 */
int rt_dev_hold(rt_handle* h, uint64_t bytes, void** out);
int rt_dev_release(rt_handle* h, void* p);

/*
 * Two zeroed device blocks of at least bytes_a and bytes_b for arrays that an
 * update reads and writes together (the optimizer's ema and ema_squared pools),
 * placed so that the two never share an HBM region (see rt_stream_probe): *a
 * and *b.  Nothing in the reference corresponds to it.  The blocks are built
 * from physical chunks of 1 GiB taken one by one through the virtual-memory
 * API (hipMemCreate), each probed with the update's traffic -- p, g, ema in the
 * first chunk, ema_squared at the chunk's two ends -- and sorted into "with the
 * first chunk" and "elsewhere"; one block is mapped from chunks of the first
 * kind, the other from chunks of the second, side by side in an address range
 * of its own.  Chunk by chunk, so it works as well in a process whose earlier
 * allocations have left the free memory in scattered order, where one large
 * allocation straddles regions.  On the way the search holds at most
 * max_extra_bytes more than the two blocks and gives up when taking and
 * probing chunks beyond those of the blocks has cost max_seconds (two and a
 * half times that while the driver hands out chunks slowly because it is
 * still clearing memory that was given back shortly before);
 * blocks it could not complete from the right kind of chunk are completed with
 * others.  Each block is given back with rt_dev_release (which waits for the
 * device first).  RT_EUNSUPPORTED when the runtime has no such allocations.
 * ref_p, ref_m, ref_v, ref_elems (optional, ref_elems == 0: none): three
 * disjoint 16-byte-aligned arrays of ref_elems 16-bit elements in the memory
 * of the parameters the blocks will be used with (ref_elems a multiple of
 * 8192 between 2^25 and 2^27).  The probes then run with the first two as p
 * and ema, and the third as ema_squared gives the rate of the parameters' own
 * region, so that the kinds are "with the parameters" (no faster than that)
 * and "elsewhere" (3.5 % faster at least): *a is built from
 * the first kind (or, when that region has too few free chunks, from the
 * second as well), *b from the second, and an update never has p, ema and
 * ema_squared in one region nor, with *a complete, in three.  The probe
 * writes the reference arrays back bit for bit as they are (it stores p ^ g
 * with g zero); nothing else may write them while the call runs.  Reference
 * arrays that do not lie in one region themselves (the probe with all of
 * them runs faster than with all arrays inside one chunk) are not used.
 *   report[0] = 1 when both blocks are wholly of their kind, else 0
 *   report[1] = share of the second block that lies apart from the first
 *   report[2] = chunks taken and probed       report[3] = seconds
 *   report[4], report[5] = GB/s of the probe within one region / across two
 *   report[6] = why the search ended: 0 complete, 1 memory limit, 2 time limit, 3 no free chunk left
 *   report[7] = 2 when the kinds were told apart relative to the reference arrays (*a lies with them), else
 *               1 when *a is the block in the first chunk's region, 0 when *b is
 */
int rt_dev_hold_pair(rt_handle* h, uint64_t bytes_a, uint64_t bytes_b, uint64_t max_extra_bytes, double max_seconds,
                     void* ref_p, void* ref_m, void* ref_v, uint64_t ref_elems, void** a, void** b,
                     double report[8], void* stream);

/*
 * Self-test, nothing in the reference corresponds to it.  The update kernels
 * take the square root of the second moment (adamw.py:193) with a shortened
 * instruction sequence whenever a whole wavefront's values lie in
 * [2^-96, +inf).  This runs that sequence and the compiler's correctly rounded
 * sqrtf over every float of that range on the device and returns the number of
 * bit patterns whose results differ (expected: 0).  Blocks until done.
 */
int rt_selftest_sqrt(rt_handle* h, uint64_t* mismatches);

/*
 * Streamed-path statistics of the most recent rt_step_streamed:
 * out[0] = bytes H2D, out[1] = bytes D2H, out[2] = wall seconds of the call.
 */
int rt_streamed_stats(rt_handle* h, double out[3]);

/*
 * How often the streamed path met host arrays that are not pinned, since the
 * handle was created: out[0] = calls that went through the bounce buffers,
 * out[1] = bytes the host threads copied into them.
 */
int rt_streamed_bounce_stats(rt_handle* h, uint64_t out[2]);

/*
 * Per-chunk timeline of the most recent rt_step_streamed made while timing was
 * enabled (rt_set_timing): four floats per chunk, milliseconds since the first
 * H2D began: H2D begin, H2D end, D2H begin, D2H end.  *n_out receives the
 * number of floats available; at most `cap` are written to `out` (may be NULL).
 */
int rt_streamed_timeline(rt_handle* h, float* out, uint32_t cap, uint32_t* n_out);

#ifdef __cplusplus
}
#endif
#endif /* RAMTORCH_SR_ADAMW_H */
