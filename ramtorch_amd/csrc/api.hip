// Host side of the C ABI declared in include/ramtorch_sr_adamw.h: argument
// checks, the device-side tensor / chunk tables, kernel dispatch by dtype
// combination, and the streamed (host-resident) pipeline.  gfx950 only.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <chrono>
#include <cstdarg>
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <climits>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "copy_pool.h"
#include "kernels.h"

using namespace rt;

// ---------------------------------------------------------------------------
// error reporting
// ---------------------------------------------------------------------------
static thread_local char g_err[512] = "";

static int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                          \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess)                                                                  \
            return fail(RT_EHIP, "%s failed: %s (%d) at %s:%d", #expr, hipGetErrorString(e_), \
                        (int)e_, __FILE__, __LINE__);                                          \
    } while (0)

// ---------------------------------------------------------------------------
// handle
// ---------------------------------------------------------------------------
namespace {

constexpr int kSlots = 2;            // table staging slots (host runs at most this far ahead)
constexpr size_t kTablePool = 8;     // table images of streamed calls in flight
constexpr size_t kTablePoolBytes = 64 << 10;
constexpr int kNormPartials = 2048;  // workgroups of the norm pass
constexpr size_t kTimingRing = 256;   // timed launches whose durations can be read back
constexpr uint64_t kMaxGrid = 0x7FFFFFFFull;  // workgroups of one launch (one per chunk of 8192 elements)
constexpr int kStageBufs = 2;        // device staging buffers per array (chunks in different stages of the pipeline)
constexpr int kBounce = 4;           // pinned bounce buffers per array for host arrays that are not pinned
constexpr uint64_t kPacedInFlight = 2;  // chunks on the streams while the host feeds the pipeline chunk by chunk

struct DevBuf {
    void* ptr = nullptr;
    size_t cap = 0;
};

// One staging slot for the tables of one launch batch: pinned host image,
// device copy, and an event recorded after the kernels that read the copy.
struct TableSlot {
    DevBuf dev;
    void* host = nullptr;  // pinned; keeps the image last uploaded to `dev`
    size_t host_cap = 0;
    size_t valid_bytes = 0;  // bytes of `host` that `dev` currently mirrors
    uint64_t static_gen = 0; // layout generation of the lists behind the scalars, 0 = unknown
    hipEvent_t done = nullptr;
    bool in_flight = false;
};

struct Streamed {
    hipStream_t h2d = nullptr, comp = nullptr, d2h = nullptr;
    hipEvent_t start = nullptr;
    hipEvent_t h2d_done[kStageBufs] = {};
    hipEvent_t comp_done[kStageBufs] = {};
    hipEvent_t d2h_done[kStageBufs] = {};
    DevBuf stage[4][kStageBufs];  // [p,g,m,v][buffer]
    // Table images of every chunk of one call, back to back.  A pool, because an
    // asynchronous call may still be running when the next one builds its tables; an
    // entry is free again once the ticket of the call that used it has been published,
    // and the pool grows when there is none.  The host never waits inside the runtime
    // here (see streamed_wait).
    struct TableRing {
        DevBuf dev;
        void* host = nullptr;  // pinned image
        size_t host_cap = 0;
        uint64_t ticket = 0;  // call that reads `dev`; free again once that ticket is published
        bool in_flight = false;
    };
    std::vector<TableRing> ring;
    // The pipeline state survives across calls so that asynchronous calls chain correctly:
    uint64_t seq = 0;                      // chunks enqueued so far; chunk `seq` uses buffer seq % kStageBufs
    bool used_buf[kStageBufs] = {};        // buffer has a D2H whose completion the next H2D must await
    bool pending = false;                  // work enqueued since the last wait
    // Tickets: a one-thread kernel behind the last D2H copy of a call writes the call's number
    // into a word of pinned host memory; the host learns about completion by reading that word.
    uint64_t tickets_issued = 0;
    volatile uint64_t* ticket_word = nullptr;
    // Progress: a second pinned word (ticket_word + 1) that receives the running chunk count at
    // every batch boundary inside a long call; one call never has more than batch_chunks chunks
    // queued on the streams (RT_STREAM_BATCH_CHUNKS in the environment overrides the default).
    uint64_t batch_chunks = 64;
    bool ready = false;
    double bytes_h2d = 0, bytes_d2h = 0, seconds = 0;
    std::vector<hipEvent_t> tl_events;  // 4 per chunk when timing is on: H2D begin/end, D2H begin/end
    std::vector<float> timeline;        // ms since the first H2D began
    // Host arrays that are not pinned (ordinary CPU tensors) go up through pinned bounce buffers that
    // host threads fill while earlier chunks are on the link; see streamed_enqueue_impl.
    void* bounce[4][kBounce] = {};
    size_t bounce_cap[4] = {0, 0, 0, 0};   // bytes of each of the kBounce buffers of an array
    // The same for the way back: updated p / m / v that belong into host memory that is not pinned land in
    // these and host threads copy them out (index 1, the gradient, stays unused).
    void* bounce_down[4][kBounce] = {};
    size_t bounce_down_cap[4] = {0, 0, 0, 0};
    std::unique_ptr<CopyPool> pool;
    int bounce_threads = 8;   // RT_STREAM_BOUNCE_THREADS in the environment overrides; 0 leaves such copies to the runtime
    uint64_t paced_calls = 0, bounced_bytes = 0;
};

}  // namespace

// ---------------------------------------------------------------------------
// what one table image holds
// ---------------------------------------------------------------------------
namespace {

struct Batch {            // tensors of one dtype combination inside a table image
    uint32_t combo;
    uint32_t first_range, n_ranges, n_units;   // fast kernel: entries of the range list, fast units
    uint32_t first_piece, n_pieces;            // pieces served by the fast kernel's first workgroups
    uint32_t first_generic, n_generic;         // chunk range of the generic kernel
    uint32_t first_cen_range, n_cen_ranges, n_cen_units;  // the same lists for tensors with centralization
    // tensors whose row means the kernel takes itself, as lists of first rows: [0] rows longer than
    // kRowwiseShortMax elements, [1] the others
    uint32_t first_rw_range[2], n_rw_ranges[2], n_rw_rows[2];
};

struct Plan {
    size_t off_sets = 0, off_tensors = 0, off_ranges = 0, off_fast_tensors = 0, off_pieces = 0, off_chunks = 0,
           bytes = 0;
    uint32_t n_sets = 0, n_tensors = 0, n_chunks = 0;
    DevScalars first_set;   // passed by value when n_sets == 1
    std::vector<Batch> batches;
    std::vector<std::pair<uint32_t, uint32_t>> set_keys;  // set index -> (scalars_idx, step)
};

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// All arrays 16 bit wide: the layouts whose fast kernel has a piece path.
inline bool narrow_combo(uint32_t combo) {
    if (combo & 0x100u) return false;
    for (int k = 0; k < 4; ++k)
        if (((combo >> (2 * k)) & 3u) == RT_DT_F32) return false;
    return true;
}

}  // namespace

// ---------------------------------------------------------------------------
// Device memory of the entry point that allocates nothing (rt_grad_norm_static): the per-workgroup
// partial sums and the gradient table, in one array that is part of the loaded code object -- every
// GPU the library runs on holds its own copy at its own address until the process ends.  Host code
// never uses the array's name as an address: rt_create asks for the address once per device
// (hipGetSymbolAddress) and everything below works with that pointer.
// ---------------------------------------------------------------------------
namespace {
constexpr uint32_t kStaticMaxTensors = 4096;  // non-empty gradients per rt_grad_norm_static call
constexpr size_t kStaticPartialsBytes = kNormPartials * sizeof(double);
constexpr size_t kStaticScratchBytes = kStaticPartialsBytes + kStaticMaxTensors * sizeof(NormEntry);  // 144 KiB
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices];  // device -> address of that device's copy of `scratch`
// Every call on a device shares that device's array.  An event recorded behind the last call's kernels
// lets the next call wait for them on the GPU, whichever handle or stream it comes from, so that calls
// which would overlap take turns instead of racing.  (Not under stream capture: a graph's replays are its
// owner's to order.)
static hipEvent_t g_scratch_done[kMaxDevices];
static std::mutex g_scratch_mutex;

struct rt_handle {
    int device = 0;
    TableSlot slots[kSlots];
    uint64_t slot_counter = 0;
    DevBuf norm_partials;
    void* static_scratch = nullptr;       // this device's copy of `scratch`
    std::vector<NormEntry> norm_entries;  // host image of the table of rt_grad_norm_static
    std::vector<NormEntry> norm_table;    // the same for rt_grad_norm
    std::vector<RowMeanEntry> rowmean_table;  // host image of the table of rt_row_means_multi
    // The table image of the most recent rt_step_multi call, kept so that a call over the same tensors
    // (same addresses, sizes, types; every step count advanced by one common amount) rebuilds only
    // the per-step scalars.
    struct LayoutCache {
        bool valid = false;
        int noise_mode = 0;
        uint64_t gen = 0;
        std::vector<rt_tensor_desc> descs;
        std::vector<uint8_t> image;
        std::vector<uint8_t> cen;  // per set: centralization was on when the image was built
        Plan plan;
    } layout;
    uint64_t layout_gen = 0;
    std::vector<uint8_t> image;  // scratch for building a table image
    std::vector<DevTensor> tens;
    std::vector<uint32_t> ranges;       // first unit of each tensor of the fast kernel
    std::vector<DevTensor> fast_tens;   // their records
    std::vector<PieceRef> pieces;
    std::vector<ChunkRef> chunks;
    bool timing = false;
    // Timing: a ring of event pairs, one pair per timed launch, so that the launches of a whole
    // run can be timed without reading (and waiting for) any event in between.
    std::vector<std::pair<hipEvent_t, hipEvent_t>> tring;
    uint64_t timed_launches = 0;  // since timing was last switched on
    hipEvent_t t0 = nullptr, t1 = nullptr;  // rt_stream_probe's own pair
    Streamed st;
};

static int dev_reserve(DevBuf& b, size_t bytes) {
    if (bytes <= b.cap) return RT_OK;
    if (b.ptr) {
        HIP_TRY(hipFree(b.ptr));
        b.ptr = nullptr;
        b.cap = 0;
    }
    size_t want = std::max(bytes + bytes / 4, (size_t)4096);
    hipError_t e = hipMalloc(&b.ptr, want);
    if (e != hipSuccess) {
        b.ptr = nullptr;
        return fail(RT_ENOMEM, "hipMalloc(%zu) failed: %s", want, hipGetErrorString(e));
    }
    b.cap = want;
    return RT_OK;
}

static int dtype_size(int dt) { return dt == RT_DT_F32 ? 4 : dt == RT_DT_F64 ? 8 : 2; }

// ---------------------------------------------------------------------------
// kernel dispatch
// ---------------------------------------------------------------------------
using MultiKernel = void (*)(const LaunchArgs);

struct KernelPair {
    MultiKernel fast;     // whole fast units of aligned tensors, plus (16-bit layouts, Philox) their pieces
    MultiKernel generic;  // unaligned tensors, debug outputs, leftovers without a piece path, rows shorter than 8
    MultiKernel fast_cen; // whole fast units of aligned tensors with centralization (16-bit layouts, Philox), or NULL
    MultiKernel rowwise;  // whole tensors with centralization whose row means the kernel takes itself (same layouts), or NULL
    MultiKernel rowwise_short;  // the same for rows of at most kRowwiseShortMax elements
};

template <int P, int G, int M, int V>
static KernelPair pick_noise(int noise) {
    // combinations with an fp32 array use the lane mapping that keeps every access contiguous across the wave
    constexpr bool wide = P == RT_DT_F32 || G == RT_DT_F32 || M == RT_DT_F32 || V == RT_DT_F32;
    if constexpr (wide) {
        if (noise == RT_NOISE_EXPLICIT)
            return {sr_adamw_fast_wide_kernel<P, G, M, V, RT_NOISE_EXPLICIT>,
                    sr_adamw_generic_kernel<P, G, M, V, RT_NOISE_EXPLICIT>, nullptr, nullptr, nullptr};
        return {sr_adamw_fast_wide_kernel<P, G, M, V, RT_NOISE_PHILOX>,
                sr_adamw_generic_kernel<P, G, M, V, RT_NOISE_PHILOX>, nullptr, nullptr, nullptr};
    } else {
        if (noise == RT_NOISE_EXPLICIT)
            return {sr_adamw_fast_kernel<P, G, M, V, RT_NOISE_EXPLICIT>,
                    sr_adamw_generic_kernel<P, G, M, V, RT_NOISE_EXPLICIT>, nullptr, nullptr, nullptr};
        return {sr_adamw_fast_kernel<P, G, M, V, RT_NOISE_PHILOX>, sr_adamw_generic_kernel<P, G, M, V, RT_NOISE_PHILOX>,
                sr_adamw_fast_kernel<P, G, M, V, RT_NOISE_PHILOX, true>, sr_adamw_rowwise_kernel<P, G, M, V, false>,
                sr_adamw_rowwise_kernel<P, G, M, V, true>};
    }
}
// State dtype pairs the templated kernels are instantiated for: every bf16 / fp32 mix, and both fp16.
template <int P, int G>
static KernelPair pick_mv(int m, int v, int noise) {
    if (m == RT_DT_F16) return pick_noise<P, G, RT_DT_F16, RT_DT_F16>(noise);
    if (m == RT_DT_BF16)
        return v == RT_DT_BF16 ? pick_noise<P, G, RT_DT_BF16, RT_DT_BF16>(noise)
                               : pick_noise<P, G, RT_DT_BF16, RT_DT_F32>(noise);
    return v == RT_DT_BF16 ? pick_noise<P, G, RT_DT_F32, RT_DT_BF16>(noise) : pick_noise<P, G, RT_DT_F32, RT_DT_F32>(noise);
}
template <int P>
static KernelPair pick_g(int g, int m, int v, int noise) {
    switch (g) {
        case RT_DT_BF16: return pick_mv<P, RT_DT_BF16>(m, v, noise);
        case RT_DT_F32: return pick_mv<P, RT_DT_F32>(m, v, noise);
        default: return pick_mv<P, RT_DT_F16>(m, v, noise);
    }
}
static KernelPair pick_kernel(int p, int g, int m, int v, int noise) {
    switch (p) {
        case RT_DT_BF16: return pick_g<RT_DT_BF16>(g, m, v, noise);
        case RT_DT_F32: return pick_g<RT_DT_F32>(g, m, v, noise);
        default: return pick_g<RT_DT_F16>(g, m, v, noise);
    }
}

static inline uint32_t dtypes_of(const rt_tensor_desc& d) {
    return (uint32_t)d.p_dtype | ((uint32_t)d.g_dtype << 2) | ((uint32_t)d.m_dtype << 4) |
           ((uint32_t)d.v_dtype << 6);
}

// Tensors with an fp64 array, or with fp16 states in any other pairing than both fp16, all go to the
// one runtime-typed kernel.
constexpr uint32_t kComboAny = 0x100u;

static inline bool compiled_combo(const rt_tensor_desc& d) {
    if (d.p_dtype == RT_DT_F64 || d.m_dtype == RT_DT_F64 || d.v_dtype == RT_DT_F64) return false;
    return (d.m_dtype == RT_DT_F16) == (d.v_dtype == RT_DT_F16);
}

// Launch group of a tensor: its dtype combination when the templated kernels cover it.
static inline uint32_t combo_of(const rt_tensor_desc& d) { return compiled_combo(d) ? dtypes_of(d) : kComboAny; }

// Centralization with row_mean == NULL: whether the row-wise kernel can take this tensor
// (see sr_adamw_rowwise_kernel).
static inline bool rowwise_ok(const rt_tensor_desc& d, int noise_mode, bool allow_host) {
    const uintptr_t all = (uintptr_t)d.p | (uintptr_t)d.g | (uintptr_t)d.m | (uintptr_t)d.v;
    return !allow_host && noise_mode == RT_NOISE_PHILOX && compiled_combo(d) && d.p_dtype != RT_DT_F32 &&
           d.g_dtype != RT_DT_F32 && d.m_dtype != RT_DT_F32 && d.v_dtype != RT_DT_F32 && (all & 15u) == 0 &&
           !d.dbg_p && !d.dbg_m && !d.dbg_v && d.elem_offset == 0 && d.row_len % kVec == 0 &&
           d.row_len >= kRowwiseMinLen && d.row_len <= kWaveRowMax && d.numel % d.row_len == 0 &&
           d.numel / d.row_len <= kMaxGrid;
}

// ---------------------------------------------------------------------------
// argument validation shared by the resident and streamed entry points
// ---------------------------------------------------------------------------
static int validate(const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars, uint32_t n_scalars,
                    int noise_mode, bool allow_host) {
    if (n > 0 && descs == nullptr) return fail(RT_EINVAL, "descs is NULL with n=%u", n);
    if (n > 0 && (scalars == nullptr || n_scalars == 0)) return fail(RT_EINVAL, "scalars missing");
    if (noise_mode != RT_NOISE_PHILOX && noise_mode != RT_NOISE_EXPLICIT)
        return fail(RT_EINVAL, "unknown noise_mode %d", noise_mode);
    uint64_t total_chunks = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const rt_tensor_desc& d = descs[i];
        if (d.p_dtype > RT_DT_F64 || d.m_dtype > RT_DT_F64 || d.v_dtype > RT_DT_F64)
            return fail(RT_EINVAL, "tensor %u: unknown p/m/v dtype %d/%d/%d", i, d.p_dtype, d.m_dtype, d.v_dtype);
        if (d.g_dtype > RT_DT_F16)
            return fail(RT_EINVAL, "tensor %u: g_dtype %d (need bf16, f32 or f16)", i, d.g_dtype);
        if (d.scalars_idx >= n_scalars)
            return fail(RT_EINVAL, "tensor %u: scalars_idx %u >= %u", i, d.scalars_idx, n_scalars);
        if (d.tensor_id >= (1u << 30)) return fail(RT_EINVAL, "tensor %u: tensor_id %u >= 2^30", i, d.tensor_id);
        if (d.elem_offset & 7u)
            return fail(RT_EINVAL, "tensor %u: elem_offset %llu not a multiple of 8", i,
                        (unsigned long long)d.elem_offset);
        if (!allow_host && d.host_mask != 0)
            return fail(RT_EINVAL, "tensor %u: host_mask set on the resident entry point", i);
        if (d.numel == 0) continue;
        if (!d.p || !d.g || !d.m || !d.v) return fail(RT_EINVAL, "tensor %u: NULL array pointer", i);
        if (((uintptr_t)d.p % dtype_size(d.p_dtype)) || ((uintptr_t)d.g % dtype_size(d.g_dtype)) ||
            ((uintptr_t)d.m % dtype_size(d.m_dtype)) || ((uintptr_t)d.v % dtype_size(d.v_dtype)))
            return fail(RT_EINVAL, "tensor %u: array pointer not aligned to its element size", i);
        if (d.numel / kChunkElems >= 0xFFFFFFFFull)
            return fail(RT_EUNSUPPORTED, "tensor %u: numel %llu too large", i, (unsigned long long)d.numel);
        total_chunks += (d.numel + kChunkElems - 1) / kChunkElems;
        if (total_chunks > kMaxGrid)
            return fail(RT_EUNSUPPORTED, "more than %llu chunks of %u elements in one call",
                        (unsigned long long)kMaxGrid, kChunkElems);
        if (noise_mode == RT_NOISE_EXPLICIT) {
            if ((d.p_dtype == RT_DT_BF16 && !d.noise_p) || (d.m_dtype == RT_DT_BF16 && !d.noise_m) ||
                (d.v_dtype == RT_DT_BF16 && !d.noise_v))
                return fail(RT_EINVAL, "tensor %u: explicit noise missing for a bf16 array", i);
        }
        if (scalars[d.scalars_idx].centralization != 0.0f) {
            if (d.row_len == 0) return fail(RT_EINVAL, "tensor %u: centralization without row_len", i);
            if (!d.row_mean && !rowwise_ok(d, noise_mode, allow_host))
                return fail(RT_EINVAL,
                            "tensor %u: centralization without row_mean (the update takes the row means itself only "
                            "for whole 16-byte-aligned device tensors of 16-bit arrays with Philox noise, rows a "
                            "multiple of 8 and %u .. %u elements long, no debug outputs)",
                            i, kRowwiseMinLen, kWaveRowMax);
        }
    }
    return RT_OK;
}

// ---------------------------------------------------------------------------
// table building and launch
// ---------------------------------------------------------------------------

// Lays out [DevScalars sets][DevTensor records][first units][their DevTensor records][PieceRef pieces][ChunkRef list]
// in h->image.  Tensors are grouped by dtype combination so that each combination
// is one contiguous range of every list = at most two launches.
// Whole fast units of plain tensors (16-byte aligned, no debug output, no centralization) become
// ranges; what such a tensor leaves over becomes pieces where the layout has a piece path (all
// arrays 16 bit, Philox noise), chunks of the generic kernel otherwise; every other tensor goes to
// the generic kernel chunk by chunk.
static void build_image(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                        bool want_explicit, Plan& plan) {
    // (scalars_idx, step) -> set index
    std::map<std::pair<uint32_t, uint32_t>, uint32_t> set_of;
    std::vector<DevScalars> sets;
    std::vector<uint32_t> order;
    order.reserve(n);
    for (uint32_t i = 0; i < n; ++i)
        if (descs[i].numel != 0) order.push_back(i);
    const auto by_combo = [&](uint32_t a, uint32_t b) { return combo_of(descs[a]) < combo_of(descs[b]); };
    if (!std::is_sorted(order.begin(), order.end(), by_combo))  // one combination is the common case
        std::stable_sort(order.begin(), order.end(), by_combo);

    std::vector<DevTensor>& tens = h->tens;
    tens.resize(order.size());
    auto it = set_of.end();
    for (size_t k = 0; k < order.size(); ++k) {
        const rt_tensor_desc& d = descs[order[k]];
        auto key = std::make_pair(d.scalars_idx, d.step);
        if (it == set_of.end() || it->first != key) it = set_of.find(key);  // neighbours mostly share a set
        if (it == set_of.end()) {
            DevScalars ds;
            memset(&ds, 0, sizeof(ds));
            ds.s = scalars[d.scalars_idx];
            ds.step = d.step;
            it = set_of.emplace(key, (uint32_t)sets.size()).first;
            sets.push_back(ds);
        }
        DevTensor& t = tens[k];
        memset(&t, 0, sizeof(t));
        t.p = (uint64_t)d.p; t.g = (uint64_t)d.g; t.m = (uint64_t)d.m; t.v = (uint64_t)d.v;
        if (want_explicit) {
            t.np = (uint64_t)d.noise_p; t.nm = (uint64_t)d.noise_m; t.nv = (uint64_t)d.noise_v;
        }
        t.dp = (uint64_t)d.dbg_p; t.dm = (uint64_t)d.dbg_m; t.dv = (uint64_t)d.dbg_v;
        t.row_mean = sets[it->second].s.centralization != 0.0f ? (uint64_t)d.row_mean : 0;
        t.numel = d.numel;
        t.block_base = d.elem_offset >> 3;
        t.row_len = d.row_len ? d.row_len : 1;
        t.tensor_id4 = d.tensor_id * 4u;
        t.set_idx = it->second;
        t.dtypes = dtypes_of(d);
        const uint64_t all = t.p | t.g | t.m | t.v | t.np | t.nm | t.nv;
        t.flags = (all & 15u) == 0 ? kFlagAligned : 0u;
        if (sets[it->second].s.centralization != 0.0f && !d.row_mean) t.flags |= kFlagRowwise;   // validated: rowwise_ok
    }

    // ---- work lists, combination by combination
    std::vector<uint32_t>& ranges = h->ranges;
    std::vector<DevTensor>& fast_tens = h->fast_tens;
    std::vector<PieceRef>& pieces = h->pieces;
    std::vector<ChunkRef>& chunks = h->chunks;
    ranges.clear();
    fast_tens.clear();
    pieces.clear();
    chunks.clear();
    plan.batches.clear();
    constexpr uint64_t unit = kFastUnitElems;
    size_t k0 = 0;
    while (k0 < order.size()) {
        const uint32_t combo = combo_of(descs[order[k0]]);
        size_t k1 = k0;
        while (k1 < order.size() && combo_of(descs[order[k1]]) == combo) ++k1;
        Batch b{};
        b.combo = combo;
        b.first_range = (uint32_t)ranges.size();
        b.first_piece = (uint32_t)pieces.size();
        const bool has_pieces = !want_explicit && narrow_combo(combo);
        auto plain = [&](const DevTensor& t) {
            return combo != kComboAny && (t.flags & kFlagAligned) && !(t.flags & kFlagRowwise) &&
                   (t.dp | t.dm | t.dv | t.row_mean) == 0;
        };
        uint32_t units = 0;
        for (size_t k = k0; k < k1; ++k) {
            const DevTensor& t = tens[k];
            if (!plain(t)) continue;
            const uint32_t nu = (uint32_t)(t.numel / unit);
            if (nu) {
                ranges.push_back(units);
                fast_tens.push_back(t);
                units += nu;
            }
            if (has_pieces) {
                for (uint64_t e = (uint64_t)nu * unit; e < t.numel; e += kPieceElems) {
                    PieceRef r;
                    memset(&r, 0, sizeof(r));
                    const int ep = dtype_size(t.dtypes & 3u), eg = dtype_size((t.dtypes >> 2) & 3u),
                              em = dtype_size((t.dtypes >> 4) & 3u), ev = dtype_size((t.dtypes >> 6) & 3u);
                    r.p = t.p + e * ep; r.g = t.g + e * eg; r.m = t.m + e * em; r.v = t.v + e * ev;
                    r.block = t.block_base + (e >> 3);
                    r.count = (uint32_t)std::min<uint64_t>(kPieceElems, t.numel - e);
                    r.tensor_id4 = t.tensor_id4;
                    r.set_idx = t.set_idx;
                    pieces.push_back(r);
                }
            }
        }
        b.n_ranges = (uint32_t)ranges.size() - b.first_range;
        b.n_units = units;
        b.n_pieces = (uint32_t)pieces.size() - b.first_piece;
        // Tensors with centralization that are otherwise plain: their whole units go to the fast
        // kernel's centralizing variant (16-bit layouts with Philox noise have one), the rest of them
        // to the generic kernel.  A lane's 8 elements must lie in at most two rows.
        auto cen_plain = [&](const DevTensor& t) {
            return has_pieces && (t.flags & kFlagAligned) && (t.dp | t.dm | t.dv) == 0 && t.row_mean != 0 &&
                   t.row_len >= (uint64_t)kVec && t.row_len < (1ull << 31);
        };
        b.first_cen_range = (uint32_t)ranges.size();
        uint32_t cen_units = 0;
        for (size_t k = k0; k < k1; ++k) {
            const DevTensor& t = tens[k];
            if (!cen_plain(t) || t.numel < unit) continue;
            ranges.push_back(cen_units);
            fast_tens.push_back(t);
            cen_units += (uint32_t)(t.numel / unit);
        }
        b.n_cen_ranges = (uint32_t)ranges.size() - b.first_cen_range;
        b.n_cen_units = cen_units;
        // Tensors whose row means the update takes itself: whole tensors, a wavefront per row.
        for (int kind = 0; kind < 2; ++kind) {
            b.first_rw_range[kind] = (uint32_t)ranges.size();
            uint64_t rw_rows = 0;
            for (size_t k = k0; k < k1; ++k) {
                const DevTensor& t = tens[k];
                if (!(t.flags & kFlagRowwise) || (int)(t.row_len <= kRowwiseShortMax) != kind) continue;
                ranges.push_back((uint32_t)rw_rows);
                fast_tens.push_back(t);
                rw_rows += t.numel / t.row_len;
            }
            b.n_rw_ranges[kind] = (uint32_t)ranges.size() - b.first_rw_range[kind];
            b.n_rw_rows[kind] = (uint32_t)std::min<uint64_t>(rw_rows, 0xFFFFFFFFull);   // checked against the grid limit at launch
        }
        b.first_generic = (uint32_t)chunks.size();
        for (size_t k = k0; k < k1; ++k) {
            const DevTensor& t = tens[k];
            const uint32_t nc = (uint32_t)((t.numel + kChunkElems - 1) / kChunkElems);
            uint32_t j0 = 0;
            if (plain(t)) j0 = has_pieces ? nc : (uint32_t)((t.numel / unit) * unit / kChunkElems);
            if (cen_plain(t)) j0 = (uint32_t)((t.numel / unit) * unit / kChunkElems);
            if (t.flags & kFlagRowwise) j0 = nc;
            for (uint32_t j = j0; j < nc; ++j) chunks.push_back(ChunkRef{(uint32_t)k, j});
        }
        b.n_generic = (uint32_t)chunks.size() - b.first_generic;
        plan.batches.push_back(b);
        k0 = k1;
    }

    plan.set_keys.assign(sets.size(), {0u, 0u});
    for (const auto& kv : set_of) plan.set_keys[kv.second] = kv.first;
    plan.n_sets = (uint32_t)sets.size();
    plan.n_tensors = (uint32_t)tens.size();
    plan.n_chunks = (uint32_t)chunks.size();
    if (!sets.empty()) plan.first_set = sets[0];
    plan.off_sets = 0;
    plan.off_tensors = align_up(sets.size() * sizeof(DevScalars), 256);
    plan.off_ranges = plan.off_tensors + align_up(tens.size() * sizeof(DevTensor), 128);
    plan.off_fast_tensors = plan.off_ranges + align_up(ranges.size() * sizeof(uint32_t), 128);
    plan.off_pieces = plan.off_fast_tensors + align_up(fast_tens.size() * sizeof(DevTensor), 128);
    plan.off_chunks = plan.off_pieces + align_up(pieces.size() * sizeof(PieceRef), 128);
    plan.bytes = plan.off_chunks + align_up(chunks.size() * sizeof(ChunkRef), 128);
    h->image.assign(plan.bytes, 0);
    uint8_t* img = h->image.data();
    if (!sets.empty()) memcpy(img + plan.off_sets, sets.data(), sets.size() * sizeof(DevScalars));
    if (!tens.empty()) memcpy(img + plan.off_tensors, tens.data(), tens.size() * sizeof(DevTensor));
    if (!ranges.empty()) memcpy(img + plan.off_ranges, ranges.data(), ranges.size() * sizeof(uint32_t));
    if (!fast_tens.empty())
        memcpy(img + plan.off_fast_tensors, fast_tens.data(), fast_tens.size() * sizeof(DevTensor));
    if (!pieces.empty()) memcpy(img + plan.off_pieces, pieces.data(), pieces.size() * sizeof(PieceRef));
    if (!chunks.empty()) memcpy(img + plan.off_chunks, chunks.data(), chunks.size() * sizeof(ChunkRef));
}

// Puts a table image into a free table slot (skipping what the slot's device memory already
// holds) and returns the slot.  `static_gen` != 0 names the layout the lists behind the scalars
// belong to: a slot that holds the same generation is not even compared.
static int stage_image(rt_handle* h, const Plan& plan, const uint8_t* img, uint64_t static_gen, hipStream_t stream,
                       TableSlot** out) {
    TableSlot& s = h->slots[h->slot_counter++ % kSlots];
    if (s.in_flight) {
        HIP_TRY(hipEventSynchronize(s.done));
        s.in_flight = false;
    }
    if (plan.bytes > s.host_cap) {
        if (s.host) HIP_TRY(hipHostFree(s.host));
        s.host = nullptr;
        s.host_cap = 0;
        s.valid_bytes = 0;
        const size_t want = plan.bytes + plan.bytes / 4 + 4096;
        hipError_t e = hipHostMalloc(&s.host, want, hipHostMallocDefault);
        if (e != hipSuccess) return fail(RT_ENOMEM, "hipHostMalloc(%zu) failed: %s", want, hipGetErrorString(e));
        s.host_cap = want;
    }
    if (plan.bytes > s.dev.cap) {
        s.valid_bytes = 0;
        int rc = dev_reserve(s.dev, plan.bytes);
        if (rc != RT_OK) return rc;
    }
    // Two regions: the DevScalars sets change with every step, the lists behind them only when the
    // tensors do; each region is copied only if the device copy differs.
    const size_t split = std::min(plan.off_tensors, plan.bytes);
    const bool known = s.valid_bytes == plan.bytes;
    if (split > 0 && !(known && memcmp(s.host, img, split) == 0)) {
        memcpy(s.host, img, split);
        HIP_TRY(hipMemcpyAsync(s.dev.ptr, s.host, split, hipMemcpyHostToDevice, stream));
    }
    const bool same_gen = known && static_gen != 0 && s.static_gen == static_gen;
    if (plan.bytes > split && !same_gen &&
        !(known && memcmp((uint8_t*)s.host + split, img + split, plan.bytes - split) == 0)) {
        memcpy((uint8_t*)s.host + split, img + split, plan.bytes - split);
        HIP_TRY(hipMemcpyAsync((uint8_t*)s.dev.ptr + split, (uint8_t*)s.host + split, plan.bytes - split,
                               hipMemcpyHostToDevice, stream));
    }
    s.valid_bytes = plan.bytes;
    s.static_gen = static_gen;
    *out = &s;
    return RT_OK;
}

// Enqueues the update kernels of one table image that already sits in device memory at `base`.
// `t_begin` / `t_end` (timed launches): events attached to the dispatches themselves -- the first
// kernel's start and the last kernel's end -- so that what is read back is kernel time, without the
// few microseconds a marker before and after a dispatch adds.
static int enqueue_kernels(const Plan& plan, const uint8_t* base, uint64_t seed, int noise_mode,
                           const float* d_clip_coef, const uint32_t* d_skip, hipStream_t stream,
                           hipEvent_t t_begin = nullptr, hipEvent_t t_end = nullptr) {
    LaunchArgs a;
    memset(&a, 0, sizeof(a));
    a.tensors = (const DevTensor*)(base + plan.off_tensors);
    a.sets = (const DevScalars*)(base + plan.off_sets);
    a.clip_coef = d_clip_coef;
    a.skip = d_skip;
    a.seed_lo = (uint32_t)seed;
    a.seed_hi = (uint32_t)(seed >> 32);
    a.use_ks = plan.n_sets == 1 ? 1u : 0u;
    a.ks = plan.first_set;
    struct Launch {
        MultiKernel kernel;
        uint32_t grid;
        LaunchArgs args;
    };
    std::vector<Launch> launches;
    for (const Batch& b : plan.batches) {
        KernelPair k{};
        if (b.combo == kComboAny) {
            k.fast = nullptr;  // no ranges and no pieces for this group
            k.generic = noise_mode == RT_NOISE_EXPLICIT ? sr_adamw_any_kernel<RT_NOISE_EXPLICIT>
                                                        : sr_adamw_any_kernel<RT_NOISE_PHILOX>;
        } else {
            k = pick_kernel(b.combo & 3, (b.combo >> 2) & 3, (b.combo >> 4) & 3, (b.combo >> 6) & 3, noise_mode);
        }
        a.first = (const uint32_t*)(base + plan.off_ranges) + b.first_range;
        a.fast_tensors = (const DevTensor*)(base + plan.off_fast_tensors) + b.first_range;
        a.n_ranges = b.n_ranges;
        a.pieces = (const PieceRef*)(base + plan.off_pieces) + b.first_piece;
        a.n_pieces = b.n_pieces;
        a.n_piece_wgs = (b.n_pieces + 3u) / 4u;
        a.chunks = (const ChunkRef*)(base + plan.off_chunks) + b.first_generic;
        const uint64_t grid = (uint64_t)a.n_piece_wgs + b.n_units;
        a.piece_rate = 0;  // only pieces, or none
        if (a.n_piece_wgs != 0 && b.n_units != 0)
            a.piece_rate = (uint32_t)((((uint64_t)a.n_piece_wgs << 32) + grid - 1) / grid);  // < 2^32: n_piece_wgs < grid
        if (grid > kMaxGrid || b.n_generic > kMaxGrid) return fail(RT_EUNSUPPORTED, "too many workgroups in one launch");
        if (grid) launches.push_back(Launch{k.fast, (uint32_t)grid, a});
        if (b.n_generic) launches.push_back(Launch{k.generic, b.n_generic, a});
        if (b.n_cen_units) {
            if (!k.fast_cen) return fail(RT_EHIP, "internal: centralized units without a kernel for them");
            LaunchArgs c = a;
            c.first = (const uint32_t*)(base + plan.off_ranges) + b.first_cen_range;
            c.fast_tensors = (const DevTensor*)(base + plan.off_fast_tensors) + b.first_cen_range;
            c.n_ranges = b.n_cen_ranges;
            c.n_pieces = c.n_piece_wgs = c.piece_rate = 0;
            launches.push_back(Launch{k.fast_cen, b.n_cen_units, c});
        }
        for (int kind = 0; kind < 2; ++kind) {
            if (!b.n_rw_rows[kind]) continue;
            const MultiKernel kern = kind ? k.rowwise_short : k.rowwise;
            if (!kern) return fail(RT_EHIP, "internal: row-wise tensors without a kernel for them");
            const uint64_t rw_grid = ((uint64_t)b.n_rw_rows[kind] + kThreads / 64 - 1) / (kThreads / 64);
            if (b.n_rw_rows[kind] == 0xFFFFFFFFu || rw_grid > kMaxGrid)
                return fail(RT_EUNSUPPORTED, "too many rows in one launch");
            LaunchArgs c = a;
            c.first = (const uint32_t*)(base + plan.off_ranges) + b.first_rw_range[kind];
            c.fast_tensors = (const DevTensor*)(base + plan.off_fast_tensors) + b.first_rw_range[kind];
            c.n_ranges = b.n_rw_ranges[kind];
            c.n_rows = b.n_rw_rows[kind];
            c.n_pieces = c.n_piece_wgs = c.piece_rate = 0;
            launches.push_back(Launch{kern, (uint32_t)rw_grid, c});
        }
    }
    for (size_t i = 0; i < launches.size(); ++i) {
        const Launch& l = launches[i];
        const hipEvent_t e0 = i == 0 ? t_begin : nullptr;
        const hipEvent_t e1 = i + 1 == launches.size() ? t_end : nullptr;
        if (e0 || e1)
            hipExtLaunchKernelGGL(l.kernel, dim3(l.grid), dim3(kThreads), 0, stream, e0, e1, 0, l.args);
        else
            hipLaunchKernelGGL(l.kernel, dim3(l.grid), dim3(kThreads), 0, stream, l.args);
        HIP_TRY(hipGetLastError());
    }
    return RT_OK;
}

// Whether `descs` describe the tensors of the cached layout: everything but the step counts equal,
// and every step count ahead of the cached one by the same amount (*delta).
static bool same_layout(const rt_handle::LayoutCache& lc, const rt_tensor_desc* descs, uint32_t n, int noise_mode,
                        const rt_scalars* scalars, uint32_t n_scalars, uint32_t* delta) {
    if (!lc.valid || lc.noise_mode != noise_mode || lc.descs.size() != n || n == 0) return false;
    static_assert(offsetof(rt_tensor_desc, step) == 116 && sizeof(rt_tensor_desc) == 136, "rt_tensor_desc layout");
    const uint32_t d0 = descs[0].step - lc.descs[0].step;
    for (uint32_t i = 0; i < n; ++i) {
        const uint8_t* a = (const uint8_t*)&descs[i];
        const uint8_t* b = (const uint8_t*)&lc.descs[i];
        if (memcmp(a, b, 116) != 0 || memcmp(a + 120, b + 120, 16) != 0) return false;
        if (descs[i].step - lc.descs[i].step != d0) return false;
    }
    for (size_t j = 0; j < lc.plan.set_keys.size(); ++j) {
        const uint32_t si = lc.plan.set_keys[j].first;
        if (si >= n_scalars || (scalars[si].centralization != 0.0f) != (lc.cen[j] != 0)) return false;
    }
    *delta = d0;
    return true;
}

static int launch_update(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                         uint32_t n_scalars, uint64_t seed, int noise_mode, const float* d_clip_coef,
                         const uint32_t* d_skip, hipStream_t stream) {
    rt_handle::LayoutCache& lc = h->layout;
    uint32_t delta = 0;
    if (same_layout(lc, descs, n, noise_mode, scalars, n_scalars, &delta)) {
        // only the per-step scalars are new: the arguments were validated when the layout was built
        DevScalars* sets = (DevScalars*)(lc.image.data() + lc.plan.off_sets);
        for (size_t j = 0; j < lc.plan.set_keys.size(); ++j) {
            auto& key = lc.plan.set_keys[j];
            key.second += delta;
            memset(&sets[j], 0, sizeof(DevScalars));
            sets[j].s = scalars[key.first];
            sets[j].step = key.second;
        }
        if (!lc.plan.set_keys.empty()) lc.plan.first_set = sets[0];
        if (delta != 0)
            for (uint32_t i = 0; i < n; ++i) lc.descs[i].step = descs[i].step;
    } else {
        lc.valid = false;
        int rc = validate(descs, n, scalars, n_scalars, noise_mode, /*allow_host=*/false);
        if (rc != RT_OK) return rc;
        build_image(h, descs, n, scalars, noise_mode == RT_NOISE_EXPLICIT, lc.plan);
        lc.image = h->image;
        lc.descs.assign(descs, descs + n);
        lc.cen.resize(lc.plan.set_keys.size());
        for (size_t j = 0; j < lc.plan.set_keys.size(); ++j)
            lc.cen[j] = scalars[lc.plan.set_keys[j].first].centralization != 0.0f;
        lc.noise_mode = noise_mode;
        lc.gen = ++h->layout_gen;
        lc.valid = true;
    }
    const Plan& plan = lc.plan;
    if (plan.n_tensors == 0) return RT_OK;
    TableSlot* slot = nullptr;
    int rc = stage_image(h, plan, lc.image.data(), lc.gen, stream, &slot);
    if (rc != RT_OK) return rc;
    std::pair<hipEvent_t, hipEvent_t>* tp = h->timing ? &h->tring[h->timed_launches % kTimingRing] : nullptr;
    rc = enqueue_kernels(plan, (const uint8_t*)slot->dev.ptr, seed, noise_mode, d_clip_coef, d_skip, stream,
                         tp ? tp->first : nullptr, tp ? tp->second : nullptr);
    if (rc != RT_OK) return rc;
    if (tp) ++h->timed_launches;
    HIP_TRY(hipEventRecord(slot->done, stream));
    slot->in_flight = true;
    return RT_OK;
}

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
extern "C" {

int rt_version(void) { return RT_ABI_VERSION; }

const char* rt_last_error(void) { return g_err; }

int rt_destroy(rt_handle* h);

int rt_create(int device, rt_handle** out) {
    if (!out) return fail(RT_EINVAL, "out is NULL");
    *out = nullptr;
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(RT_EINVAL, "device %d out of range (have %d)", device, count);
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(RT_EUNSUPPORTED, "device %d is %s; this library is built for gfx950 only", device,
                    prop.gcnArchName);
    if (device >= kMaxDevices) return fail(RT_EUNSUPPORTED, "device %d: at most %d devices", device, kMaxDevices);
    void* scratch_ptr = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[device]) {
            void* ptr = nullptr;
            HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));  // with `device` current: its own copy
            HIP_TRY(hipEventCreateWithFlags(&g_scratch_done[device], hipEventDisableTiming));
            g_scratch_ptr[device] = ptr;
        }
        scratch_ptr = g_scratch_ptr[device];
    }
    rt_handle* h = new (std::nothrow) rt_handle();
    if (!h) return fail(RT_ENOMEM, "out of host memory");
    h->device = device;
    h->static_scratch = scratch_ptr;
    h->norm_entries.reserve(kStaticMaxTensors);
    hipError_t e = hipSuccess;
    for (int i = 0; i < kSlots && e == hipSuccess; ++i)
        e = hipEventCreateWithFlags(&h->slots[i].done, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreate(&h->t0);
    if (e == hipSuccess) e = hipEventCreate(&h->t1);
    if (e != hipSuccess) {
        rt_destroy(h);
        return fail(RT_EHIP, "creating events failed: %s (%d)", hipGetErrorString(e), (int)e);
    }
    *out = h;
    return RT_OK;
}

int rt_destroy(rt_handle* h) {
    if (!h) return RT_OK;
    (void)hipSetDevice(h->device);
    (void)hipDeviceSynchronize();
    for (int i = 0; i < kSlots; ++i) {
        if (h->slots[i].dev.ptr) (void)hipFree(h->slots[i].dev.ptr);
        if (h->slots[i].host) (void)hipHostFree(h->slots[i].host);
        if (h->slots[i].done) (void)hipEventDestroy(h->slots[i].done);
    }
    if (h->norm_partials.ptr) (void)hipFree(h->norm_partials.ptr);
    if (h->t0) (void)hipEventDestroy(h->t0);
    if (h->t1) (void)hipEventDestroy(h->t1);
    for (auto& pr : h->tring) {
        if (pr.first) (void)hipEventDestroy(pr.first);
        if (pr.second) (void)hipEventDestroy(pr.second);
    }
    Streamed& st = h->st;
    for (int a = 0; a < 4; ++a)
        for (int b = 0; b < kStageBufs; ++b)
            if (st.stage[a][b].ptr) (void)hipFree(st.stage[a][b].ptr);
    for (int b = 0; b < kStageBufs; ++b) {
        if (st.h2d_done[b]) (void)hipEventDestroy(st.h2d_done[b]);
        if (st.comp_done[b]) (void)hipEventDestroy(st.comp_done[b]);
        if (st.d2h_done[b]) (void)hipEventDestroy(st.d2h_done[b]);
    }
    for (auto& r : st.ring) {
        if (r.dev.ptr) (void)hipFree(r.dev.ptr);
        if (r.host) (void)hipHostFree(r.host);
    }
    st.pool.reset();  // joins the copy threads
    for (int a = 0; a < 4; ++a)
        for (int k = 0; k < kBounce; ++k) {
            if (st.bounce[a][k]) (void)hipHostFree(st.bounce[a][k]);
            if (st.bounce_down[a][k]) (void)hipHostFree(st.bounce_down[a][k]);
        }
    if (st.ticket_word) (void)hipHostFree((void*)st.ticket_word);
    for (hipEvent_t e : st.tl_events) (void)hipEventDestroy(e);
    if (st.start) (void)hipEventDestroy(st.start);
    if (st.h2d) (void)hipStreamDestroy(st.h2d);
    if (st.comp) (void)hipStreamDestroy(st.comp);
    if (st.d2h) (void)hipStreamDestroy(st.d2h);
    delete h;
    return RT_OK;
}

int rt_set_timing(rt_handle* h, int enabled) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    if (enabled && h->tring.size() < kTimingRing) {
        HIP_TRY(hipSetDevice(h->device));
        h->tring.reserve(kTimingRing);
        while (h->tring.size() < kTimingRing) {
            std::pair<hipEvent_t, hipEvent_t> pr{nullptr, nullptr};
            HIP_TRY(hipEventCreate(&pr.first));
            hipError_t e = hipEventCreate(&pr.second);
            if (e != hipSuccess) {
                (void)hipEventDestroy(pr.first);
                return fail(RT_EHIP, "hipEventCreate failed: %s (%d)", hipGetErrorString(e), (int)e);
            }
            h->tring.push_back(pr);
        }
    }
    h->timing = enabled != 0;
    if (enabled) h->timed_launches = 0;
    return RT_OK;
}

int rt_last_kernel_ms(rt_handle* h, float* ms) {
    if (!h || !ms) return fail(RT_EINVAL, "NULL argument");
    if (h->timed_launches == 0) return fail(RT_EINVAL, "no timed launch on this handle (rt_set_timing first)");
    const auto& pr = h->tring[(h->timed_launches - 1) % kTimingRing];
    HIP_TRY(hipEventSynchronize(pr.second));
    HIP_TRY(hipEventElapsedTime(ms, pr.first, pr.second));
    return RT_OK;
}

int rt_kernel_ms_history(rt_handle* h, float* out_ms, uint32_t cap, uint32_t* n_out) {
    if (!h || !n_out || (cap > 0 && !out_ms)) return fail(RT_EINVAL, "NULL argument");
    const uint64_t have = std::min<uint64_t>(h->timed_launches, kTimingRing);
    const uint64_t n = std::min<uint64_t>(have, cap);
    for (uint64_t k = 0; k < n; ++k) {  // oldest of the n most recent launches first
        const auto& pr = h->tring[(h->timed_launches - n + k) % kTimingRing];
        HIP_TRY(hipEventSynchronize(pr.second));
        HIP_TRY(hipEventElapsedTime(&out_ms[k], pr.first, pr.second));
    }
    *n_out = (uint32_t)n;
    return RT_OK;
}

int rt_step_multi(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                  uint32_t n_scalars, uint64_t seed, int noise_mode, const float* d_clip_coef,
                  const uint32_t* d_skip, void* stream) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    if (n == 0) return validate(descs, n, scalars, n_scalars, noise_mode, /*allow_host=*/false);
    if (!descs || !scalars || n_scalars == 0 || (noise_mode != RT_NOISE_PHILOX && noise_mode != RT_NOISE_EXPLICIT))
        return validate(descs, n, scalars, n_scalars, noise_mode, /*allow_host=*/false);  // names the bad argument
    HIP_TRY(hipSetDevice(h->device));
    return launch_update(h, descs, n, scalars, n_scalars, seed, noise_mode, d_clip_coef, d_skip, (hipStream_t)stream);
}

// The gradient table of the norm pass: one NormEntry per non-empty gradient.  Chunks of 8192
// elements are numbered in two sequences -- every whole chunk of the 16-byte aligned gradients
// first, then all other chunks, each in tensor order -- and chunk c belongs to workgroup c mod grid.
static int build_norm_table(const rt_tensor_desc* descs, uint32_t n, size_t max_entries, std::vector<NormEntry>& tab,
                            uint64_t& n_whole, uint64_t& n_rest) {
    tab.clear();
    n_whole = n_rest = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const rt_tensor_desc& d = descs[i];
        if (d.g_dtype > RT_DT_F16) return fail(RT_EINVAL, "tensor %u: g_dtype %d unknown", i, d.g_dtype);
        if (d.host_mask) return fail(RT_EINVAL, "tensor %u: host_mask set (grads must be device resident)", i);
        if (d.numel == 0) continue;
        if (!d.g) return fail(RT_EINVAL, "tensor %u: g is NULL", i);
        if ((uintptr_t)d.g % dtype_size(d.g_dtype))
            return fail(RT_EINVAL, "tensor %u: g not aligned to its element size", i);
        if (d.numel / kChunkElems >= 0xFFFFFFFFull) return fail(RT_EUNSUPPORTED, "tensor %u: numel too large", i);
        if (tab.size() >= max_entries)
            return fail(RT_EUNSUPPORTED,
                        "rt_grad_norm_static takes at most %zu non-empty gradients per call (its table is a fixed "
                        "device array); use rt_grad_norm", max_entries);
        const uint64_t chunks = (d.numel + kChunkElems - 1) / kChunkElems;
        const uint64_t whole = ((uintptr_t)d.g & 15u) == 0 ? d.numel / kChunkElems : 0;
        NormEntry e;
        e.g = (uint64_t)d.g;
        e.numel = d.numel;
        e.first_whole = (uint32_t)n_whole;
        e.first_rest = (uint32_t)n_rest;
        e.n_whole = (uint32_t)whole;
        e.dtype = d.g_dtype;
        tab.push_back(e);
        n_whole += whole;
        n_rest += chunks - whole;
        if (n_whole + n_rest > kMaxGrid) return fail(RT_EUNSUPPORTED, "too many elements in one call");
    }
    return RT_OK;
}

int rt_grad_norm(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, float inv_loss_scale, float max_norm,
                 void* d_out, void* stream_) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    if (!d_out || ((uintptr_t)d_out & 15u)) return fail(RT_EINVAL, "d_out must be a 16-byte aligned device pointer");
    if (n > 0 && !descs) return fail(RT_EINVAL, "descs is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    HIP_TRY(hipSetDevice(h->device));
    std::vector<NormEntry>& tab = h->norm_table;
    uint64_t n_whole = 0, n_rest = 0;
    int rc = build_norm_table(descs, n, SIZE_MAX, tab, n_whole, n_rest);
    if (rc != RT_OK) return rc;
    rc = dev_reserve(h->norm_partials, kNormPartials * sizeof(double));
    if (rc != RT_OK) return rc;
    // With nothing to sum the finish kernel reads no partials (a total of zero).  (2048 - 4096
    // workgroups read at 6.6 - 7.0 TB/s; more workgroups were slower.)
    const uint32_t n_chunks = (uint32_t)(n_whole + n_rest);
    const uint32_t grid = std::min<uint32_t>(kNormPartials, n_chunks);
    if (n_chunks != 0) {
        // the table goes through a staging slot: the same gradients step after step upload nothing
        Plan plan;
        plan.bytes = tab.size() * sizeof(NormEntry);
        h->image.assign((const uint8_t*)tab.data(), (const uint8_t*)tab.data() + plan.bytes);
        TableSlot* slot = nullptr;
        rc = stage_image(h, plan, h->image.data(), 0, stream, &slot);
        if (rc != RT_OK) return rc;
        hipLaunchKernelGGL(grad_sumsq_table_kernel, dim3(grid), dim3(kThreads), 0, stream,
                           (const NormEntry*)slot->dev.ptr, (uint32_t)tab.size(), (uint32_t)n_whole, n_chunks,
                           inv_loss_scale, (double*)h->norm_partials.ptr);
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipEventRecord(slot->done, stream));
        slot->in_flight = true;
    }
    hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(kThreads), 0, stream,
                       (const double*)h->norm_partials.ptr, grid, max_norm, (float*)d_out);
    HIP_TRY(hipGetLastError());
    return RT_OK;
}

int rt_grad_norm_static(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, float inv_loss_scale, float max_norm,
                        void* d_out, void* stream_) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    if (!d_out || ((uintptr_t)d_out & 15u)) return fail(RT_EINVAL, "d_out must be a 16-byte aligned device pointer");
    if (n > 0 && !descs) return fail(RT_EINVAL, "descs is NULL");
    if (!h->static_scratch) return fail(RT_EHIP, "the static scratch array has no address on device %d", h->device);
    hipStream_t stream = (hipStream_t)stream_;
    HIP_TRY(hipSetDevice(h->device));
    std::vector<NormEntry>& tab = h->norm_entries;  // capacity reserved by rt_create
    uint64_t n_whole = 0, n_rest = 0;
    const int rc = build_norm_table(descs, n, kStaticMaxTensors, tab, n_whole, n_rest);
    if (rc != RT_OK) return rc;
    double* partials = (double*)h->static_scratch;
    NormEntry* table = (NormEntry*)((uint8_t*)h->static_scratch + kStaticPartialsBytes);
    // take turns with whatever call used the array last (nothing is allocated: the event exists since rt_create)
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusNone;
    }
    std::unique_lock<std::mutex> turn(g_scratch_mutex, std::defer_lock);
    if (capturing == hipStreamCaptureStatusNone) {
        turn.lock();   // wait-then-record is one step as seen by other host threads
        HIP_TRY(hipStreamWaitEvent(stream, g_scratch_done[h->device], 0));
    }
    const uint32_t n_chunks = (uint32_t)(n_whole + n_rest);
    const uint32_t grid = std::min<uint32_t>(kNormPartials, n_chunks);
    // the table reaches the device array as kernel arguments, a slice per launch
    for (uint32_t first = 0; first < tab.size(); first += kNormEntriesPerWrite) {
        NormEntrySlice slice;
        const uint32_t count = std::min<uint32_t>(kNormEntriesPerWrite, (uint32_t)tab.size() - first);
        memcpy(slice.e, tab.data() + first, count * sizeof(NormEntry));
        hipLaunchKernelGGL(norm_table_write_kernel, dim3(1), dim3(kNormEntriesPerWrite), 0, stream, table, first,
                           count, slice);
        HIP_TRY(hipGetLastError());
    }
    if (n_chunks != 0) {
        hipLaunchKernelGGL(grad_sumsq_table_kernel, dim3(grid), dim3(kThreads), 0, stream, (const NormEntry*)table,
                           (uint32_t)tab.size(), (uint32_t)n_whole, n_chunks, inv_loss_scale, partials);
        HIP_TRY(hipGetLastError());
    }
    hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(kThreads), 0, stream, (const double*)partials, grid,
                       max_norm, (float*)d_out);
    HIP_TRY(hipGetLastError());
    if (capturing == hipStreamCaptureStatusNone) HIP_TRY(hipEventRecord(g_scratch_done[h->device], stream));
    return RT_OK;
}

int rt_row_means(rt_handle* h, const void* g, int g_dtype, uint64_t rows, uint64_t row_len, float inv_loss_scale,
                 float* d_row_mean, void* stream_) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    if (rows == 0) return RT_OK;
    if (!g || !d_row_mean || row_len == 0) return fail(RT_EINVAL, "NULL pointer or empty row");
    if (rows > 0x7FFFFFFFull) return fail(RT_EUNSUPPORTED, "too many rows");
    if (g_dtype < 0 || g_dtype > RT_DT_F16) return fail(RT_EINVAL, "g_dtype %d unknown", g_dtype);
    if ((uintptr_t)g % dtype_size(g_dtype)) return fail(RT_EINVAL, "gradient pointer not aligned to its element size");
    hipStream_t stream = (hipStream_t)stream_;
    HIP_TRY(hipSetDevice(h->device));
    if (row_len <= kWaveRowMax) {
        const uint32_t grid = (uint32_t)((rows + kThreads / 64 - 1) / (kThreads / 64));
        hipLaunchKernelGGL(row_mean_kernel, dim3(grid), dim3(kThreads), 0, stream, (uint64_t)g, (uint32_t)g_dtype, rows,
                           (uint32_t)row_len, inv_loss_scale, d_row_mean);
    } else {
        hipLaunchKernelGGL(row_mean_long_kernel, dim3((uint32_t)rows), dim3(kThreads), 0, stream, (uint64_t)g,
                           (uint32_t)g_dtype, row_len, inv_loss_scale, d_row_mean);
    }
    HIP_TRY(hipGetLastError());
    return RT_OK;
}

int rt_row_means_multi(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, float inv_loss_scale, void* stream_) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    if (n > 0 && !descs) return fail(RT_EINVAL, "descs is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    HIP_TRY(hipSetDevice(h->device));
    // Two tables, one per kernel: gradients whose rows one wavefront sums, and gradients with longer rows.
    std::vector<RowMeanEntry>& tab = h->rowmean_table;
    tab.clear();
    std::vector<RowMeanEntry> long_tab;
    uint64_t rows_short = 0, rows_long = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const rt_tensor_desc& d = descs[i];
        if (d.numel == 0 || !d.row_mean) continue;
        if (!d.g || d.row_len == 0 || d.numel % d.row_len != 0)
            return fail(RT_EINVAL, "tensor %u: NULL gradient, or numel %llu is not a multiple of row_len %llu", i,
                        (unsigned long long)d.numel, (unsigned long long)d.row_len);
        if (d.g_dtype > RT_DT_F16) return fail(RT_EINVAL, "tensor %u: g_dtype %d (need bf16, f32 or f16)", i, d.g_dtype);
        if (d.host_mask & RT_HOST_G) return fail(RT_EINVAL, "tensor %u: the gradient must be device resident", i);
        if ((uintptr_t)d.g % dtype_size(d.g_dtype)) return fail(RT_EINVAL, "tensor %u: gradient pointer not aligned", i);
        const bool is_long = d.row_len > kWaveRowMax;
        uint64_t& rows = is_long ? rows_long : rows_short;
        RowMeanEntry e;
        e.g = (uint64_t)d.g;
        e.out = (uint64_t)d.row_mean;
        e.row_len = d.row_len;
        e.first_row = (uint32_t)rows;
        e.dtype = (uint32_t)d.g_dtype;
        if (d.numel / d.row_len > kMaxGrid) return fail(RT_EUNSUPPORTED, "tensor %u: too many rows", i);
        e.rows = (uint32_t)(d.numel / d.row_len);
        e.pad[0] = e.pad[1] = e.pad[2] = 0;
        (is_long ? long_tab : tab).push_back(e);
        rows += d.numel / d.row_len;
        if (rows > kMaxGrid) return fail(RT_EUNSUPPORTED, "more than %llu rows in one call", (unsigned long long)kMaxGrid);
    }
    if (rows_short + rows_long == 0) return RT_OK;
    // image: [first rows, short][records, short][first rows, long][records, long]; through a staging slot, like
    // the tables of the update (the same gradients step after step upload nothing)
    const size_t ns = tab.size(), nl = long_tab.size();
    const size_t off_rec_s = align_up(ns * sizeof(uint32_t), 128);
    const size_t off_first_l = off_rec_s + align_up(ns * sizeof(RowMeanEntry), 128);
    const size_t off_rec_l = off_first_l + align_up(nl * sizeof(uint32_t), 128);
    Plan plan;
    plan.bytes = off_rec_l + align_up(nl * sizeof(RowMeanEntry), 128);
    h->image.assign(plan.bytes, 0);
    uint8_t* img = h->image.data();
    for (size_t k = 0; k < ns; ++k) ((uint32_t*)img)[k] = tab[k].first_row;
    if (ns) memcpy(img + off_rec_s, tab.data(), ns * sizeof(RowMeanEntry));
    for (size_t k = 0; k < nl; ++k) ((uint32_t*)(img + off_first_l))[k] = long_tab[k].first_row;
    if (nl) memcpy(img + off_rec_l, long_tab.data(), nl * sizeof(RowMeanEntry));
    TableSlot* slot = nullptr;
    int rc = stage_image(h, plan, img, 0, stream, &slot);
    if (rc != RT_OK) return rc;
    const uint8_t* dev = (const uint8_t*)slot->dev.ptr;
    if (rows_short) {
        const uint32_t grid = (uint32_t)((rows_short + kThreads / 64 - 1) / (kThreads / 64));
        hipLaunchKernelGGL(row_mean_table_kernel, dim3(grid), dim3(kThreads), 0, stream, (const uint32_t*)dev,
                           (const RowMeanEntry*)(dev + off_rec_s), (uint32_t)ns, (uint32_t)rows_short, inv_loss_scale);
        HIP_TRY(hipGetLastError());
    }
    if (rows_long) {
        hipLaunchKernelGGL(row_mean_table_long_kernel, dim3((uint32_t)rows_long), dim3(kThreads), 0, stream,
                           (const uint32_t*)(dev + off_first_l), (const RowMeanEntry*)(dev + off_rec_l), (uint32_t)nl,
                           inv_loss_scale);
        HIP_TRY(hipGetLastError());
    }
    HIP_TRY(hipEventRecord(slot->done, stream));
    slot->in_flight = true;
    return RT_OK;
}

int rt_sr_copy(void* target_bf16, const float* source, uint64_t numel, const void* noise, uint64_t seed,
               void* stream_) {
    if (numel == 0) return RT_OK;
    if (!target_bf16 || !source) return fail(RT_EINVAL, "NULL pointer");
    if (((uintptr_t)target_bf16 & 1u) || ((uintptr_t)source & 3u) || ((uintptr_t)noise & 1u))
        return fail(RT_EINVAL, "pointer not aligned to its element size");
    hipStream_t stream = (hipStream_t)stream_;
    const int aligned = ((((uintptr_t)target_bf16) | ((uintptr_t)source) | ((uintptr_t)noise)) & 15u) == 0;
    const uint64_t blocks = (numel + (uint64_t)kThreads * kVec - 1) / ((uint64_t)kThreads * kVec);
    // one block of 2048 elements per workgroup: a capped grid with a grid-stride loop ran 25 % slower
    const uint32_t grid = (uint32_t)std::min<uint64_t>(blocks, kMaxGrid);
    if (noise)
        hipLaunchKernelGGL(sr_copy_kernel<RT_NOISE_EXPLICIT>, dim3(grid), dim3(kThreads), 0, stream,
                           (uint64_t)target_bf16, (uint64_t)source, numel, (uint64_t)noise, (uint32_t)seed,
                           (uint32_t)(seed >> 32), aligned);
    else
        hipLaunchKernelGGL(sr_copy_kernel<RT_NOISE_PHILOX>, dim3(grid), dim3(kThreads), 0, stream,
                           (uint64_t)target_bf16, (uint64_t)source, numel, (uint64_t)0, (uint32_t)seed,
                           (uint32_t)(seed >> 32), aligned);
    HIP_TRY(hipGetLastError());
    return RT_OK;
}

// ---------------------------------------------------------------------------
// streamed variant
// ---------------------------------------------------------------------------
static int streamed_init(rt_handle* h) {
    Streamed& st = h->st;
    if (st.ready) return RT_OK;
    // Every step creates only what is still missing, so a call that failed halfway (out of
    // memory, say) can be repeated without leaking what the first attempt created.
    for (hipStream_t* s : {&st.h2d, &st.comp, &st.d2h})
        if (!*s) HIP_TRY(hipStreamCreateWithFlags(s, hipStreamNonBlocking));
    if (!st.start) HIP_TRY(hipEventCreateWithFlags(&st.start, hipEventDisableTiming));
    for (int b = 0; b < kStageBufs; ++b)
        for (hipEvent_t* e : {&st.h2d_done[b], &st.comp_done[b], &st.d2h_done[b]})
            if (!*e) HIP_TRY(hipEventCreateWithFlags(e, hipEventDisableTiming));
    // Table memory for the calls in flight is set aside now: allocating (device or pinned
    // host memory) while the copy pipeline runs stalls the copies for tens of milliseconds.
    if (st.ring.size() < kTablePool) st.ring.resize(kTablePool);
    for (auto& r : st.ring) {
        int rc = dev_reserve(r.dev, kTablePoolBytes);
        if (rc != RT_OK) return rc;
        if (r.host) continue;
        hipError_t e = hipHostMalloc(&r.host, kTablePoolBytes, hipHostMallocDefault);
        if (e != hipSuccess) {
            r.host = nullptr;
            return fail(RT_ENOMEM, "hipHostMalloc(%zu) failed: %s", kTablePoolBytes, hipGetErrorString(e));
        }
        r.host_cap = kTablePoolBytes;
    }
    if (!st.ticket_word) {
        void* word = nullptr;
        HIP_TRY(hipHostMalloc(&word, 64, hipHostMallocDefault));
        ((volatile uint64_t*)word)[0] = 0;
        ((volatile uint64_t*)word)[1] = 0;
        st.ticket_word = (volatile uint64_t*)word;
    }
    if (const char* e = getenv("RT_STREAM_BATCH_CHUNKS")) {
        const long v = atol(e);
        if (v > 0) st.batch_chunks = (uint64_t)v;
    }
    if (const char* e = getenv("RT_STREAM_BOUNCE_THREADS")) st.bounce_threads = (int)std::min(64l, std::max(0l, atol(e)));
    st.ready = true;
    return RT_OK;
}

namespace {
struct Segment {       // a contiguous piece of one tensor inside one chunk
    uint32_t tensor;   // index into descs
    uint64_t start;    // first element of the piece inside the tensor
    uint64_t count;
    uint64_t stage_off;  // element offset inside the staging buffers (multiple of 8)
};
}  // namespace

// Cuts the tensor list into chunks of at most chunk_elems staged elements.  A tensor may span
// chunks; every piece starts at a multiple of 8 elements, both inside its tensor (so the Philox
// blocks line up) and inside the staging buffers (so 128-bit accesses stay aligned).
static void cut_into_chunks(const rt_tensor_desc* descs, uint32_t n, uint64_t chunk_elems,
                            std::vector<std::vector<Segment>>& chunks) {
    std::vector<Segment> cur;
    uint64_t used = 0;
    for (uint32_t i = 0; i < n; ++i) {
        uint64_t done = 0;
        const uint64_t numel = descs[i].numel;
        while (done < numel) {
            if (used >= chunk_elems) {
                chunks.push_back(std::move(cur));
                cur.clear();
                used = 0;
            }
            const uint64_t take = std::min(numel - done, chunk_elems - used);
            cur.push_back(Segment{i, done, take, used});
            done += take;
            used = align_up(used + take, kVec);  // next piece starts 16-byte aligned
        }
    }
    if (!cur.empty()) chunks.push_back(std::move(cur));
}

int rt_streamed_plan(const rt_tensor_desc* descs, uint32_t n, uint64_t chunk_elems, uint64_t* out, uint32_t cap,
                     uint32_t* n_out) {
    if (!n_out) return fail(RT_EINVAL, "n_out is NULL");
    if (n > 0 && !descs) return fail(RT_EINVAL, "descs is NULL");
    if (chunk_elems < kVec || (chunk_elems % kVec) != 0)
        return fail(RT_EINVAL, "chunk_elems %llu must be a positive multiple of 8", (unsigned long long)chunk_elems);
    std::vector<std::vector<Segment>> chunks;
    cut_into_chunks(descs, n, chunk_elems, chunks);
    uint32_t k = 0;
    for (size_t c = 0; c < chunks.size(); ++c)
        for (const Segment& s : chunks[c]) {
            if (out && k < cap) {
                uint64_t* row = out + 5 * (size_t)k;
                row[0] = c; row[1] = s.tensor; row[2] = s.start; row[3] = s.count; row[4] = s.stage_off;
            }
            ++k;
        }
    *n_out = k;
    return RT_OK;
}

// ---------------------------------------------------------------------------
// The order of everything a streamed call does, as data.  build_schedule lists, in the order the host
// issues them, the operations of a call over n_chunks chunks: what runs on which stream, which
// staging buffer and bounce slot it touches, which event it waits for and which it records, and where
// the host itself waits.  streamed_enqueue_impl executes exactly this list, and rt_streamed_schedule
// hands it out so that the discipline -- no staging or bounce buffer is written while something still
// reads it or reads it before it has been written -- can be checked on a CPU by replaying the list
// under arbitrary interleavings of the streams (tests/test_host.py).
//
//   H2D(c)    upload stream:  waits for D2H_DONE of the staging buffer's previous chunk, records H2D_DONE
//   KERNEL(c) compute stream: waits for H2D_DONE, records COMP_DONE
//   D2H(c)    download stream: waits for COMP_DONE, records D2H_DONE
// Up front (everything pinned) the whole call is queued at once, in batches of `batch` chunks with a
// drain in between.  Paced (some host array is not pinned) the host feeds the pipeline chunk by chunk:
// chunk c goes onto the streams when chunk c - kPacedInFlight has come back (a counter the download
// stream publishes behind every chunk), when host threads have filled its upload bounce slot, and when
// the copies out of the download bounce slot it is going to reuse are done.
// ---------------------------------------------------------------------------
static void build_schedule(uint32_t n_chunks, uint64_t seq0, uint32_t used_mask, bool paced_up, bool paced_down,
                           uint64_t batch, std::vector<rt_sched_op>& ops) {
    ops.clear();
    const bool paced = paced_up || paced_down;
    bool used[kStageBufs];
    for (int b = 0; b < kStageBufs; ++b) used[b] = (used_mask >> b) & 1u;
    auto push = [&](uint32_t kind, uint32_t chunk, uint32_t stage, uint32_t bounce, uint32_t wait_ev, uint32_t rec_ev,
                    uint64_t value) {
        rt_sched_op op;
        op.kind = kind; op.chunk = chunk; op.stage = stage; op.bounce = bounce;
        op.wait_event = wait_ev; op.record_event = rec_ev; op.value = value;
        ops.push_back(op);
    };
    const uint32_t none = RT_SCHED_NONE;
    auto slot_of = [&](uint64_t c) { return (uint32_t)((seq0 + c) % kBounce); };
    uint32_t fills_submitted = 0, drains_submitted = 0;
    if (paced && n_chunks) push(RT_OP_HOST_WAIT_IDLE, 0, none, none, none, none, 0);
    for (uint32_t c = 0; c < n_chunks; ++c) {
        const uint32_t b = (uint32_t)((seq0 + c) % kStageBufs);
        if (paced) {
            if (c >= kPacedInFlight) {
                push(RT_OP_HOST_WAIT_BACK, c - (uint32_t)kPacedInFlight, none, none, none, none, seq0 + c - kPacedInFlight + 1);
                if (paced_down) {   // that chunk's results lie in its download bounce slot: copy them out
                    push(RT_OP_HOST_DRAIN, c - (uint32_t)kPacedInFlight, none, slot_of(c - kPacedInFlight), none, none, 0);
                    drains_submitted = c - (uint32_t)kPacedInFlight + 1;
                }
            }
            if (paced_down && c >= (uint32_t)kBounce)   // the download slot of this chunk was chunk c - kBounce's
                push(RT_OP_HOST_WAIT_DRAIN, c - (uint32_t)kBounce, none, slot_of(c - kBounce), none, none, 0);
            if (paced_up) {
                // chunk k may be copied into its upload slot once chunk k - kBounce has left it, which is
                // known when that chunk has come back
                const uint32_t last = std::min<uint64_t>((uint64_t)c + kBounce - kPacedInFlight, n_chunks - 1);
                for (; fills_submitted <= last; ++fills_submitted)
                    push(RT_OP_HOST_FILL, fills_submitted, none, slot_of(fills_submitted), none, none, 0);
                push(RT_OP_HOST_WAIT_FILL, c, none, slot_of(c), none, none, 0);
            }
        } else if (c > 0 && batch > 0 && c % batch == 0) {
            // a long call is queued in batches and the pipeline drains between them
            push(RT_OP_PUBLISH, c - 1, none, none, none, none, seq0 + c);
            push(RT_OP_HOST_WAIT_BACK, c - 1, none, none, none, none, seq0 + c);
        }
        push(RT_OP_H2D, c, b, paced_up ? slot_of(c) : none, used[b] ? RT_EV_D2H_DONE + b : none, RT_EV_H2D_DONE + b, 0);
        push(RT_OP_KERNEL, c, b, none, RT_EV_H2D_DONE + b, RT_EV_COMP_DONE + b, 0);
        push(RT_OP_D2H, c, b, paced_down ? slot_of(c) : none, RT_EV_COMP_DONE + b, RT_EV_D2H_DONE + b, 0);
        used[b] = true;
        if (paced) push(RT_OP_PUBLISH, c, none, none, none, none, seq0 + c + 1);
    }
    push(RT_OP_TICKET, n_chunks ? n_chunks - 1 : 0, none, none, none, none, 0);
    if (paced_down) {
        // the last chunks: wait for each, copy its results out, and wait for every copy still running
        for (uint32_t c = drains_submitted; c < n_chunks; ++c) {
            push(RT_OP_HOST_WAIT_BACK, c, none, none, none, none, seq0 + c + 1);
            push(RT_OP_HOST_DRAIN, c, none, slot_of(c), none, none, 0);
        }
        for (uint32_t c = n_chunks > (uint32_t)kBounce ? n_chunks - kBounce : 0; c < n_chunks; ++c)
            push(RT_OP_HOST_WAIT_DRAIN, c, none, slot_of(c), none, none, 0);
    }
}

extern "C" int rt_streamed_schedule(uint32_t n_chunks, uint64_t seq0, uint32_t used_mask, int paced_up, int paced_down,
                                    uint64_t batch_chunks, rt_sched_op* out, uint32_t cap, uint32_t* n_out) {
    if (!n_out) return fail(RT_EINVAL, "n_out is NULL");
    if (used_mask >> kStageBufs) return fail(RT_EINVAL, "used_mask names a staging buffer that does not exist");
    std::vector<rt_sched_op> ops;
    build_schedule(n_chunks, seq0, used_mask, paced_up != 0, paced_down != 0, batch_chunks, ops);
    for (size_t i = 0; out && i < ops.size() && i < cap; ++i) out[i] = ops[i];
    *n_out = (uint32_t)ops.size();
    return RT_OK;
}

// Highest ticket whose copies have all landed: a plain read of pinned host memory.
static inline uint64_t tickets_done(const Streamed& st) {
    return st.ticket_word ? __atomic_load_n((const uint64_t*)st.ticket_word, __ATOMIC_ACQUIRE) : 0;
}


// Sleeps until ticket `want` has been published.  While the pipeline runs the host stays out
// of the runtime: a thread spinning in a synchronise call, or polling events, was measured to
// slow the copies down severalfold (the runtime resolves their cross-stream dependencies on
// host threads).  The sleep is bounded: after kStallSeconds without a new ticket it returns
// false and the caller falls back to a blocking synchronise, which also reports a failed device.
static bool sleep_until_word(const volatile uint64_t* word, uint64_t want) {
    constexpr double kStallSeconds = 60.0;
    if (!word) return false;
    auto read_word = [word] { return __atomic_load_n((const uint64_t*)word, __ATOMIC_ACQUIRE); };
    uint64_t seen = read_word();
    auto last_progress = std::chrono::steady_clock::now();
    while (seen < want) {
        std::this_thread::sleep_for(std::chrono::microseconds(100));
        const uint64_t now_done = read_word();
        const auto now = std::chrono::steady_clock::now();
        if (now_done != seen) {
            seen = now_done;
            last_progress = now;
        } else if (std::chrono::duration<double>(now - last_progress).count() > kStallSeconds) {
            return false;
        }
    }
    return true;
}

static bool sleep_until_ticket(const Streamed& st, uint64_t want) {
    return sleep_until_word(st.ticket_word, want);
}

static int streamed_wait(rt_handle* h) {
    Streamed& st = h->st;
    if (!st.ready) return RT_OK;
    HIP_TRY(hipSetDevice(h->device));
    (void)sleep_until_ticket(st, st.tickets_issued);
    // returns at once when the last ticket is out; otherwise this is the blocking fallback
    HIP_TRY(hipStreamSynchronize(st.d2h));
    HIP_TRY(hipStreamSynchronize(st.comp));
    HIP_TRY(hipStreamSynchronize(st.h2d));
    st.pending = false;
    for (auto& r : st.ring) r.in_flight = false;
    return RT_OK;
}

// True for host memory the runtime has pinned (hipHostMalloc, torch's pin_memory): copies from it
// are asynchronous.  Anything else -- an ordinary CPU tensor -- the runtime would stage through
// its own buffers while the calling thread waits.
static bool is_pinned_host(const void* p) {
    hipPointerAttribute_t attr;
    memset(&attr, 0, sizeof(attr));
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();  // unknown pointer: the error is the answer, not a failure
        return false;
    }
    return attr.type == hipMemoryTypeHost;
}

// Waits for the copies of every chunk whose fill has been submitted when a call leaves early: the
// workers read the caller's arrays and the groups live on the caller's stack.
namespace {
struct FillGuard {
    CopyPool* pool = nullptr;
    std::vector<CopyPool::Group*> started;   // groups with copies submitted
    ~FillGuard() {
        for (CopyPool::Group* g : started)
            if (pool) pool->wait(g);
    }
};
}  // namespace

// Validates and enqueues the whole pipeline of one call; does not wait for it.
static int streamed_enqueue_impl(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                            uint32_t n_scalars, uint64_t seed, int noise_mode, uint64_t chunk_elems,
                            const float* d_clip_coef, const uint32_t* d_skip, void* stream_, bool trace,
                            bool blocking, uint64_t* ticket_out) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    int rc = validate(descs, n, scalars, n_scalars, noise_mode, /*allow_host=*/true);
    if (rc != RT_OK) return rc;
    if (chunk_elems < kVec || (chunk_elems % kVec) != 0)
        return fail(RT_EINVAL, "chunk_elems %llu must be a positive multiple of 8", (unsigned long long)chunk_elems);
    if (noise_mode == RT_NOISE_EXPLICIT) {
        // noise arrays are addressed per piece below; they must be device resident
    }
    for (uint32_t i = 0; i < n; ++i)
        if (descs[i].row_mean && scalars[descs[i].scalars_idx].centralization != 0.0f && descs[i].row_len == 0)
            return fail(RT_EINVAL, "tensor %u: row_len is 0", i);
    hipStream_t user = (hipStream_t)stream_;
    HIP_TRY(hipSetDevice(h->device));
    rc = streamed_init(h);
    if (rc != RT_OK) return rc;
    Streamed& st = h->st;
    if (ticket_out) *ticket_out = st.tickets_issued;  // nothing to wait for beyond what is already issued
    if (n == 0) return RT_OK;

    // ---- cut the tensor list into chunks of at most chunk_elems staged elements
    std::vector<std::vector<Segment>> chunks;
    cut_into_chunks(descs, n, chunk_elems, chunks);

    // ---- staging buffers sized for the widest element type that is host resident
    int stage_esize[4] = {0, 0, 0, 0};
    for (uint32_t i = 0; i < n; ++i) {
        const rt_tensor_desc& d = descs[i];
        if (d.numel == 0) continue;
        if (d.host_mask & RT_HOST_P) stage_esize[0] = std::max(stage_esize[0], dtype_size(d.p_dtype));
        if (d.host_mask & RT_HOST_G) stage_esize[1] = std::max(stage_esize[1], dtype_size(d.g_dtype));
        if (d.host_mask & RT_HOST_M) stage_esize[2] = std::max(stage_esize[2], dtype_size(d.m_dtype));
        if (d.host_mask & RT_HOST_V) stage_esize[3] = std::max(stage_esize[3], dtype_size(d.v_dtype));
    }
    uint64_t max_used = 0;
    for (const auto& c : chunks)
        if (!c.empty()) max_used = std::max(max_used, align_up(c.back().stage_off + c.back().count, kVec));
    for (int a = 0; a < 4; ++a)
        for (int b = 0; b < kStageBufs; ++b)
            if (stage_esize[a]) {
                // sized for fp32 (or wider) so that the common dtype changes never reallocate
                const size_t want = max_used * std::max(4, stage_esize[a]);
                if (want > st.stage[a][b].cap && st.pending) {
                    rc = streamed_wait(h);  // the buffer may be in use by an earlier asynchronous call
                    if (rc != RT_OK) return rc;
                }
                rc = dev_reserve(st.stage[a][b], want);
                if (rc != RT_OK) return rc;
            }

    // ---- host arrays that are not pinned.  Their uploads go through pinned bounce buffers: host
    //      threads copy chunk c+1 and c+2 into them while chunk c is on the link, and the host hands
    //      the pipeline one chunk at a time (at most kPacedInFlight on the streams, see below)
    //      instead of queuing everything up front.  Left to the runtime, such a copy is staged
    //      inside hipMemcpyAsync while the calling thread waits, and nothing else gets queued.
    std::vector<uint8_t> unpinned_probe(n, 0);  // bit a: array a of the tensor is host memory that is not pinned
    for (uint32_t i = 0; i < n; ++i) {
        const rt_tensor_desc& d = descs[i];
        if (d.numel == 0) continue;
        const void* host[4] = {d.p, d.g, d.m, d.v};
        for (int a = 0; a < 4; ++a)
            if ((d.host_mask & (1u << a)) && !is_pinned_host(host[a])) unpinned_probe[i] |= (uint8_t)(1u << a);
    }
    std::vector<uint8_t> unpinned(n, 0);  // the same, for the arrays that go up through bounce buffers
    bool paced = false;
    if (st.bounce_threads > 0) {
        unpinned = unpinned_probe;
        for (uint32_t i = 0; i < n; ++i) paced |= unpinned[i] != 0;
    }
    if (paced) {
        // the bounce buffers and the chunk counter are shared with earlier calls: let those finish
        if (st.pending) {
            rc = streamed_wait(h);
            if (rc != RT_OK) return rc;
        }
        if (!st.pool) st.pool.reset(new CopyPool((unsigned)st.bounce_threads));
        bool need[4] = {false, false, false, false};
        for (uint32_t i = 0; i < n; ++i)
            for (int a = 0; a < 4; ++a) need[a] |= (unpinned[i] >> a) & 1;
        // upload slots for every such array, download slots for the ones that are written (not the gradient)
        for (int dir = 0; dir < 2 && paced; ++dir)
            for (int a = 0; a < 4; ++a) {
                if (dir == 1 && a == 1) continue;
                void* (&slots)[kBounce] = dir == 0 ? st.bounce[a] : st.bounce_down[a];
                size_t& cap = dir == 0 ? st.bounce_cap[a] : st.bounce_down_cap[a];
                const size_t want = max_used * (size_t)stage_esize[a];
                if (!need[a] || want <= cap) continue;
                for (int k = 0; k < kBounce; ++k) {
                    if (slots[k]) HIP_TRY(hipHostFree(slots[k]));
                    slots[k] = nullptr;
                }
                cap = 0;
                bool got_all = true;
                for (int k = 0; k < kBounce && got_all; ++k) {
                    if (hipHostMalloc(&slots[k], want, hipHostMallocDefault) != hipSuccess) {
                        (void)hipGetLastError();
                        slots[k] = nullptr;
                        got_all = false;
                    }
                }
                if (!got_all) {
                    // No pinned memory to be had (a locked-memory limit, say): this call leaves the unpinned
                    // copies to the runtime, which is slower but needs nothing from us.
                    for (int k = 0; k < kBounce; ++k) {
                        if (slots[k]) (void)hipHostFree(slots[k]);
                        slots[k] = nullptr;
                    }
                    paced = false;
                    break;
                }
                cap = want;
            }
        if (paced) {
            ++st.paced_calls;
        } else {
            std::fill(unpinned.begin(), unpinned.end(), (uint8_t)0);
        }
    }

    // ---- descriptors of every piece (pointers into staging for host-resident arrays), and the
    //      table images of all chunks, uploaded in one copy before the pipeline starts
    std::vector<std::vector<rt_tensor_desc>> pieces(chunks.size());
    std::vector<Plan> plans(chunks.size());
    std::vector<size_t> plan_off(chunks.size());
    std::vector<uint8_t> blob;
    for (size_t c = 0; c < chunks.size(); ++c) {
        const int b = (int)((st.seq + c) % kStageBufs);
        for (const Segment& s : chunks[c]) {
            const rt_tensor_desc& d = descs[s.tensor];
            rt_tensor_desc q = d;
            q.numel = s.count;
            q.elem_offset = d.elem_offset + s.start;
            q.host_mask = 0;
            const int es[4] = {dtype_size(d.p_dtype), dtype_size(d.g_dtype), dtype_size(d.m_dtype),
                               dtype_size(d.v_dtype)};
            const void* src[4] = {d.p, d.g, d.m, d.v};
            void* dst[4];
            for (int a = 0; a < 4; ++a)
                dst[a] = (d.host_mask & (1u << a)) ? (void*)((uint8_t*)st.stage[a][b].ptr + s.stage_off * es[a])
                                                   : (void*)((uint8_t*)src[a] + s.start * es[a]);
            q.p = dst[0]; q.g = dst[1]; q.m = dst[2]; q.v = dst[3];
            if (d.noise_p) q.noise_p = (const uint8_t*)d.noise_p + s.start * 2;
            if (d.noise_m) q.noise_m = (const uint8_t*)d.noise_m + s.start * 2;
            if (d.noise_v) q.noise_v = (const uint8_t*)d.noise_v + s.start * 2;
            if (d.dbg_p) q.dbg_p = d.dbg_p + s.start;
            if (d.dbg_m) q.dbg_m = d.dbg_m + s.start;
            if (d.dbg_v) q.dbg_v = d.dbg_v + s.start;
            pieces[c].push_back(q);
        }
        build_image(h, pieces[c].data(), (uint32_t)pieces[c].size(), scalars, noise_mode == RT_NOISE_EXPLICIT,
                    plans[c]);
        plan_off[c] = align_up(blob.size(), 256);
        blob.resize(plan_off[c] + plans[c].bytes);
        if (plans[c].bytes) memcpy(blob.data() + plan_off[c], h->image.data(), plans[c].bytes);
    }
    // A free pool entry (the call that used it has published its ticket), preferably one that is
    // already large enough.  With every entry in use the host sleeps until the oldest call is
    // done -- reading the ticket word, not waiting inside the runtime.
    size_t slot = st.ring.size();
    for (;;) {
        const uint64_t done_now = tickets_done(st);
        uint64_t oldest = UINT64_MAX;
        for (size_t i = 0; i < st.ring.size(); ++i) {
            Streamed::TableRing& r = st.ring[i];
            if (r.in_flight && r.ticket <= done_now) r.in_flight = false;
            if (r.in_flight) oldest = std::min(oldest, r.ticket);
            if (!r.in_flight && (slot == st.ring.size() || (st.ring[slot].host_cap < blob.size() && r.host_cap >= blob.size())))
                slot = i;
        }
        if (slot != st.ring.size()) break;
        if (!sleep_until_ticket(st, oldest)) {
            rc = streamed_wait(h);  // blocking fallback; frees every entry or reports the device error
            if (rc != RT_OK) return rc;
        }
    }
    Streamed::TableRing& tab = st.ring[slot];
    if (blob.size() > tab.host_cap) {
        if (tab.host) HIP_TRY(hipHostFree(tab.host));
        tab.host = nullptr;
        tab.host_cap = 0;
        const size_t want = blob.size() + blob.size() / 4 + 4096;
        hipError_t e = hipHostMalloc(&tab.host, want, hipHostMallocDefault);
        if (e != hipSuccess) return fail(RT_ENOMEM, "hipHostMalloc(%zu) failed: %s", want, hipGetErrorString(e));
        tab.host_cap = want;
    }
    rc = dev_reserve(tab.dev, blob.size() + 16);
    if (rc != RT_OK) return rc;
    memcpy(tab.host, blob.data(), blob.size());

    // grads (and anything else already queued by the caller) must be ready
    // The kernels read device arrays (gradients above all) that work on the caller's stream may still
    // be producing, so the compute stream always waits for it.  The upload stream waits only when it
    // has to: a copy engine waiting on a compute stream's event was measured to stall the pipeline
    // for 50 ms every few dozen chunks when updates are handed over chunk by chunk.  It has to when a
    // gradient lies in pinned host memory, which an asynchronous copy on the caller's stream may still
    // be filling (grad.to("cpu", non_blocking=True)), or when the caller asks for it (RT_HOST_ORDERED).
    // Host memory that is not pinned cannot be the target of an asynchronous copy, and host-resident
    // p / m / v are the optimizer's own to write.
    bool upload_waits = false;
    for (uint32_t i = 0; i < n && !upload_waits; ++i) {
        const rt_tensor_desc& d = descs[i];
        if (d.numel == 0) continue;
        upload_waits = (d.host_mask & RT_HOST_ORDERED) != 0 ||
                       ((d.host_mask & RT_HOST_G) != 0 && !(unpinned_probe[i] & RT_HOST_G));
    }
    HIP_TRY(hipEventRecord(st.start, user));
    // A call that returns only when everything is done, with nothing of the pipeline running yet,
    // waits for the caller's stream on the host, whatever the tensors: it costs nothing (the call
    // blocks anyway), it covers every way in which work on that stream may still be writing host
    // arrays, and even one wait on the upload stream per call was measured to cost most calls 50 ms.
    if (blocking && !st.pending) HIP_TRY(hipStreamSynchronize(user));
    else if (upload_waits) HIP_TRY(hipStreamWaitEvent(st.h2d, st.start, 0));
    HIP_TRY(hipStreamWaitEvent(st.comp, st.start, 0));
    if (!blob.empty()) {
        const uint64_t n_vec = (blob.size() + 15) / 16;  // buffers are padded well past the blob
        const uint32_t grid = (uint32_t)std::min<uint64_t>((n_vec + kThreads - 1) / kThreads, 64);
        hipLaunchKernelGGL(table_upload_kernel, dim3(grid), dim3(kThreads), 0, st.comp, (uint64_t)tab.dev.ptr,
                           (uint64_t)tab.host, n_vec);
        HIP_TRY(hipGetLastError());
    }

    st.bytes_h2d = st.bytes_d2h = 0;
    st.timeline.clear();
    st.pending = true;
    if (trace) {
        while (st.tl_events.size() < 4 * chunks.size()) {
            hipEvent_t e;
            HIP_TRY(hipEventCreate(&e));
            st.tl_events.push_back(e);
        }
    }
    // ---- the order of everything that follows is build_schedule's; this loop only carries it out
    bool paced_up = false, paced_down = false;
    for (uint32_t i = 0; i < n; ++i) {
        paced_up |= unpinned[i] != 0;
        paced_down |= (unpinned[i] & (RT_HOST_P | RT_HOST_M | RT_HOST_V)) != 0;
    }
    uint32_t used_mask = 0;
    for (int b = 0; b < kStageBufs; ++b) used_mask |= st.used_buf[b] ? 1u << b : 0u;
    std::vector<rt_sched_op> ops;
    build_schedule((uint32_t)chunks.size(), st.seq, used_mask, paced_up, paced_down, st.batch_chunks, ops);
    std::unique_ptr<CopyPool::Group[]> fills(paced_up ? new CopyPool::Group[chunks.size()] : nullptr);
    std::unique_ptr<CopyPool::Group[]> drains(paced_down ? new CopyPool::Group[chunks.size()] : nullptr);
    FillGuard guard;   // a call that leaves early waits for the copies already handed to the host threads
    guard.pool = st.pool.get();
    hipStream_t streams[3] = {st.h2d, st.comp, st.d2h};
    auto event_of = [&](uint32_t id) -> hipEvent_t {
        const uint32_t b = id & 1u;
        return id < RT_EV_COMP_DONE ? st.h2d_done[b] : id < RT_EV_D2H_DONE ? st.comp_done[b] : st.d2h_done[b];
    };
    for (const rt_sched_op& op : ops) {
        const size_t c = op.chunk;
        switch (op.kind) {
            case RT_OP_HOST_WAIT_BACK:
                // Every wait is a sleep on a word of pinned memory, never inside the runtime.
                if (!sleep_until_word(st.ticket_word + 1, op.value))
                    HIP_TRY(hipStreamSynchronize(st.d2h));  // stalled: block, and surface a device error
                break;
            case RT_OP_HOST_FILL:
            case RT_OP_HOST_DRAIN: {
                const bool up = op.kind == RT_OP_HOST_FILL;
                CopyPool::Group* grp = up ? &fills[c] : &drains[c];
                guard.started.push_back(grp);
                for (const Segment& sg : chunks[c]) {
                    const rt_tensor_desc& d = descs[sg.tensor];
                    const uint8_t mask = up ? unpinned[sg.tensor]
                                            : (uint8_t)(unpinned[sg.tensor] & (RT_HOST_P | RT_HOST_M | RT_HOST_V));
                    if (!mask) continue;
                    const int es[4] = {dtype_size(d.p_dtype), dtype_size(d.g_dtype), dtype_size(d.m_dtype),
                                       dtype_size(d.v_dtype)};
                    void* host[4] = {d.p, (void*)d.g, d.m, d.v};
                    for (int a = 0; a < 4; ++a)
                        if (mask & (1u << a)) {
                            uint8_t* user = (uint8_t*)host[a] + sg.start * es[a];
                            uint8_t* slot = (uint8_t*)(up ? st.bounce[a] : st.bounce_down[a])[op.bounce] + sg.stage_off * es[a];
                            if (up) st.pool->submit(grp, slot, user, sg.count * es[a]);
                            else st.pool->submit(grp, user, slot, sg.count * es[a]);
                            st.bounced_bytes += sg.count * es[a];
                        }
                }
                break;
            }
            case RT_OP_HOST_WAIT_IDLE:
                if (tickets_done(st) < st.tickets_issued) {
                    rc = streamed_wait(h);
                    if (rc != RT_OK) return rc;
                    st.pending = true;   // this call's own work follows
                }
                break;
            case RT_OP_HOST_WAIT_FILL: st.pool->wait(&fills[c]); break;
            case RT_OP_HOST_WAIT_DRAIN: st.pool->wait(&drains[c]); break;
            case RT_OP_H2D:
            case RT_OP_D2H: {
                const bool up = op.kind == RT_OP_H2D;
                hipStream_t stream = up ? st.h2d : st.d2h;
                if (op.wait_event != RT_SCHED_NONE) HIP_TRY(hipStreamWaitEvent(stream, event_of(op.wait_event), 0));
                if (trace) HIP_TRY(hipEventRecord(st.tl_events[4 * c + (up ? 0 : 2)], stream));
                const auto& segs = chunks[c];
                for (size_t k = 0; k < segs.size(); ++k) {
                    const Segment& sg = segs[k];
                    const rt_tensor_desc& d = descs[sg.tensor];
                    const int es[4] = {dtype_size(d.p_dtype), dtype_size(d.g_dtype), dtype_size(d.m_dtype),
                                       dtype_size(d.v_dtype)};
                    void* host[4] = {d.p, (void*)d.g, d.m, d.v};
                    void* dev[4] = {pieces[c][k].p, (void*)pieces[c][k].g, pieces[c][k].m, pieces[c][k].v};
                    for (int a = 0; a < 4; ++a) {
                        if (!(d.host_mask & (1u << a)) || (!up && a == 1)) continue;   // gradients only go up
                        const size_t bytes = sg.count * es[a];
                        const bool bounced = (unpinned[sg.tensor] & (1u << a)) != 0;
                        uint8_t* h_addr = bounced ? (uint8_t*)(up ? st.bounce[a] : st.bounce_down[a])[op.bounce] + sg.stage_off * es[a]
                                                  : (uint8_t*)host[a] + sg.start * es[a];
                        if (up) HIP_TRY(hipMemcpyAsync(dev[a], h_addr, bytes, hipMemcpyHostToDevice, stream));
                        else HIP_TRY(hipMemcpyAsync(h_addr, dev[a], bytes, hipMemcpyDeviceToHost, stream));
                        (up ? st.bytes_h2d : st.bytes_d2h) += (double)bytes;
                    }
                }
                if (trace) HIP_TRY(hipEventRecord(st.tl_events[4 * c + (up ? 1 : 3)], stream));
                HIP_TRY(hipEventRecord(event_of(op.record_event), stream));
                if (!up) st.used_buf[op.stage] = true;
                break;
            }
            case RT_OP_KERNEL:
                HIP_TRY(hipStreamWaitEvent(st.comp, event_of(op.wait_event), 0));
                rc = enqueue_kernels(plans[c], (const uint8_t*)tab.dev.ptr + plan_off[c], seed, noise_mode, d_clip_coef,
                                     d_skip, st.comp);
                if (rc != RT_OK) return rc;
                HIP_TRY(hipEventRecord(event_of(op.record_event), st.comp));
                break;
            case RT_OP_PUBLISH:
                hipLaunchKernelGGL(publish_ticket_kernel, dim3(1), dim3(1), 0, st.d2h, (uint64_t)(st.ticket_word + 1),
                                   op.value);
                HIP_TRY(hipGetLastError());
                break;
            case RT_OP_TICKET:
                st.seq += chunks.size();
                tab.ticket = st.tickets_issued + 1;
                tab.in_flight = true;
                // ticket: published when the last D2H of this call has landed (D2H follows compute, so
                // device-resident arrays are final by then as well)
                ++st.tickets_issued;
                hipLaunchKernelGGL(publish_ticket_kernel, dim3(1), dim3(1), 0, st.d2h, (uint64_t)st.ticket_word,
                                   st.tickets_issued);
                HIP_TRY(hipGetLastError());
                break;
            default: return fail(RT_EHIP, "internal: unknown operation %u in the schedule", op.kind);
        }
    }
    (void)streams;
    if (ticket_out) *ticket_out = st.tickets_issued;
    if (trace) st.timeline.assign(4 * chunks.size(), 0.0f);
    return RT_OK;
}

// A call that fails after it has started to enqueue (a HIP error halfway through the chunk loop)
// would leave the shared pipeline state -- buffer parity, buffer-free events -- out of step with
// what the streams hold.  Drain the streams and start over from a clean state; the error of the
// failed call is what the caller sees.
static int streamed_enqueue(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                            uint32_t n_scalars, uint64_t seed, int noise_mode, uint64_t chunk_elems,
                            const float* d_clip_coef, const uint32_t* d_skip, void* stream_, bool trace,
                            bool blocking, uint64_t* ticket_out) {
    const int rc = streamed_enqueue_impl(h, descs, n, scalars, n_scalars, seed, noise_mode, chunk_elems, d_clip_coef,
                                         d_skip, stream_, trace, blocking, ticket_out);
    if (rc != RT_OK && h && h->st.ready) {
        char saved[sizeof(g_err)];
        memcpy(saved, g_err, sizeof(saved));
        Streamed& st = h->st;
        (void)hipStreamSynchronize(st.h2d);
        (void)hipStreamSynchronize(st.comp);
        (void)hipStreamSynchronize(st.d2h);
        for (bool& u : st.used_buf) u = false;
        st.pending = false;
        for (auto& r : st.ring) r.in_flight = false;
        // The failed call may have published chunk counts beyond what `seq` says (it advances only when a
        // call succeeds): the next paced call must not take those for its own chunks coming back.
        if (st.ticket_word) {
            const uint64_t published = __atomic_load_n((const uint64_t*)(st.ticket_word + 1), __ATOMIC_ACQUIRE);
            if (published > st.seq) st.seq = published;
        }
        memcpy(g_err, saved, sizeof(saved));
    }
    return rc;
}

int rt_step_streamed(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                     uint32_t n_scalars, uint64_t seed, int noise_mode, uint64_t chunk_elems,
                     const float* d_clip_coef, const uint32_t* d_skip, void* stream) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    const auto wall0 = std::chrono::steady_clock::now();
    const bool trace = h->timing;
    int rc = streamed_enqueue(h, descs, n, scalars, n_scalars, seed, noise_mode, chunk_elems, d_clip_coef, d_skip,
                              stream, trace, /*blocking=*/true, nullptr);
    if (rc != RT_OK) return rc;
    // Host memory is final on return; device-resident arrays are final for the caller's stream.
    rc = streamed_wait(h);
    if (rc != RT_OK) return rc;
    Streamed& st = h->st;
    st.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - wall0).count();
    if (trace)
        for (size_t i = 0; i < st.timeline.size(); ++i)
            HIP_TRY(hipEventElapsedTime(&st.timeline[i], st.tl_events[0], st.tl_events[i]));
    return RT_OK;
}

int rt_step_streamed_async(rt_handle* h, const rt_tensor_desc* descs, uint32_t n, const rt_scalars* scalars,
                           uint32_t n_scalars, uint64_t seed, int noise_mode, uint64_t chunk_elems,
                           const float* d_clip_coef, const uint32_t* d_skip, void* stream, uint64_t* ticket) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    return streamed_enqueue(h, descs, n, scalars, n_scalars, seed, noise_mode, chunk_elems, d_clip_coef, d_skip,
                            stream, false, /*blocking=*/false, ticket);
}

int rt_streamed_wait(rt_handle* h) {
    if (!h) return fail(RT_EINVAL, "handle is NULL");
    return streamed_wait(h);
}

int rt_streamed_completed(rt_handle* h, uint64_t* ticket_done) {
    if (!h || !ticket_done) return fail(RT_EINVAL, "NULL argument");
    *ticket_done = tickets_done(h->st);
    return RT_OK;
}


int rt_streamed_timeline(rt_handle* h, float* out, uint32_t cap, uint32_t* n_out) {
    if (!h || !n_out) return fail(RT_EINVAL, "NULL argument");
    const uint32_t n = (uint32_t)h->st.timeline.size();
    *n_out = n;
    if (out)
        for (uint32_t i = 0; i < n && i < cap; ++i) out[i] = h->st.timeline[i];
    return RT_OK;
}

int rt_stream_probe(rt_handle* h, void* p, const void* g, void* m, void* v, uint64_t numel, int reps, float* ms_out,
                    void* stream_) {
    if (!h || !ms_out) return fail(RT_EINVAL, "NULL argument");
    if (!p || !g || !m || !v) return fail(RT_EINVAL, "NULL array pointer");
    if ((((uintptr_t)p | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v) & 15u) != 0)
        return fail(RT_EINVAL, "arrays must be 16-byte aligned");
    if (numel == 0 || numel % kChunkElems != 0 || numel / kChunkElems > 0x7FFFFFFFull)
        return fail(RT_EINVAL, "numel must be a positive multiple of %u", kChunkElems);
    if (reps < 1) return fail(RT_EINVAL, "reps must be >= 1");
    hipStream_t stream = (hipStream_t)stream_;
    HIP_TRY(hipSetDevice(h->device));
    const dim3 grid((uint32_t)(numel / kChunkElems));
    hipLaunchKernelGGL(stream_probe_kernel, grid, dim3(kThreads), 0, stream, (uint64_t)p, (uint64_t)g, (uint64_t)m,
                       (uint64_t)v);  // warm-up (page tables, clocks)
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipEventRecord(h->t0, stream));
    for (int r = 0; r < reps; ++r)
        hipLaunchKernelGGL(stream_probe_kernel, grid, dim3(kThreads), 0, stream, (uint64_t)p, (uint64_t)g,
                           (uint64_t)m, (uint64_t)v);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipEventRecord(h->t1, stream));
    HIP_TRY(hipEventSynchronize(h->t1));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, h->t0, h->t1));
    *ms_out = ms / (float)reps;
    return RT_OK;
}

int rt_host_link_probe(rt_handle* h, uint64_t bytes, int reps, double out[3]) {
    if (!h || !out) return fail(RT_EINVAL, "NULL argument");
    if (bytes == 0 || reps < 1) return fail(RT_EINVAL, "bytes and reps must be positive");
    HIP_TRY(hipSetDevice(h->device));
    int rc = streamed_init(h);
    if (rc != RT_OK) return rc;
    rc = streamed_wait(h);
    if (rc != RT_OK) return rc;
    Streamed& st = h->st;
    void *hbuf[2] = {nullptr, nullptr}, *dbuf[2] = {nullptr, nullptr};
    hipError_t e = hipSuccess;
    for (int k = 0; k < 2 && e == hipSuccess; ++k) {
        e = hipHostMalloc(&hbuf[k], bytes, hipHostMallocDefault);
        if (e == hipSuccess) e = hipMalloc(&dbuf[k], bytes);
    }
    auto release = [&] {
        for (int k = 0; k < 2; ++k) {
            if (hbuf[k]) (void)hipHostFree(hbuf[k]);
            if (dbuf[k]) (void)hipFree(dbuf[k]);
        }
    };
    if (e != hipSuccess) {
        release();
        (void)hipGetLastError();
        return fail(RT_ENOMEM, "allocating the probe buffers (%llu bytes each) failed: %s", (unsigned long long)bytes,
                    hipGetErrorString(e));
    }
    memset(hbuf[0], 0, bytes);
    memset(hbuf[1], 0, bytes);
    using clock = std::chrono::steady_clock;
    auto run = [&](bool up, bool down) -> double {   // seconds for `reps` copies each way
        if (up) (void)hipMemcpyAsync(dbuf[0], hbuf[0], bytes, hipMemcpyHostToDevice, st.h2d);    // warm-up
        if (down) (void)hipMemcpyAsync(hbuf[1], dbuf[1], bytes, hipMemcpyDeviceToHost, st.d2h);
        (void)hipStreamSynchronize(st.h2d);
        (void)hipStreamSynchronize(st.d2h);
        const auto t0 = clock::now();
        for (int r = 0; r < reps; ++r) {
            if (up) (void)hipMemcpyAsync(dbuf[0], hbuf[0], bytes, hipMemcpyHostToDevice, st.h2d);
            if (down) (void)hipMemcpyAsync(hbuf[1], dbuf[1], bytes, hipMemcpyDeviceToHost, st.d2h);
        }
        (void)hipStreamSynchronize(st.h2d);
        (void)hipStreamSynchronize(st.d2h);
        return std::chrono::duration<double>(clock::now() - t0).count();
    };
    const double total = (double)bytes * reps / 1e9;
    out[0] = total / run(true, false);
    out[1] = total / run(false, true);
    out[2] = total / run(true, true);
    release();
    HIP_TRY(hipGetLastError());
    return RT_OK;
}

int rt_dev_hold(rt_handle* h, uint64_t bytes, void** out) {
    if (!h || !out) return fail(RT_EINVAL, "NULL argument");
    *out = nullptr;
    if (bytes == 0) return fail(RT_EINVAL, "bytes must be positive");
    HIP_TRY(hipSetDevice(h->device));
    void* p = nullptr;
    const hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // a failed allocation must not surface again behind a later launch
        return fail(RT_ENOMEM, "hipMalloc(%llu) failed: %s", (unsigned long long)bytes, hipGetErrorString(e));
    }
    *out = p;
    return RT_OK;
}

// ---------------------------------------------------------------------------
// rt_dev_hold_pair: two blocks assembled from physical chunks that were probed one by one.
// ---------------------------------------------------------------------------
namespace {
constexpr size_t kPairChunk = 1ull << 30;          // physical chunks of 1 GiB
constexpr uint64_t kPairProbeElems = 128ull << 20;  // 256 MiB of bf16 per probed array: three of them and a fourth fit a chunk
constexpr uint64_t kPairMinProbeElems = 32ull << 20;  // shorter probes scatter too much to tell the regions apart

struct PairBlock {   // one block handed out by rt_dev_hold_pair
    size_t bytes = 0;
    int device = 0;
    std::vector<hipMemGenericAllocationHandle_t> chunks;
};
std::mutex g_pair_mutex;
std::map<void*, PairBlock> g_pair_blocks;

// Unmaps `mapped` chunks of 1 GiB that sit side by side from `va` on, releases their handles and
// frees the address range of `reserved` bytes; goes on after an error and returns the first one.
static hipError_t pair_teardown(void* va, size_t reserved, std::vector<hipMemGenericAllocationHandle_t>& chunks,
                                size_t mapped) {
    hipError_t first = hipSuccess;
    auto note = [&](hipError_t e) { if (e != hipSuccess && first == hipSuccess) first = e; };
    for (size_t i = 0; va && i < mapped; ++i) note(hipMemUnmap((uint8_t*)va + i * kPairChunk, kPairChunk));
    for (auto hnd : chunks) note(hipMemRelease(hnd));
    chunks.clear();
    if (va && reserved) note(hipMemAddressFree(va, reserved));
    return first;
}
}  // namespace

int rt_dev_hold_pair(rt_handle* h, uint64_t bytes_a, uint64_t bytes_b, uint64_t max_extra_bytes, double max_seconds,
                     void* ref_p, void* ref_m, void* ref_v, uint64_t ref_elems, void** a_out, void** b_out,
                     double report[8], void* stream_) {
    if (!h || !a_out || !b_out || !report) return fail(RT_EINVAL, "NULL argument");
    *a_out = *b_out = nullptr;
    for (int i = 0; i < 8; ++i) report[i] = 0.0;
    if (bytes_a == 0 || bytes_b == 0) return fail(RT_EINVAL, "sizes must be positive");
    const bool has_ref = ref_elems != 0;
    if (has_ref) {
        if (!ref_p || !ref_m || !ref_v || (((uintptr_t)ref_p | (uintptr_t)ref_m | (uintptr_t)ref_v) & 15u) != 0)
            return fail(RT_EINVAL, "reference arrays must be 16-byte aligned device addresses");
        if (ref_elems % kChunkElems != 0 || ref_elems < kPairMinProbeElems || ref_elems > kPairProbeElems)
            return fail(RT_EINVAL, "ref_elems must be a multiple of %u between %llu and %llu", kChunkElems,
                        (unsigned long long)kPairMinProbeElems, (unsigned long long)kPairProbeElems);
    }
    const uint64_t probe_elems = has_ref ? ref_elems : kPairProbeElems;
    HIP_TRY(hipSetDevice(h->device));
    hipStream_t stream = (hipStream_t)stream_;
    const auto t_start = std::chrono::steady_clock::now();
    auto elapsed = [&] { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count(); };
    const size_t C = kPairChunk;
    const size_t n_a = (bytes_a + C - 1) / C, n_b = (bytes_b + C - 1) / C;
    const size_t n_max = n_a + n_b + (size_t)(max_extra_bytes / C);

    hipMemAllocationProp prop;
    memset(&prop, 0, sizeof(prop));
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = h->device;
    hipMemAccessDesc access;
    memset(&access, 0, sizeof(access));
    access.location = prop.location;
    access.flags = hipMemAccessFlagsProtReadWrite;
    size_t gran = 0;
    if (hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended) != hipSuccess || gran == 0 ||
        C % gran != 0) {
        (void)hipGetLastError();
        return fail(RT_EUNSUPPORTED, "the device has no virtual-memory allocation of 1 GiB chunks");
    }

    // Every chunk is mapped where it was taken, side by side in one scratch range, and probed there.
    void* scratch = nullptr;
    if (hipMemAddressReserve(&scratch, n_max * C, 0, nullptr, 0) != hipSuccess) {
        (void)hipGetLastError();
        return fail(RT_EUNSUPPORTED, "reserving %zu GiB of device address space failed", n_max);
    }
    std::vector<hipMemGenericAllocationHandle_t> chunks;   // chunk k is mapped at scratch + k * C
    std::vector<float> rate;                                // GB/s of the probe with ema_squared in chunk k; < 0: mixed
    auto fail_all = [&](int code, const char* what, hipError_t e) {
        (void)hipDeviceSynchronize();
        (void)pair_teardown(scratch, n_max * C, chunks, chunks.size());
        (void)hipGetLastError();
        return fail(code, "%s: %s", what, hipGetErrorString(e));
    };
    // The update's traffic with ema_squared where the caller says.  Without reference arrays p, g and ema
    // stand in the first chunk.  With them, p and ema are the caller's own arrays -- parameter memory, so
    // that "the first kind" means "where the parameters are"; the probe writes p ^ g and ema ^ g back and
    // g is a zeroed part of the first chunk, so every bit of them stays as it is.
    bool use_ref = has_ref;   // dropped when the reference arrays turn out not to lie in one region themselves
    auto probe4 = [&](uint64_t pp, uint64_t gg, uint64_t mm, uint64_t vv, float* gbps) -> hipError_t {
        const dim3 grid((uint32_t)(probe_elems / kChunkElems));
        hipLaunchKernelGGL(stream_probe_kernel, grid, dim3(kThreads), 0, stream, pp, gg, mm, vv);
        hipError_t e = hipEventRecord(h->t0, stream);
        for (int r = 0; r < 3 && e == hipSuccess; ++r)
            hipLaunchKernelGGL(stream_probe_kernel, grid, dim3(kThreads), 0, stream, pp, gg, mm, vv);
        if (e == hipSuccess) e = hipGetLastError();
        if (e == hipSuccess) e = hipEventRecord(h->t1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(h->t1);
        float ms = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, h->t0, h->t1);
        if (e == hipSuccess) *gbps = (float)(14.0 * (double)probe_elems * 3 / (ms * 1e-3) / 1e9);
        return e;
    };
    auto probe = [&](void* v, float* gbps) -> hipError_t {
        uint8_t* base = (uint8_t*)scratch;
        const size_t arr = probe_elems * 2;
        if (use_ref) return probe4((uint64_t)ref_p, (uint64_t)base, (uint64_t)ref_m, (uint64_t)v, gbps);
        return probe4((uint64_t)base, (uint64_t)(base + arr), (uint64_t)(base + 2 * arr), (uint64_t)v, gbps);
    };

    float lo = 0.0f, hi = 0.0f;   // mean rates of the two kinds of chunk
    size_t near_n = 0, far_n = 0;
    // Two kinds of chunk: those that run at the rate of the first chunk's own region and those that run at the
    // higher rate of another region.  Two-means over the rates seen so far; the kinds count as told apart only
    // when their means differ by 4 % (single probes scatter by 2 - 3 %, the regions differ by 7 %).
    // (With reference arrays the rates come in three levels, e.g. 5.9 / 6.2 / 6.44 TB/s: the chunk in the
    // parameters' region; elsewhere, with the gradient's stand-in -- the first chunk -- in a third region; and
    // elsewhere with it in one of the two.  The lowest level is the first kind, the two others are the second.)
    float ref_level = 0.0f;   // with reference arrays: the rate with ema_squared in parameter memory as well
    auto classify = [&]() -> float {
        near_n = far_n = 0;
        float mn = 1e30f, mx = 0.0f;
        for (float r : rate)
            if (r >= 0.0f) { mn = std::min(mn, r); mx = std::max(mx, r); }
        if (mx == 0.0f) return 1e30f;
        float c1 = mn, c2 = mx;
        for (int it = 0; it < 8; ++it) {
            const float mid = 0.5f * (c1 + c2);
            double s1 = 0, s2 = 0;
            size_t k1 = 0, k2 = 0;
            for (float r : rate) {
                if (r < 0.0f) continue;
                if (r < mid) { s1 += r; ++k1; } else { s2 += r; ++k2; }
            }
            if (k1) c1 = (float)(s1 / k1);
            if (k2) c2 = (float)(s2 / k2);
        }
        lo = c1;
        hi = c2;
        // One kind only so far: without reference arrays it is the first chunk's; with them it is "elsewhere"
        // when it runs 3.5 % faster than the probe that has all its arrays inside the parameters' memory.
        float thr = 1e30f;
        if (c2 >= 1.04f * c1) thr = 0.5f * (c1 + c2);
        else if (use_ref && 0.5f * (c1 + c2) >= 1.035f * ref_level) thr = 0.0f;
        for (float r : rate) {
            if (r < 0.0f) continue;
            (r < thr ? near_n : far_n) += 1;
        }
        return thr;
    };
    // Without reference arrays either block may be the one in the first chunk's region.  With them, the second
    // block is the one away from the parameters and the first lies with them; when their region has too few free
    // chunks for that, the search runs to its limits and the first block is completed with chunks from elsewhere
    // (the parameters then have their region to themselves, which is still better than sharing it with both).
    auto is_complete = [&] {
        if (use_ref) return far_n >= n_b && near_n >= n_a;
        return (near_n >= n_a && far_n >= n_b) || (far_n >= n_a && near_n >= n_b);
    };
    double create_seconds = 0.0;   // spent inside hipMemCreate so far
    double base_seconds = 0.0;     // when the chunks that the blocks need anyway had been taken
    int ended = 0;   // 0: both blocks complete, 1: memory limit, 2: time limit, 3: no more free chunks
    bool complete = false;
    while (true) {
        classify();
        if (is_complete()) {
            complete = true;
            break;
        }
        if (chunks.size() >= n_max) { ended = 1; break; }
        // Time.  The chunks that the two blocks consist of have to be taken whatever their kind: the limit is for
        // what the search costs beyond that.  While the driver is still clearing memory that was given back shortly
        // before (by this process or by one that has just ended), it hands out chunks only as fast as it clears
        // them, about 30 ms per GiB instead of next to nothing, and takes as long to take them back; the search is
        // then given two and a half times as long, because a place found once serves every step that follows.
        const size_t surplus = chunks.size() > n_a + n_b ? chunks.size() - (n_a + n_b) : 0;
        const double per_chunk = chunks.empty() ? 0.0 : create_seconds / (double)chunks.size();
        if (chunks.size() == n_a + n_b) base_seconds = elapsed();
        if (surplus && elapsed() - base_seconds > (per_chunk > 0.012 ? 2.5 : 1.0) * max_seconds) { ended = 2; break; }
        hipMemGenericAllocationHandle_t hnd;
        const double t_create = elapsed();
        hipError_t e = hipMemCreate(&hnd, C, &prop, 0);
        create_seconds += elapsed() - t_create;
        if (e != hipSuccess) {
            (void)hipGetLastError();
            ended = 3;
            break;
        }
        uint8_t* at = (uint8_t*)scratch + chunks.size() * C;
        e = hipMemMap(at, C, 0, hnd, 0);
        if (e != hipSuccess) {
            (void)hipMemRelease(hnd);
            return fail_all(RT_EHIP, "hipMemMap", e);
        }
        chunks.push_back(hnd);
        e = hipMemSetAccess(at, C, &access, 1);
        if (e != hipSuccess) return fail_all(RT_EHIP, "hipMemSetAccess", e);
        float r0 = 0.0f, r1 = 0.0f;
        const size_t arr = probe_elems * 2;
        if (chunks.size() == 1 && use_ref) {
            // The first chunk holds the zeroed stand-in for the gradient at its beginning.  First of all the
            // reference arrays are checked against the chunk: with all four arrays inside one chunk the probe runs
            // at the rate of a single region, and with all of them inside the parameters' memory it must run no
            // faster -- if it does, that memory lies across a region boundary itself and is no reference.
            e = hipMemsetAsync(at, 0, arr, stream);
            float l0 = 0.0f, l1 = 0.0f, own = 0.0f;
            if (e == hipSuccess) e = probe(ref_v, &l0);
            if (e == hipSuccess) e = probe(ref_v, &l1);
            ref_level = std::max(l0, l1);
            for (int rep = 0; rep < 2 && e == hipSuccess; ++rep) {
                float r = 0.0f;
                e = probe4((uint64_t)(at + arr), (uint64_t)at, (uint64_t)(at + 2 * arr), (uint64_t)(at + 3 * arr), &r);
                own = std::max(own, r);
            }
            // (two regions differ by 7 %, single probes scatter by 2 - 3 %)
            if (e == hipSuccess && ref_level > 1.05f * own) use_ref = false;
        }
        if (e != hipSuccess) return fail_all(RT_EHIP, "probing a chunk", e);
        if (chunks.size() == 1 && use_ref) {
            e = probe(at + arr, &r0);
            if (e == hipSuccess) e = probe(at + C - arr, &r1);
        } else if (chunks.size() == 1) {
            // all four arrays inside the first chunk: the rate of one region
            e = probe(at + 3 * arr, &r0);
            r1 = r0;
        } else {
            e = probe(at, &r0);
            if (e == hipSuccess) e = probe(at + C - arr, &r1);
        }
        if (e != hipSuccess) return fail_all(RT_EHIP, "probing a chunk", e);
        const float mean = 0.5f * (r0 + r1);
        // a chunk whose two ends disagree lies across a region boundary: it serves neither block
        rate.push_back(fabsf(r0 - r1) > 0.04f * mean ? -1.0f : mean);
    }
    const float thr = classify();
    complete = is_complete();
    // Without reference arrays: the block that must lie in one region takes the chunks of the first chunk's kind
    // ("near"), the other takes chunks that are anywhere else -- whichever way round the counts allow.
    const bool a_is_near = use_ref ? true : !(complete && !(near_n >= n_a && far_n >= n_b));
    std::vector<size_t> pick_a, pick_b, rest;
    for (size_t k = 0; k < chunks.size(); ++k) {
        const bool usable = rate[k] >= 0.0f;
        const bool is_near = usable && rate[k] < thr;
        const bool is_far = usable && !is_near;
        if (use_ref) {
            // far chunks go to the second block first; the first block takes near ones, or far ones that are left
            if (is_far && pick_b.size() < n_b) pick_b.push_back(k);
            else if ((a_is_near ? is_near : is_far) && pick_a.size() < n_a) pick_a.push_back(k);
            else rest.push_back(k);
        } else if ((a_is_near ? is_near : is_far) && pick_a.size() < n_a) pick_a.push_back(k);
        else if ((a_is_near ? is_far : is_near) && pick_b.size() < n_b) pick_b.push_back(k);
        else rest.push_back(k);
    }
    const size_t good_b = pick_b.size();
    // not enough of a kind: the blocks are completed with whatever else was taken, and with fresh chunks
    for (int which = 0; which < 2; ++which) {
        std::vector<size_t>& pick = which ? pick_b : pick_a;
        const size_t want = which ? n_b : n_a;
        while (pick.size() < want && !rest.empty()) {
            pick.push_back(rest.back());
            rest.pop_back();
        }
    }
    (void)hipStreamSynchronize(stream);
    // ---- the final blocks: the picked chunks side by side in address ranges of their own
    void* va[2] = {nullptr, nullptr};
    std::vector<hipMemGenericAllocationHandle_t> mine[2];
    const std::vector<size_t>* picks[2] = {&pick_a, &pick_b};
    const size_t want_n[2] = {n_a, n_b};
    size_t n_mapped[2] = {0, 0};
    hipError_t e = hipSuccess;
    for (size_t k = 0; k < chunks.size() && e == hipSuccess; ++k) e = hipMemUnmap((uint8_t*)scratch + k * C, C);
    std::vector<bool> taken(chunks.size(), false);
    for (int which = 0; which < 2 && e == hipSuccess; ++which) {
        e = hipMemAddressReserve(&va[which], want_n[which] * C, 0, nullptr, 0);
        if (e != hipSuccess) { va[which] = nullptr; break; }
        for (size_t k : *picks[which]) {
            mine[which].push_back(chunks[k]);
            taken[k] = true;
        }
        while (mine[which].size() < want_n[which] && e == hipSuccess) {   // the search ended early: fresh chunks
            hipMemGenericAllocationHandle_t hnd;
            e = hipMemCreate(&hnd, C, &prop, 0);
            if (e == hipSuccess) mine[which].push_back(hnd);
        }
        for (size_t i = 0; i < mine[which].size() && e == hipSuccess; ++i) {
            e = hipMemMap((uint8_t*)va[which] + i * C, C, 0, mine[which][i], 0);
            if (e == hipSuccess) {
                ++n_mapped[which];
                e = hipMemSetAccess((uint8_t*)va[which] + i * C, C, &access, 1);
            }
        }
        if (e == hipSuccess) e = hipMemsetAsync(va[which], 0, want_n[which] * C, stream);
    }
    // chunks that serve neither block go back to the driver, and so does the scratch range
    for (size_t k = 0; k < chunks.size(); ++k)
        if (!taken[k]) (void)hipMemRelease(chunks[k]);
    (void)hipMemAddressFree(scratch, n_max * C);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
        (void)hipDeviceSynchronize();
        for (int which = 0; which < 2; ++which)
            (void)pair_teardown(va[which], va[which] ? want_n[which] * C : 0, mine[which], n_mapped[which]);
        (void)hipGetLastError();
        return fail(e == hipErrorOutOfMemory ? RT_ENOMEM : RT_EHIP, "assembling the two blocks failed: %s",
                    hipGetErrorString(e));
    }
    {
        std::lock_guard<std::mutex> lock(g_pair_mutex);
        for (int which = 0; which < 2; ++which) {
            PairBlock pb;
            pb.bytes = want_n[which] * C;
            pb.device = h->device;
            pb.chunks = std::move(mine[which]);
            g_pair_blocks[va[which]] = std::move(pb);
        }
    }
    *a_out = va[0];
    *b_out = va[1];
    report[0] = complete ? 1.0 : 0.0;
    report[1] = (double)good_b / (double)n_b;          // share of the second block that lies apart from the first
    report[2] = (double)rate.size();                    // chunks taken and probed
    report[3] = elapsed();
    report[4] = lo;                                     // GB/s of the probe with everything in one region ...
    report[5] = hi;                                     // ... and with ema_squared in another
    report[6] = (double)ended;
    report[7] = use_ref ? 2.0 : a_is_near ? 1.0 : 0.0;
    return RT_OK;
}

int rt_dev_release(rt_handle* h, void* p) {
    if (!p) return RT_OK;
    {
        std::unique_lock<std::mutex> lock(g_pair_mutex);
        auto it = g_pair_blocks.find(p);
        if (it != g_pair_blocks.end()) {
            PairBlock pb = std::move(it->second);
            g_pair_blocks.erase(it);
            lock.unlock();
            HIP_TRY(hipSetDevice(pb.device));
            HIP_TRY(hipDeviceSynchronize());   // nothing may still be using the block when its mapping goes
            const hipError_t e = pair_teardown(p, pb.bytes, pb.chunks, pb.chunks.size());
            if (e != hipSuccess) return fail(RT_EHIP, "releasing a block of rt_dev_hold_pair: %s", hipGetErrorString(e));
            return RT_OK;
        }
    }
    if (h) HIP_TRY(hipSetDevice(h->device));
    HIP_TRY(hipFree(p));  // the runtime finds the owning device by the address
    return RT_OK;
}

int rt_selftest_sqrt(rt_handle* h, uint64_t* mismatches) {
    if (!h || !mismatches) return fail(RT_EINVAL, "NULL argument");
    HIP_TRY(hipSetDevice(h->device));
    unsigned long long* d = nullptr;
    HIP_TRY(hipMalloc((void**)&d, sizeof(*d)));
    hipError_t e = hipMemset(d, 0, sizeof(*d));
    if (e == hipSuccess) {
        hipLaunchKernelGGL(sqrt_selftest_kernel, dim3(16384), dim3(kThreads), 0, nullptr, d);
        e = hipGetLastError();
    }
    unsigned long long host = 0;
    if (e == hipSuccess) e = hipMemcpy(&host, d, sizeof(host), hipMemcpyDeviceToHost);
    (void)hipFree(d);
    if (e != hipSuccess) return fail(RT_EHIP, "sqrt self-test failed: %s (%d)", hipGetErrorString(e), (int)e);
    *mismatches = host;
    return RT_OK;
}

int rt_streamed_stats(rt_handle* h, double out[3]) {
    if (!h || !out) return fail(RT_EINVAL, "NULL argument");
    out[0] = h->st.bytes_h2d;
    out[1] = h->st.bytes_d2h;
    out[2] = h->st.seconds;
    return RT_OK;
}

int rt_streamed_bounce_stats(rt_handle* h, uint64_t out[2]) {
    if (!h || !out) return fail(RT_EINVAL, "NULL argument");
    out[0] = h->st.paced_calls;
    out[1] = h->st.bounced_bytes;
    return RT_OK;
}

}  // extern "C"
