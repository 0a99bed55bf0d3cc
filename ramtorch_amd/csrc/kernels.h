// Device code of the stochastic-rounding AdamW step for gfx950 (wave64).
//
// The step is HBM-bound (14 bytes and ~25 flops per all-bf16 element), so the
// kernels are plain vector code: 128-bit global loads and stores (64-bit ones
// for 16-bit arrays in the layout with fp32 arrays), each instruction
// contiguous across the wave, fp32 math in registers, a counter-based
// Philox4x32-10 for the rounding noise.  No LDS and no MFMA in the update;
// wavefront reductions only in the norm / row-mean passes.
//
// Floating-point contraction is switched off for the whole file: the rounding
// sequence of every operation is part of the contract (it has to reproduce
// torch's GPU kernels bit for bit), so each fused multiply-add below is an
// explicit __builtin_fmaf and nothing else may fuse.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_types.h"

#pragma clang fp contract(off)

namespace rt {

// Every tensor pointer arrives as a 64-bit integer from a table; telling the
// compiler it is global memory (address space 1) yields global_load/store
// instead of flat accesses.
#define RT_GLOBAL __attribute__((address_space(1)))
// The tables a launch reads (scalars, tensor records, work lists, clip coefficient, skip flag) do not
// change while its kernels run.  Reading them through the constant address space says so: a load
// whose address is uniform then becomes a scalar load into scalar registers.  Through a plain
// pointer the compiler cannot rule out that the kernel's own stores hit the table, issues a vector
// load per lane and keeps the record in vector registers (20 more of them in the fast kernel).
#define RT_CONST __attribute__((address_space(4)))
template <typename T>
__device__ __forceinline__ T load_const(const T* p) {
    static_assert(sizeof(T) % 4 == 0, "table records are whole words");
    T out;
    const RT_CONST uint32_t* src = (const RT_CONST uint32_t*)(uint64_t)p;
    uint32_t* dst = (uint32_t*)&out;
#pragma unroll
    for (int k = 0; k < (int)(sizeof(T) / 4); ++k) dst[k] = src[k];
    return out;
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// The step streams every byte exactly once, so the 128-bit accesses carry the
// nontemporal hint: lines are not kept in L2 (4 MB per XCD, far smaller than
// what 256 CUs have in flight), which removed re-fetches of evicted lines and
// measured ~10 % faster than plain accesses on the 8B-element set.
__device__ __forceinline__ u32x4 ldg128(uint64_t addr) {
    return __builtin_nontemporal_load((const RT_GLOBAL u32x4*)addr);
}
__device__ __forceinline__ void stg128(uint64_t addr, u32x4 v) {
    __builtin_nontemporal_store(v, (RT_GLOBAL u32x4*)addr);
}
__device__ __forceinline__ uint32_t ldg16(uint64_t addr) { return *(const RT_GLOBAL uint16_t*)addr; }
__device__ __forceinline__ void stg16(uint64_t addr, uint32_t v) { *(RT_GLOBAL uint16_t*)addr = (uint16_t)v; }
__device__ __forceinline__ float ldg32f(uint64_t addr) { return *(const RT_GLOBAL float*)addr; }
__device__ __forceinline__ void stg32f(uint64_t addr, float v) { *(RT_GLOBAL float*)addr = v; }

template <int DT>
__device__ __forceinline__ constexpr int esize() {
    return DT == RT_DT_F32 ? 4 : 2;
}

// ---------------------------------------------------------------------------
// Philox4x32-10 (Salmon et al. 2011).  The key schedule is wave-uniform (the
// key is the seed), so the per-round key bumps stay in scalar registers.
// ---------------------------------------------------------------------------
// a ^ b ^ c in one VALU instruction (gfx950 v_bitop3_b32, truth table 0x96).
__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
    return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
}

__device__ __forceinline__ u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                               uint32_t k1) {
    constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
    constexpr uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)M0 * c0;
        const uint64_t p1 = (uint64_t)M1 * c2;
        const uint32_t n0 = xor3((uint32_t)(p1 >> 32), c1, k0);
        const uint32_t n2 = xor3((uint32_t)(p0 >> 32), c3, k1);
        c1 = (uint32_t)p1;
        c3 = (uint32_t)p0;
        c0 = n0;
        c2 = n2;
        k0 += W0;
        k1 += W1;
    }
    u32x4 r;
    r.x = c0; r.y = c1; r.z = c2; r.w = c3;
    return r;
}

// ---------------------------------------------------------------------------
// Raw 8-element vectors: one 128-bit word for 16-bit types, two for fp32.
// ---------------------------------------------------------------------------
template <int DT>
struct Raw8 {
    u32x4 a;
    u32x4 b;  // used by fp32 only
};

template <int DT>
__device__ __forceinline__ Raw8<DT> load_raw(uint64_t base, uint64_t i) {
    Raw8<DT> r;
    const uint64_t addr = base + i * esize<DT>();
    r.a = ldg128(addr);
    if constexpr (DT == RT_DT_F32) r.b = ldg128(addr + 16);
    return r;
}

// Per-element load for tails and unaligned tensors: elements at or past n read as 0.
template <int DT>
__device__ __forceinline__ Raw8<DT> load_raw_guarded(uint64_t base, uint64_t i, uint64_t n) {
    Raw8<DT> r;
    uint32_t w[8];
    if constexpr (DT == RT_DT_F32) {
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = (i + j < n) ? f2u(ldg32f(base + (i + j) * 4)) : 0u;
        r.a.x = w[0]; r.a.y = w[1]; r.a.z = w[2]; r.a.w = w[3];
        r.b.x = w[4]; r.b.y = w[5]; r.b.z = w[6]; r.b.w = w[7];
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t lo = (i + 2 * k < n) ? ldg16(base + (i + 2 * k) * 2) : 0u;
            const uint32_t hi = (i + 2 * k + 1 < n) ? ldg16(base + (i + 2 * k + 1) * 2) : 0u;
            w[k] = lo | (hi << 16);
        }
        r.a.x = w[0]; r.a.y = w[1]; r.a.z = w[2]; r.a.w = w[3];
    }
    return r;
}

template <int DT>
__device__ __forceinline__ void decode(const Raw8<DT>& r, float (&x)[8]) {
    if constexpr (DT == RT_DT_F32) {
        x[0] = u2f(r.a.x); x[1] = u2f(r.a.y); x[2] = u2f(r.a.z); x[3] = u2f(r.a.w);
        x[4] = u2f(r.b.x); x[5] = u2f(r.b.y); x[6] = u2f(r.b.z); x[7] = u2f(r.b.w);
    } else {
        const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
        if constexpr (DT == RT_DT_BF16) {  // bf16 -> fp32 is the 16 bits moved to the high half
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                x[2 * k] = u2f(w[k] << 16);
                x[2 * k + 1] = u2f(w[k] & 0xFFFF0000u);
            }
        } else {  // IEEE half: v_cvt_f32_f16 is exact
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                x[2 * k] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[k] & 0xFFFFu));
                x[2 * k + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[k] >> 16));
            }
        }
    }
}

// Stochastic rounding to bf16: bits(x) + noise16, keep the high half
// (copy_stochastic_: int32 add, mask 0xFFFF0000).  Two results are packed per
// word with one byte permute (bytes 2,3 of each sum).
__device__ __forceinline__ u32x4 sr_pack(const float (&x)[8], u32x4 noise) {
    const uint32_t nz[4] = {noise.x, noise.y, noise.z, noise.w};
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t lo = f2u(x[2 * k]) + (nz[k] & 0xFFFFu);
        const uint32_t hi = f2u(x[2 * k + 1]) + (nz[k] >> 16);
        w[k] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
    }
    u32x4 r;
    r.x = w[0]; r.y = w[1]; r.z = w[2]; r.w = w[3];
    return r;
}

// fp32 -> IEEE half, round to nearest even (v_cvt_f16_f32: gradual underflow, overflow to infinity),
// which is what a plain copy_ into an fp16 tensor does; two results per word.
// The value converted must be the fp32 result as rounded: left to itself the compiler folds the
// conversion into the fused multiply-add that produced it (v_fma_mixlo_f16: one rounding, straight
// to fp16), which differs from round-to-fp32-then-to-fp16 in the last bit of ~0.5 % of the results.
// The empty asm makes the fp32 value opaque at no cost.
__device__ __forceinline__ uint32_t f16_bits(float x) {
    asm volatile("" : "+v"(x));
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
}
__device__ __forceinline__ uint32_t f16_pair(float lo, float hi) { return f16_bits(lo) | (f16_bits(hi) << 16); }
__device__ __forceinline__ u32x4 f16_pack(const float (&x)[8]) {
    u32x4 r;
    r.x = f16_pair(x[0], x[1]); r.y = f16_pair(x[2], x[3]); r.z = f16_pair(x[4], x[5]); r.w = f16_pair(x[6], x[7]);
    return r;
}

// Write-back of one array: bf16 targets are stochastically rounded, fp16 targets rounded to
// nearest, fp32 targets stored as they are.
template <int DT>
__device__ __forceinline__ void store_out(uint64_t base, uint64_t i, const float (&x)[8], u32x4 noise) {
    if constexpr (DT == RT_DT_BF16) {
        stg128(base + i * 2, sr_pack(x, noise));
    } else if constexpr (DT == RT_DT_F16) {
        stg128(base + i * 2, f16_pack(x));
    } else {
        u32x4 a, b;
        a.x = f2u(x[0]); a.y = f2u(x[1]); a.z = f2u(x[2]); a.w = f2u(x[3]);
        b.x = f2u(x[4]); b.y = f2u(x[5]); b.z = f2u(x[6]); b.w = f2u(x[7]);
        stg128(base + i * 4, a);
        stg128(base + i * 4 + 16, b);
    }
}

template <int DT>
__device__ __forceinline__ void store_out_guarded(uint64_t base, uint64_t i, uint64_t n, const float (&x)[8],
                                                  u32x4 noise) {
    if constexpr (DT == RT_DT_BF16 || DT == RT_DT_F16) {
        const u32x4 r = DT == RT_DT_BF16 ? sr_pack(x, noise) : f16_pack(x);
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (i + 2 * k < n) stg16(base + (i + 2 * k) * 2, w[k] & 0xFFFFu);
            if (i + 2 * k + 1 < n) stg16(base + (i + 2 * k + 1) * 2, w[k] >> 16);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (i + j < n) stg32f(base + (i + j) * 4, x[j]);
    }
}

// ---------------------------------------------------------------------------
// One element of the update in float32, in the rounding sequence of torch's
// GPU elementwise kernels:
//   m' = fma(1-b1, g, fl(m*b1))
//   v' = fma(1-b2, fl(g*g), fl(v*b2))
//   den = fl(fl(sqrt(v')) * fl(1/bcs)) + eps        (sqrt correctly rounded)
//   p1 = fl(p * decay)                              (decay == 1.0f when weight_decay == 0)
//   p' = fma(-step_size, fl(m'/den), p1)            (division correctly rounded)
// ---------------------------------------------------------------------------
__device__ __forceinline__ void update1(float& p, float g, float& m, float& v, const rt_scalars& s) {
    const float t = m * s.beta1;
    const float m1 = __builtin_fmaf(s.one_m_beta1, g, t);
    const float u = v * s.beta2;
    const float gg = g * g;
    const float v1 = __builtin_fmaf(s.one_m_beta2, gg, u);
    const float sq = __builtin_sqrtf(v1);
    const float d = sq * s.inv_bcs;
    const float den = d + s.eps;
    const float p1 = p * s.decay;  // decay is exactly 1.0f when weight_decay == 0 (x * 1.0f == x)
    const float q = m1 / den;
    p = __builtin_fmaf(s.neg_step_size, q, p1);
    m = m1;
    v = v1;
}

// Per-launch uniform state of the update kernel.
struct UpdateCtx {
    rt_scalars s;
    uint32_t step;
    uint32_t seed_lo, seed_hi;
    float coef;
    bool do_clip;
    bool do_unscale;
};

// Correctly rounded sqrt for x in [2^-96, +inf): the sequence the compiler emits for sqrtf (v_sqrt_f32,
// then the neighbours one ulp below and above are tried against the residuals x - s_down * s and
// x - s_up * s), without the part that exists only for smaller inputs (scaling by 2^32 before and by
// 2^-16 after, selecting x itself for zero and infinity).  Same instructions on the same values, so
// the same bits; 12 issue slots instead of 19.
__device__ __forceinline__ float sqrt_rn_from_2m96(float x) {
    const float s = __builtin_amdgcn_sqrtf(x);
    const float s_down = u2f(f2u(s) - 1u), s_up = u2f(f2u(s) + 1u);
    const float r_down = __builtin_fmaf(-s_down, s, x);
    const float r_up = __builtin_fmaf(-s_up, s, x);
    float r = r_down <= 0.0f ? s_down : s;
    r = r_up > 0.0f ? s_up : r;
    return r;
}

// N elements of one lane through update1's arithmetic.  The second moments of a whole wavefront
// almost always lie in [2^-96, inf) (they are sums of squares of gradients around 1e-3); then every
// lane takes the short sqrt above.  One zero, denormal, tiny, negative or non-finite value anywhere
// in the wavefront sends all of it through the compiler's full sequence instead.
template <int N>
__device__ __forceinline__ void update_n(float (&p)[N], const float (&g)[N], float (&m)[N], float (&v)[N],
                                         const rt_scalars& s) {
    uint32_t lo = 0xFFFFFFFFu, hi = 0u;
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const float t = m[j] * s.beta1;
        m[j] = __builtin_fmaf(s.one_m_beta1, g[j], t);
        const float u = v[j] * s.beta2;
        const float gg = g[j] * g[j];
        v[j] = __builtin_fmaf(s.one_m_beta2, gg, u);
        lo = min(lo, f2u(v[j]));
        hi = max(hi, f2u(v[j]));
    }
    const bool special = lo < 0x0F800000u /* 2^-96 */ || hi >= 0x7F800000u /* inf, nan, negative */;
    if (__builtin_amdgcn_ballot_w64(special) == 0ull) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const float d = sqrt_rn_from_2m96(v[j]) * s.inv_bcs;
            const float den = d + s.eps;
            const float p1 = p[j] * s.decay;
            const float q = m[j] / den;
            p[j] = __builtin_fmaf(s.neg_step_size, q, p1);
        }
    } else {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const float d = __builtin_sqrtf(v[j]) * s.inv_bcs;
            const float den = d + s.eps;
            const float p1 = p[j] * s.decay;
            const float q = m[j] / den;
            p[j] = __builtin_fmaf(s.neg_step_size, q, p1);
        }
    }
}

// Noise for the block of 8 elements starting at element i of tensor t.
template <int PDT, int MDT, int VDT>
__device__ __forceinline__ void philox_noise3(const DevTensor& t, const UpdateCtx& c, uint64_t i, u32x4& zp,
                                              u32x4& zm, u32x4& zv) {
    const uint64_t blk = t.block_base + (i >> 3);
    const uint32_t b0 = (uint32_t)blk, b1 = (uint32_t)(blk >> 32);
    if constexpr (PDT == RT_DT_BF16) zp = philox4x32_10(b0, b1, t.tensor_id4 + 0u, c.step, c.seed_lo, c.seed_hi);
    if constexpr (MDT == RT_DT_BF16) zm = philox4x32_10(b0, b1, t.tensor_id4 + 1u, c.step, c.seed_lo, c.seed_hi);
    if constexpr (VDT == RT_DT_BF16) zv = philox4x32_10(b0, b1, t.tensor_id4 + 2u, c.step, c.seed_lo, c.seed_hi);
}

__device__ __forceinline__ void scale_grads(float (&g)[8], const UpdateCtx& c) {
    if (c.do_unscale) {
#pragma unroll
        for (int j = 0; j < 8; ++j) g[j] = g[j] * c.s.inv_loss_scale;
    }
    if (c.do_clip) {
#pragma unroll
        for (int j = 0; j < 8; ++j) g[j] = g[j] * c.coef;
    }
}

// What centralization subtracts from every gradient element of a row (adamw.py:179-184:
// grad.sub_(mean.mul_(c)), the product rounded before it is subtracted).  `mean` is the row mean of
// the unscaled gradient; with a clip coefficient the gradient has been multiplied by it, and so is
// its mean (clipping first and centralizing afterwards is what clip_grad_norm_ followed by step() does).
__device__ __forceinline__ float cen_term(float mean, const rt_scalars& s, bool do_clip, float coef) {
    if (do_clip) mean = mean * coef;
    return mean * s.centralization;
}

// ---------------------------------------------------------------------------
// Launch-uniform set-up shared by the update kernels.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void make_ctx(const LaunchArgs& a, uint32_t set_idx, UpdateCtx& c) {
    if (a.use_ks != 0u) {  // the usual case: one param group at one step count; no table read
        c.s = a.ks.s;
        c.step = a.ks.step;
    } else {
        const DevScalars set = load_const(&a.sets[set_idx]);
        c.s = set.s;
        c.step = set.step;
    }
    c.seed_lo = a.seed_lo;
    c.seed_hi = a.seed_hi;
    c.do_clip = a.clip_coef != nullptr;
    c.coef = c.do_clip ? load_const(a.clip_coef) : 1.0f;
    c.do_unscale = c.s.inv_loss_scale != 1.0f;
}

// Index of the last entry of the ascending list `first` (first[0] == 0) that is <= unit.  Each
// wavefront searches on its own, 64 ways at a time: lane l looks at every stride-th entry, a ballot
// counts the lanes whose entry is <= unit.  One dependent load for up to 64 tensors, two for up
// to 4096 -- a scalar binary search would chain one load per halving in front of every
// workgroup's first vector load.  (Loading up to eight entries per lane at once, one latency for up
// to 512 tensors, measured no faster on the 8B set's 226 ranges.)
__device__ __forceinline__ uint32_t find_range(const uint32_t* __restrict__ first, uint32_t n, uint32_t unit) {
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t lo = 0, len = n;
    while (len > 64u) {
        const uint32_t stride = (len + 63u) >> 6;
        const uint32_t k = lane * stride;
        const bool le = k < len && first[lo + k] <= unit;
        const uint32_t c = (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(le));  // >= 1: first[lo] <= unit
        lo += (c - 1u) * stride;
        len = min(stride, len - (c - 1u) * stride);
    }
    const bool le = lane < len && first[lo + lane] <= unit;
    return lo + (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(le)) - 1u;
}

// ---------------------------------------------------------------------------
// Piece: at most 512 consecutive elements handled by one wavefront, one 128-bit
// vector per lane (the last lane with elements may hold fewer than 8 and then
// moves them one by one).  Short tensors and the leftovers of long ones.
// ---------------------------------------------------------------------------
template <int PDT, int GDT, int MDT, int VDT>
__device__ __forceinline__ void piece_body(const LaunchArgs& a, uint32_t q) {
    // (the piece records stream through: read with vector loads they stay out of the small scalar
    // cache that the unit workgroups' tables live in -- 2.7 % faster on the 20 064-tensor set)
    const PieceRef& r = a.pieces[q];
    const uint64_t rp = r.p, rg = r.g, rm = r.m, rv = r.v;
    const uint32_t count = r.count;
    const uint64_t i = (uint64_t)(threadIdx.x & 63u) * kVec;
    if (i >= count) return;
    const bool full = i + kVec <= count;
    Raw8<PDT> xp; Raw8<GDT> xg; Raw8<MDT> xm; Raw8<VDT> xv;
    if (full) {
        xp = load_raw<PDT>(rp, i); xg = load_raw<GDT>(rg, i);
        xm = load_raw<MDT>(rm, i); xv = load_raw<VDT>(rv, i);
    } else {
        xp = load_raw_guarded<PDT>(rp, i, count); xg = load_raw_guarded<GDT>(rg, i, count);
        xm = load_raw_guarded<MDT>(rm, i, count); xv = load_raw_guarded<VDT>(rv, i, count);
    }
    UpdateCtx c;
    make_ctx(a, r.set_idx, c);
    const uint64_t blk = r.block + (i >> 3);
    const uint32_t b0 = (uint32_t)blk, b1 = (uint32_t)(blk >> 32);
    u32x4 zp = 0, zm = 0, zv = 0;
    if constexpr (PDT == RT_DT_BF16) zp = philox4x32_10(b0, b1, r.tensor_id4 + 0u, c.step, c.seed_lo, c.seed_hi);
    if constexpr (MDT == RT_DT_BF16) zm = philox4x32_10(b0, b1, r.tensor_id4 + 1u, c.step, c.seed_lo, c.seed_hi);
    if constexpr (VDT == RT_DT_BF16) zv = philox4x32_10(b0, b1, r.tensor_id4 + 2u, c.step, c.seed_lo, c.seed_hi);
    float p[8], g[8], m[8], v[8];
    decode<PDT>(xp, p); decode<GDT>(xg, g); decode<MDT>(xm, m); decode<VDT>(xv, v);
    scale_grads(g, c);
    update_n<8>(p, g, m, v, c.s);
    if (full) {
        store_out<PDT>(rp, i, p, zp);
        store_out<MDT>(rm, i, m, zm);
        store_out<VDT>(rv, i, v, zv);
    } else {
        store_out_guarded<PDT>(rp, i, count, p, zp);
        store_out_guarded<MDT>(rm, i, count, m, zm);
        store_out_guarded<VDT>(rv, i, count, v, zv);
    }
}

// ---------------------------------------------------------------------------
// Fast kernel, all arrays 16 bit wide.  One launch covers everything that needs
// no special care in 16-byte aligned tensors:
//  * n_piece_wgs workgroups serve four pieces each, one per wavefront (Philox
//    mode only);
//  * the other workgroups serve one unit of kFastUnitElems elements each, lying
//    wholly inside one tensor.  Every access is a 128-bit global load or store;
//    all loads of the unit are issued before the math of its first vector so that
//    memory latency hides behind the VALU work (Philox, sqrt, division).
// Everything is inlined and lives in registers: a stack frame here would turn
// into scratch-memory traffic on every workgroup.
// ---------------------------------------------------------------------------
// CEN: the tensors of the launch have their gradients centralized (adamw.py:179-184): fl(mean(row) * c)
// is subtracted from every gradient element before the update.  Rows are at least 8 elements long
// (shorter ones take the generic kernel), so a lane's 8 elements lie in at most two rows.
template <int PDT, int GDT, int MDT, int VDT, int NOISE, bool CEN = false>
__global__ __launch_bounds__(kThreads) void sr_adamw_fast_kernel(const LaunchArgs a) {
    if (a.skip != nullptr && load_const(a.skip) != 0u) return;
    // Piece workgroups are spread evenly among the unit workgroups: of the first b workgroups,
    // min(n_piece_wgs, floor(b * piece_rate / 2^32)) serve pieces (piece_rate = ceil(n_piece_wgs * 2^32 /
    // gridDim.x), or 0 when the launch has only pieces).  Pieces are bound by instruction issue and by
    // the latency of their short dependent chains, units by memory: resident side by side they overlap.
    const uint32_t b = blockIdx.x;
    uint32_t pieces_before = b, pieces_after = b + 1u;
    if (a.piece_rate != 0u) {
        pieces_before = min(a.n_piece_wgs, __umulhi(b, a.piece_rate));
        pieces_after = min(a.n_piece_wgs, __umulhi(b + 1u, a.piece_rate));
    } else if (a.n_piece_wgs == 0u) {
        pieces_before = pieces_after = 0u;
    }
    if (pieces_after != pieces_before) {
        if constexpr (NOISE == RT_NOISE_PHILOX) {
            const uint32_t q = (uint32_t)__builtin_amdgcn_readfirstlane((int)(pieces_before * 4u + (threadIdx.x >> 6)));
            if (q < a.n_pieces) piece_body<PDT, GDT, MDT, VDT>(a, q);
        }
        return;
    }
    const uint32_t unit = b - pieces_before;
    const uint32_t ri = find_range(a.first, a.n_ranges, unit);
    const DevTensor t = load_const(&a.fast_tensors[ri]);
    const uint32_t unit_in_tensor = unit - load_const(&a.first[ri]);
    UpdateCtx c;
    make_ctx(a, t.set_idx, c);
    const uint64_t tp = t.p, tg = t.g, tm = t.m, tv = t.v, tnp = t.np, tnm = t.nm, tnv = t.nv;

    struct In {
        Raw8<PDT> p;
        Raw8<GDT> g;
        Raw8<MDT> m;
        Raw8<VDT> v;
        u32x4 zp, zm, zv;
        float mean0, mean1;  // CEN: means of the row of the first element and of the row after it
        uint32_t rem;        // CEN: position of the first element inside its row
    };
    const uint32_t row_len = (uint32_t)t.row_len;  // CEN launches: 8 <= row_len < 2^31
    auto fetch = [&](uint64_t i, uint64_t row, uint32_t rem) {
        In r;
        r.p = load_raw<PDT>(tp, i);
        r.g = load_raw<GDT>(tg, i);
        r.m = load_raw<MDT>(tm, i);
        r.v = load_raw<VDT>(tv, i);
        if constexpr (NOISE == RT_NOISE_EXPLICIT) {
            if constexpr (PDT == RT_DT_BF16) r.zp = ldg128(tnp + i * 2);
            if constexpr (MDT == RT_DT_BF16) r.zm = ldg128(tnm + i * 2);
            if constexpr (VDT == RT_DT_BF16) r.zv = ldg128(tnv + i * 2);
        }
        if constexpr (CEN) {
            r.rem = rem;
            r.mean0 = ldg32f(t.row_mean + row * 4);
            r.mean1 = rem + (kVec - 1) >= row_len ? ldg32f(t.row_mean + row * 4 + 4) : 0.0f;
        }
        return r;
    };
    // A wave walks its own contiguous quarter of the unit (4 x 1 KB per array)
    // instead of interleaving with the other waves kilobyte by kilobyte: measured 2.5 % faster on the
    // 8B set.  (Longer runs, 2 or 8 KB, and other workgroup sizes were not faster.)
    constexpr uint64_t kStep = 64 * kVec;
    const uint64_t i0 = (uint64_t)unit_in_tensor * kFastUnitElems +
                        (uint64_t)(threadIdx.x >> 6) * (kStep * kFastIters) + (uint64_t)(threadIdx.x & 63u) * kVec;
    // CEN: one 64-bit division finds the row of the lane's first element; from vector to vector the
    // position advances by kStep elements, which a 32-bit division turns into rows.
    uint64_t row = 0;
    uint32_t rem = 0;
    if constexpr (CEN) {
        const uint64_t e0 = (t.block_base << 3) + i0;
        row = e0 / row_len;
        rem = (uint32_t)(e0 - row * row_len);
    }
    // Every load of the unit is issued before the first result is needed (kFastIters vectors per array
    // and lane in flight): the memory system sees one burst of reads per workgroup and the stores of
    // a vector leave as its arithmetic finishes (holding them back to the end of the unit costs 60
    // registers and 0.4 %; storing two vectors' results together changes nothing).  Against keeping one vector ahead this measured
    // 0.3 - 0.4 % faster on the 8B set, 5 % on a single 4096 x 4096 tensor and on the set of 20 064
    // small tensors, at 99 vector registers instead of 68 (explicit-noise instance: 159, and still 2 %
    // faster on the single tensor than with one or two vectors ahead).
    In q[kFastIters];
    auto advance = [&]() {
        if constexpr (CEN) {
            const uint32_t ahead = rem + (uint32_t)kStep;  // < 2^31 + 512
            const uint32_t d = ahead / row_len;
            row += d;
            rem = ahead - d * row_len;
        }
    };
#pragma unroll
    for (int k = 0; k < kFastIters; ++k) {
        if (k) advance();
        q[k] = fetch(i0 + (uint64_t)k * kStep, row, rem);
    }
#pragma unroll
    for (int it = 0; it < kFastIters; ++it) {
        const uint64_t i = i0 + (uint64_t)it * kStep;
        const In& cur = q[it];

        float p[8], g[8], m[8], v[8];
        decode<PDT>(cur.p, p);
        decode<GDT>(cur.g, g);
        decode<MDT>(cur.m, m);
        decode<VDT>(cur.v, v);
        u32x4 zp = cur.zp, zm = cur.zm, zv = cur.zv;
        if constexpr (NOISE == RT_NOISE_PHILOX) philox_noise3<PDT, MDT, VDT>(t, c, i, zp, zm, zv);
        scale_grads(g, c);
        if constexpr (CEN) {
            // grad.sub_(mean.mul_(c)): the product is rounded, then subtracted
            const float mc0 = cen_term(cur.mean0, c.s, c.do_clip, c.coef), mc1 = cen_term(cur.mean1, c.s, c.do_clip, c.coef);
#pragma unroll
            for (int j = 0; j < 8; ++j) g[j] = g[j] - (cur.rem + (uint32_t)j < row_len ? mc0 : mc1);
        }
        update_n<8>(p, g, m, v, c.s);
        store_out<PDT>(tp, i, p, zp);
        store_out<MDT>(tm, i, m, zm);
        store_out<VDT>(tv, i, v, zv);
    }
}

// ---------------------------------------------------------------------------
// Fast kernel for dtype combinations with an fp32 array.  With 8 consecutive
// elements per lane an fp32 array would be read as two 16-byte accesses 16
// bytes apart, i.e. every instruction would touch only half of each cache line
// it requests; a math-free probe of the bf16 p,m / fp32 g,v layout ran 10 %
// slower that way.  Here a lane owns 4 + 4 elements instead: elements
// [4l, 4l+4) of the first and of the second half of its wave's 512-element
// block, so that every instruction covers one contiguous kilobyte (fp32) or
// half kilobyte (16-bit types) across the wave.
//
// Rounding noise keeps its definition (element e takes 16-bit field e & 7 of
// the Philox block e >> 3): lanes 2j and 2j+1 share block j of the first half
// and block 32+j of the second; the even lane computes the former, the odd
// lane the latter, and they trade the 64 bits the other one needs with one
// neighbour swap (DPP quad_perm), so the Philox count per element is unchanged.
// ---------------------------------------------------------------------------
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x2 ldg64(uint64_t addr) {
    return __builtin_nontemporal_load((const RT_GLOBAL u32x2*)addr);
}
__device__ __forceinline__ void stg64(uint64_t addr, u32x2 v) {
    __builtin_nontemporal_store(v, (RT_GLOBAL u32x2*)addr);
}
__device__ __forceinline__ uint32_t swap_neighbour(uint32_t x) {  // value of lane ^ 1
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, false);
}

// Four elements: one 128-bit word for fp32, 64 bits (x, y) for 16-bit types.
template <int DT>
__device__ __forceinline__ u32x4 load_raw4(uint64_t base, uint64_t e) {
    if constexpr (DT == RT_DT_F32) {
        return ldg128(base + e * 4);
    } else {
        const u32x2 t = ldg64(base + e * 2);
        u32x4 r;
        r.x = t.x; r.y = t.y; r.z = 0; r.w = 0;
        return r;
    }
}

template <int DT>
__device__ __forceinline__ void decode4(const u32x4& r, float (&x)[4]) {
    if constexpr (DT == RT_DT_F32) {
        x[0] = u2f(r.x); x[1] = u2f(r.y); x[2] = u2f(r.z); x[3] = u2f(r.w);
    } else if constexpr (DT == RT_DT_BF16) {
        x[0] = u2f(r.x << 16); x[1] = u2f(r.x & 0xFFFF0000u);
        x[2] = u2f(r.y << 16); x[3] = u2f(r.y & 0xFFFF0000u);
    } else {
        x[0] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.x & 0xFFFFu));
        x[1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.x >> 16));
        x[2] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.y & 0xFFFFu));
        x[3] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.y >> 16));
    }
}

// noise: four 16-bit fields in (x, y), element order low half first
template <int DT>
__device__ __forceinline__ void store_out4(uint64_t base, uint64_t e, const float (&x)[4], u32x2 noise) {
    if constexpr (DT == RT_DT_BF16) {
        u32x2 w;
        w.x = __builtin_amdgcn_perm(f2u(x[1]) + (noise.x >> 16), f2u(x[0]) + (noise.x & 0xFFFFu), 0x07060302u);
        w.y = __builtin_amdgcn_perm(f2u(x[3]) + (noise.y >> 16), f2u(x[2]) + (noise.y & 0xFFFFu), 0x07060302u);
        stg64(base + e * 2, w);
    } else if constexpr (DT == RT_DT_F16) {
        u32x2 w;
        w.x = f16_pair(x[0], x[1]);
        w.y = f16_pair(x[2], x[3]);
        stg64(base + e * 2, w);
    } else {
        u32x4 a;
        a.x = f2u(x[0]); a.y = f2u(x[1]); a.z = f2u(x[2]); a.w = f2u(x[3]);
        stg128(base + e * 4, a);
    }
}

template <int PDT, int GDT, int MDT, int VDT, int NOISE>
__global__ __launch_bounds__(kThreads) void sr_adamw_fast_wide_kernel(const LaunchArgs a) {
    if (a.skip != nullptr && load_const(a.skip) != 0u) return;
    const uint32_t unit = blockIdx.x;
    const uint32_t ri = find_range(a.first, a.n_ranges, unit);
    const DevTensor t = load_const(&a.fast_tensors[ri]);
    const uint32_t unit_in_tensor = unit - load_const(&a.first[ri]);
    UpdateCtx c;
    make_ctx(a, t.set_idx, c);
    const uint64_t tp = t.p, tg = t.g, tm = t.m, tv = t.v, tnp = t.np, tnm = t.nm, tnv = t.nv;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const bool odd = (lane & 1u) != 0u;
    constexpr uint32_t kWaveElems = 64 * kVec;       // 512 elements per wave per iteration
    constexpr uint32_t kHalf = kWaveElems / 2;       // second half starts 256 elements later

    struct In {
        u32x4 p[2], g[2], m[2], v[2];  // [half]
        u32x2 zp[2], zm[2], zv[2];     // explicit noise
    };
    auto fetch = [&](uint64_t blk) {   // blk: first element of this wave's 512-element block
        In r;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint64_t e = blk + (uint64_t)h * kHalf + lane * 4u;
            r.p[h] = load_raw4<PDT>(tp, e);
            r.g[h] = load_raw4<GDT>(tg, e);
            r.m[h] = load_raw4<MDT>(tm, e);
            r.v[h] = load_raw4<VDT>(tv, e);
            if constexpr (NOISE == RT_NOISE_EXPLICIT) {
                if constexpr (PDT == RT_DT_BF16) r.zp[h] = ldg64(tnp + e * 2);
                if constexpr (MDT == RT_DT_BF16) r.zm[h] = ldg64(tnm + e * 2);
                if constexpr (VDT == RT_DT_BF16) r.zv[h] = ldg64(tnv + e * 2);
            }
        }
        return r;
    };
    // Philox noise of this lane's two half blocks for one array (`which` = 0 p, 1 m, 2 v).
    auto philox_halves = [&](uint64_t blk, uint32_t which, u32x2 (&z)[2]) {
        const uint64_t first = t.block_base + (blk >> 3) + (lane >> 1);  // block of the first-half elements
        const uint64_t mine = odd ? first + (kHalf >> 3) : first;
        const u32x4 r = philox4x32_10((uint32_t)mine, (uint32_t)(mine >> 32), t.tensor_id4 + which, c.step,
                                      c.seed_lo, c.seed_hi);
        // even lanes hand over the high 64 bits of the first-half block, odd lanes the low 64 bits of the second
        const uint32_t g0 = swap_neighbour(odd ? r.x : r.z);
        const uint32_t g1 = swap_neighbour(odd ? r.y : r.w);
        z[0].x = odd ? g0 : r.x; z[0].y = odd ? g1 : r.y;
        z[1].x = odd ? r.z : g0; z[1].y = odd ? r.w : g1;
    };

    // (here the waves interleave kilobyte blocks; giving each wave its own contiguous quarter of
    // the chunk, as the all-16-bit kernel does, measured 8 % slower for this layout)
    const uint64_t blk0 = (uint64_t)unit_in_tensor * kFastUnitElems + (uint64_t)wave * kWaveElems;
    // all loads of the unit first, as in the all-16-bit kernel (0.3 - 0.5 % faster on the 8B set)
    In q[kFastIters];
#pragma unroll
    for (int k = 0; k < kFastIters; ++k) q[k] = fetch(blk0 + (uint64_t)k * (kThreads * kVec));
#pragma unroll
    for (int it = 0; it < kFastIters; ++it) {
        const uint64_t blk = blk0 + (uint64_t)it * (kThreads * kVec);
        const In& cur = q[it];

        u32x2 zp[2] = {cur.zp[0], cur.zp[1]}, zm[2] = {cur.zm[0], cur.zm[1]}, zv[2] = {cur.zv[0], cur.zv[1]};
        if constexpr (NOISE == RT_NOISE_PHILOX) {
            if constexpr (PDT == RT_DT_BF16) philox_halves(blk, 0u, zp);
            if constexpr (MDT == RT_DT_BF16) philox_halves(blk, 1u, zm);
            if constexpr (VDT == RT_DT_BF16) philox_halves(blk, 2u, zv);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float p[4], g[4], m[4], v[4];
            decode4<PDT>(cur.p[h], p);
            decode4<GDT>(cur.g[h], g);
            decode4<MDT>(cur.m[h], m);
            decode4<VDT>(cur.v[h], v);
            if (c.do_unscale) {
#pragma unroll
                for (int j = 0; j < 4; ++j) g[j] = g[j] * c.s.inv_loss_scale;
            }
            if (c.do_clip) {
#pragma unroll
                for (int j = 0; j < 4; ++j) g[j] = g[j] * c.coef;
            }
            update_n<4>(p, g, m, v, c.s);
            const uint64_t e = blk + (uint64_t)h * kHalf + lane * 4u;
            store_out4<PDT>(tp, e, p, zp[h]);
            store_out4<MDT>(tm, e, m, zm[h]);
            store_out4<VDT>(tv, e, v, zv[h]);
        }
    }
}

// ---------------------------------------------------------------------------
// Generic kernel: the last (partial) chunk of a tensor, tensors whose pointers
// are not 16-byte aligned, debug outputs, gradient centralization.  Full
// aligned vectors still move as 128-bit accesses; everything else element by
// element under an index guard.
// ---------------------------------------------------------------------------
template <int PDT, int GDT, int MDT, int VDT, int NOISE>
__global__ __launch_bounds__(kThreads) void sr_adamw_generic_kernel(const LaunchArgs a) {
    if (a.skip != nullptr && load_const(a.skip) != 0u) return;
    const ChunkRef cr = load_const(&a.chunks[blockIdx.x]);
    const DevTensor t = load_const(&a.tensors[cr.tensor]);
    UpdateCtx c;
    make_ctx(a, t.set_idx, c);

    const uint64_t n = t.numel;
    const uint64_t chunk_base = (uint64_t)cr.chunk * kChunkElems;
    const bool aligned = (t.flags & kFlagAligned) != 0u;
#pragma unroll 1
    for (int it = 0; it < kItersPerChunk; ++it) {
        const uint64_t i = chunk_base + (uint64_t)(it * kThreads + (int)threadIdx.x) * kVec;
        if (i >= n) break;
        const bool full = aligned && (i + kVec <= n);
        Raw8<PDT> rp; Raw8<GDT> rg; Raw8<MDT> rm; Raw8<VDT> rv;
        u32x4 zp = 0, zm = 0, zv = 0;
        if (full) {
            rp = load_raw<PDT>(t.p, i); rg = load_raw<GDT>(t.g, i);
            rm = load_raw<MDT>(t.m, i); rv = load_raw<VDT>(t.v, i);
        } else {
            rp = load_raw_guarded<PDT>(t.p, i, n); rg = load_raw_guarded<GDT>(t.g, i, n);
            rm = load_raw_guarded<MDT>(t.m, i, n); rv = load_raw_guarded<VDT>(t.v, i, n);
        }
        if constexpr (NOISE == RT_NOISE_EXPLICIT) {
            if constexpr (PDT == RT_DT_BF16)
                zp = full ? ldg128(t.np + i * 2) : load_raw_guarded<RT_DT_BF16>(t.np, i, n).a;
            if constexpr (MDT == RT_DT_BF16)
                zm = full ? ldg128(t.nm + i * 2) : load_raw_guarded<RT_DT_BF16>(t.nm, i, n).a;
            if constexpr (VDT == RT_DT_BF16)
                zv = full ? ldg128(t.nv + i * 2) : load_raw_guarded<RT_DT_BF16>(t.nv, i, n).a;
        } else {
            philox_noise3<PDT, MDT, VDT>(t, c, i, zp, zm, zv);
        }
        float p[8], g[8], m[8], v[8];
        decode<PDT>(rp, p); decode<GDT>(rg, g); decode<MDT>(rm, m); decode<VDT>(rv, v);
        scale_grads(g, c);
        if (t.row_mean != 0) {
            // grad.sub_(mean.mul_(c)): the product is rounded, then subtracted.
            // One division finds the row of the first element; the rest follow by counting.
            const uint64_t e0 = (t.block_base << 3) + i;
            uint64_t row = e0 / t.row_len;
            uint64_t rem = e0 - row * t.row_len;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (i + j < n) {
                    const float mc = cen_term(ldg32f(t.row_mean + row * 4), c.s, c.do_clip, c.coef);
                    g[j] = g[j] - mc;
                }
                if (++rem == t.row_len) {
                    rem = 0;
                    ++row;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) update1(p[j], g[j], m[j], v[j], c.s);

        if (t.dp != 0) store_out_guarded<RT_DT_F32>(t.dp, i, n, p, zp);
        if (t.dm != 0) store_out_guarded<RT_DT_F32>(t.dm, i, n, m, zm);
        if (t.dv != 0) store_out_guarded<RT_DT_F32>(t.dv, i, n, v, zv);
        if (full) {
            store_out<PDT>(t.p, i, p, zp);
            store_out<MDT>(t.m, i, m, zm);
            store_out<VDT>(t.v, i, v, zv);
        } else {
            store_out_guarded<PDT>(t.p, i, n, p, zp);
            store_out_guarded<MDT>(t.m, i, n, m, zm);
            store_out_guarded<VDT>(t.v, i, n, v, zv);
        }
    }
}

// ---------------------------------------------------------------------------
// Runtime-typed kernel: tensors with an fp64 array, or with one fp16 state next
// to a state of another dtype (the templated kernels cover fp16 params and a
// pair of fp16 states).
// The reference upcasts every dtype to fp32 (adamw.py:160-170) and writes
// anything that is not bf16 back with a plain copy_ (adamw.py:208,214,221-222):
// fp16 is rounded to nearest even (v_cvt_f16_f32), fp64 widened exactly; an
// fp64 input is rounded to nearest even on the way in.  Such layouts are rare,
// so this is one kernel with a per-tensor dtype switch instead of another 200
// instantiations: a lane owns one Philox block of 8 elements, as in the
// kernels above, and moves them as 128-bit accesses where the tensor is plain
// and aligned, element by element otherwise.  The four accesses a lane makes
// to an fp64 array are ordinary cached ones: with the nontemporal hint every
// one of them fetched its 128-byte line from the L2 again (1.5 TB/s instead of
// 4.9 TB/s for an all-fp64 layout).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float load_any(uint64_t base, uint32_t dt, uint64_t idx) {
    switch (dt) {
        case RT_DT_BF16: return u2f(ldg16(base + idx * 2) << 16);
        case RT_DT_F16: return (float)__builtin_bit_cast(_Float16, (uint16_t)ldg16(base + idx * 2));
        case RT_DT_F64: return (float)*(const RT_GLOBAL double*)(base + idx * 8);
        default: return ldg32f(base + idx * 4);
    }
}

__device__ __forceinline__ void store_any(uint64_t base, uint32_t dt, uint64_t idx, float x, uint32_t noise16) {
    switch (dt) {
        case RT_DT_BF16: stg16(base + idx * 2, (f2u(x) + noise16) >> 16); break;
        case RT_DT_F16: stg16(base + idx * 2, f16_bits(x)); break;
        case RT_DT_F64: *(RT_GLOBAL double*)(base + idx * 8) = (double)x; break;
        default: stg32f(base + idx * 4, x); break;
    }
}

__device__ __forceinline__ uint32_t noise_field(const u32x4& z, int j) {
    const uint32_t w = (j >> 1) == 0 ? z.x : (j >> 1) == 1 ? z.y : (j >> 1) == 2 ? z.z : z.w;
    return (j & 1) ? (w >> 16) : (w & 0xFFFFu);
}

// Eight consecutive elements of a 16-byte-aligned array as fp32, by 128-bit accesses, with the
// dtype known only at run time (it is the same for the whole wave, so the switch is a scalar
// branch).  fp64 takes four accesses of two doubles each; the conversions are the ones load_any /
// store_any make element by element.
__device__ __forceinline__ void load8_any(uint64_t base, uint32_t dt, uint64_t i, float (&x)[8]) {
    switch (dt) {
        case RT_DT_BF16: decode<RT_DT_BF16>(load_raw<RT_DT_BF16>(base, i), x); break;
        case RT_DT_F16: decode<RT_DT_F16>(load_raw<RT_DT_F16>(base, i), x); break;
        case RT_DT_F64:
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                // ordinary (cached) accesses: a lane's four accesses fall into one 64-byte half line
                const u32x4 w = *(const RT_GLOBAL u32x4*)(base + i * 8 + (uint64_t)k * 16);
                x[2 * k] = (float)__builtin_bit_cast(double, (uint64_t)w.x | ((uint64_t)w.y << 32));
                x[2 * k + 1] = (float)__builtin_bit_cast(double, (uint64_t)w.z | ((uint64_t)w.w << 32));
            }
            break;
        default: decode<RT_DT_F32>(load_raw<RT_DT_F32>(base, i), x); break;
    }
}

__device__ __forceinline__ void store8_any(uint64_t base, uint32_t dt, uint64_t i, const float (&x)[8], u32x4 noise) {
    switch (dt) {
        case RT_DT_BF16: store_out<RT_DT_BF16>(base, i, x, noise); break;
        case RT_DT_F16: store_out<RT_DT_F16>(base, i, x, noise); break;
        case RT_DT_F64:
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint64_t lo = __builtin_bit_cast(uint64_t, (double)x[2 * k]);
                const uint64_t hi = __builtin_bit_cast(uint64_t, (double)x[2 * k + 1]);
                u32x4 w;
                w.x = (uint32_t)lo; w.y = (uint32_t)(lo >> 32); w.z = (uint32_t)hi; w.w = (uint32_t)(hi >> 32);
                *(RT_GLOBAL u32x4*)(base + i * 8 + (uint64_t)k * 16) = w;
            }
            break;
        default: store_out<RT_DT_F32>(base, i, x, noise); break;
    }
}

// The same for a whole wavefront at once, for the two wide dtypes: the wave's 512 consecutive
// elements start at element w0 of a 16-byte-aligned array, and every instruction moves one contiguous
// kilobyte (lane l takes the 16 bytes at l * 16 of the k-th kilobyte) instead of 16 bytes out of
// every 32 (fp32) or 64 (fp64) per lane.  The values change hands through `stage`, 512 floats of
// shared memory that belong to this wave alone: written in array order, read back as each lane's own
// eight consecutive elements.  A wave's shared-memory instructions execute in the order issued, so
// no barrier is needed; the fences only keep the compiler from moving them across each other.
// fp64 state layouts ran at 4.4 TB/s with per-lane accesses.  (Issuing the loads of all four arrays
// before the first of them is unpacked, each array with a stage of its own, needs 153 registers --
// three waves per SIMD instead of four -- and ran 1 - 10 % slower on every layout; fetching the next
// 512 elements ahead of the arithmetic as well needs 255.)
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ void load8_wave_wide(uint64_t base, uint32_t dt, uint64_t w0, uint32_t lane,
                                                float* stage, float (&x)[8]) {
    wave_lds_fence();  // whatever read the stage before is done with it
    if (dt == RT_DT_F64) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const u32x4 w = ldg128(base + w0 * 8 + (uint64_t)(k * 64 + (int)lane) * 16);
            float2 f;
            f.x = (float)__builtin_bit_cast(double, (uint64_t)w.x | ((uint64_t)w.y << 32));
            f.y = (float)__builtin_bit_cast(double, (uint64_t)w.z | ((uint64_t)w.w << 32));
            *(float2*)(stage + (k * 64 + (int)lane) * 2) = f;
        }
    } else {  // fp32
#pragma unroll
        for (int k = 0; k < 2; ++k)
            *(u32x4*)(stage + (k * 64 + (int)lane) * 4) = ldg128(base + w0 * 4 + (uint64_t)(k * 64 + (int)lane) * 16);
    }
    wave_lds_fence();
    const u32x4 lo = *(const u32x4*)(stage + lane * 8), hi = *(const u32x4*)(stage + lane * 8 + 4);
    x[0] = u2f(lo.x); x[1] = u2f(lo.y); x[2] = u2f(lo.z); x[3] = u2f(lo.w);
    x[4] = u2f(hi.x); x[5] = u2f(hi.y); x[6] = u2f(hi.z); x[7] = u2f(hi.w);
}

__device__ __forceinline__ void store8_wave_wide(uint64_t base, uint32_t dt, uint64_t w0, uint32_t lane,
                                                 float* stage, const float (&x)[8]) {
    wave_lds_fence();
    u32x4 lo, hi;
    lo.x = f2u(x[0]); lo.y = f2u(x[1]); lo.z = f2u(x[2]); lo.w = f2u(x[3]);
    hi.x = f2u(x[4]); hi.y = f2u(x[5]); hi.z = f2u(x[6]); hi.w = f2u(x[7]);
    *(u32x4*)(stage + lane * 8) = lo;
    *(u32x4*)(stage + lane * 8 + 4) = hi;
    wave_lds_fence();
    if (dt == RT_DT_F64) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float2 f = *(const float2*)(stage + (k * 64 + (int)lane) * 2);
            const uint64_t a = __builtin_bit_cast(uint64_t, (double)f.x), b = __builtin_bit_cast(uint64_t, (double)f.y);
            u32x4 w;
            w.x = (uint32_t)a; w.y = (uint32_t)(a >> 32); w.z = (uint32_t)b; w.w = (uint32_t)(b >> 32);
            stg128(base + w0 * 8 + (uint64_t)(k * 64 + (int)lane) * 16, w);
        }
    } else {
#pragma unroll
        for (int k = 0; k < 2; ++k)
            stg128(base + w0 * 4 + (uint64_t)(k * 64 + (int)lane) * 16, *(const u32x4*)(stage + (k * 64 + (int)lane) * 4));
    }
}

template <int NOISE>
__global__ __launch_bounds__(kThreads) void sr_adamw_any_kernel(const LaunchArgs a) {
    if (a.skip != nullptr && load_const(a.skip) != 0u) return;
    const ChunkRef cr = load_const(&a.chunks[blockIdx.x]);
    const DevTensor t = load_const(&a.tensors[cr.tensor]);
    UpdateCtx c;
    make_ctx(a, t.set_idx, c);
    const rt_scalars s = c.s;
    const bool do_clip = c.do_clip;
    const float coef = c.coef;
    const bool do_unscale = c.do_unscale;
    const uint32_t seed_lo = a.seed_lo, seed_hi = a.seed_hi;
    const uint32_t pdt = t.dtypes & 3u, gdt = (t.dtypes >> 2) & 3u, mdt = (t.dtypes >> 4) & 3u,
                   vdt = (t.dtypes >> 6) & 3u;
    const uint64_t n = t.numel;
    const uint64_t chunk_base = (uint64_t)cr.chunk * kChunkElems;
    const bool plain = (t.flags & kFlagAligned) != 0u && (t.dp | t.dm | t.dv | t.row_mean) == 0;
    __shared__ __attribute__((aligned(16))) float stage_all[kThreads / 64][64 * kVec];
#pragma unroll 1
    for (int it = 0; it < kItersPerChunk; ++it) {
        const uint64_t i = chunk_base + (uint64_t)(it * kThreads + (int)threadIdx.x) * kVec;
        if (i >= n) break;
        u32x4 zp = 0, zm = 0, zv = 0;
        if constexpr (NOISE == RT_NOISE_PHILOX) {
            const uint64_t blk = t.block_base + (i >> 3);
            const uint32_t b0 = (uint32_t)blk, b1 = (uint32_t)(blk >> 32);
            if (pdt == RT_DT_BF16) zp = philox4x32_10(b0, b1, t.tensor_id4 + 0u, c.step, seed_lo, seed_hi);
            if (mdt == RT_DT_BF16) zm = philox4x32_10(b0, b1, t.tensor_id4 + 1u, c.step, seed_lo, seed_hi);
            if (vdt == RT_DT_BF16) zv = philox4x32_10(b0, b1, t.tensor_id4 + 2u, c.step, seed_lo, seed_hi);
        }
        // A wavefront whose 512 elements all exist moves its fp32 and fp64 arrays kilobyte by kilobyte.
        const uint64_t w0 = chunk_base + (uint64_t)(it * kThreads + (int)(threadIdx.x & ~63u)) * kVec;
        if (plain && w0 + 64 * kVec <= n) {
            const uint32_t lane = threadIdx.x & 63u;
            float* stage = stage_all[threadIdx.x >> 6];
            if constexpr (NOISE == RT_NOISE_EXPLICIT) {
                if (pdt == RT_DT_BF16) zp = ldg128(t.np + i * 2);
                if (mdt == RT_DT_BF16) zm = ldg128(t.nm + i * 2);
                if (vdt == RT_DT_BF16) zv = ldg128(t.nv + i * 2);
            }
            float p[8], g[8], m[8], v[8];
            auto load8 = [&](uint64_t base, uint32_t dt, float (&x)[8]) {
                if (dt == RT_DT_F64 || dt == RT_DT_F32) load8_wave_wide(base, dt, w0, lane, stage, x);
                else load8_any(base, dt, i, x);
            };
            auto store8 = [&](uint64_t base, uint32_t dt, const float (&x)[8], u32x4 noise) {
                if (dt == RT_DT_F64 || dt == RT_DT_F32) store8_wave_wide(base, dt, w0, lane, stage, x);
                else store8_any(base, dt, i, x, noise);
            };
            load8(t.p, pdt, p);
            load8(t.g, gdt, g);
            load8(t.m, mdt, m);
            load8(t.v, vdt, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (do_unscale) g[j] = g[j] * s.inv_loss_scale;
                if (do_clip) g[j] = g[j] * coef;
                update1(p[j], g[j], m[j], v[j], s);
            }
            store8(t.p, pdt, p, zp);
            store8(t.m, mdt, m, zm);
            store8(t.v, vdt, v, zv);
            continue;
        }
        // Whole vectors of plain aligned tensors move as 128-bit accesses, like everywhere else;
        // tails, unaligned views, debug outputs and centralization go element by element below.
        if (plain && i + kVec <= n) {
            if constexpr (NOISE == RT_NOISE_EXPLICIT) {
                if (pdt == RT_DT_BF16) zp = ldg128(t.np + i * 2);
                if (mdt == RT_DT_BF16) zm = ldg128(t.nm + i * 2);
                if (vdt == RT_DT_BF16) zv = ldg128(t.nv + i * 2);
            }
            float p[8], g[8], m[8], v[8];
            load8_any(t.p, pdt, i, p);
            load8_any(t.g, gdt, i, g);
            load8_any(t.m, mdt, i, m);
            load8_any(t.v, vdt, i, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (do_unscale) g[j] = g[j] * s.inv_loss_scale;
                if (do_clip) g[j] = g[j] * coef;
                update1(p[j], g[j], m[j], v[j], s);
            }
            store8_any(t.p, pdt, i, p, zp);
            store8_any(t.m, mdt, i, m, zm);
            store8_any(t.v, vdt, i, v, zv);
            continue;
        }
        uint64_t row = 0, rem = 0;
        if (t.row_mean != 0) {
            const uint64_t e0 = (t.block_base << 3) + i;
            row = e0 / t.row_len;
            rem = e0 - row * t.row_len;
        }
#pragma unroll 1
        for (int j = 0; j < kVec; ++j) {
            const uint64_t e = i + j;
            if (e >= n) break;
            float p = load_any(t.p, pdt, e);
            float g = load_any(t.g, gdt, e);
            float m = load_any(t.m, mdt, e);
            float v = load_any(t.v, vdt, e);
            if (do_unscale) g = g * s.inv_loss_scale;
            if (do_clip) g = g * coef;
            if (t.row_mean != 0) {
                const float mc = cen_term(ldg32f(t.row_mean + row * 4), s, do_clip, coef);
                g = g - mc;
                if (++rem == t.row_len) {
                    rem = 0;
                    ++row;
                }
            }
            update1(p, g, m, v, s);
            if (t.dp != 0) stg32f(t.dp + e * 4, p);
            if (t.dm != 0) stg32f(t.dm + e * 4, m);
            if (t.dv != 0) stg32f(t.dv + e * 4, v);
            uint32_t np16, nm16, nv16;
            if constexpr (NOISE == RT_NOISE_EXPLICIT) {
                np16 = pdt == RT_DT_BF16 ? ldg16(t.np + e * 2) : 0u;
                nm16 = mdt == RT_DT_BF16 ? ldg16(t.nm + e * 2) : 0u;
                nv16 = vdt == RT_DT_BF16 ? ldg16(t.nv + e * 2) : 0u;
            } else {
                np16 = noise_field(zp, j);
                nm16 = noise_field(zm, j);
                nv16 = noise_field(zv, j);
            }
            store_any(t.p, pdt, e, p, np16);
            store_any(t.m, mdt, e, m, nm16);
            store_any(t.v, vdt, e, v, nv16);
        }
    }
}

// ---------------------------------------------------------------------------
// Copies a table image from pinned host memory (read over the host link by the
// kernel itself) into device memory.  The streamed pipeline uses this instead
// of a DMA copy: a small hipMemcpyAsync queued between the large H2D / D2H
// copies was measured to slow the D2H copies down fourfold.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void table_upload_kernel(uint64_t dst, uint64_t src_host, uint64_t n_vec) {
    for (uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x; i < n_vec; i += (uint64_t)gridDim.x * kThreads)
        *(RT_GLOBAL u32x4*)(dst + i * 16) = *(const RT_GLOBAL u32x4*)(src_host + i * 16);
}

// Publishes a ticket number to a word in pinned host memory.  Queued on the D2H
// stream behind the last copy of a call, it lets the host see completion by
// reading memory, without entering the runtime.
__global__ void publish_ticket_kernel(uint64_t host_word, uint64_t ticket) {
    __hip_atomic_store((RT_GLOBAL uint64_t*)host_word, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// ---------------------------------------------------------------------------
// Stream probe: the memory traffic of the all-bf16 fast kernel (read p, g, m, v;
// write p, m, v in place, same chunking and prefetch) with the arithmetic
// replaced by two integer ops.  Its rate is what this access pattern can get
// out of HBM on the device at hand, i.e. the practical ceiling of the update.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void stream_probe_kernel(uint64_t p, uint64_t g, uint64_t m, uint64_t v) {
    constexpr uint64_t kStride = (uint64_t)64 * kVec * 2;  // a wave walks its own contiguous quarter of the chunk
    const uint64_t i0 = ((uint64_t)blockIdx.x * kChunkElems + (uint64_t)(threadIdx.x >> 6) * (64 * kVec * kItersPerChunk) +
                         (uint64_t)(threadIdx.x & 63u) * kVec) * 2;
    u32x4 a = ldg128(p + i0), b = ldg128(g + i0), c = ldg128(m + i0), d = ldg128(v + i0);
#pragma unroll
    for (int it = 0; it < kItersPerChunk; ++it) {
        const uint64_t i = i0 + it * kStride;
        u32x4 na, nb, nc, nd;
        if (it + 1 < kItersPerChunk) {
            na = ldg128(p + i + kStride); nb = ldg128(g + i + kStride);
            nc = ldg128(m + i + kStride); nd = ldg128(v + i + kStride);
        }
        stg128(p + i, a ^ b);
        stg128(m + i, c ^ b);
        stg128(v + i, d ^ b);
        if (it + 1 < kItersPerChunk) { a = na; b = nb; c = nc; d = nd; }
    }
}

// ---------------------------------------------------------------------------
// copy_stochastic_ on its own: fp32 -> bf16.  Philox counter word 2 is 3
// ("which" values 0..2 belong to the step), word 3 is 0.
// ---------------------------------------------------------------------------
template <int NOISE>
__global__ __launch_bounds__(kThreads) void sr_copy_kernel(uint64_t target, uint64_t source, uint64_t n,
                                                           uint64_t noise, uint32_t seed_lo, uint32_t seed_hi,
                                                           int aligned) {
    // Whole blocks of 2048 elements of aligned arrays use the lane mapping of the wide update
    // kernel (a lane owns 4 + 4 elements of its wave's 512-element block, so the fp32 loads are
    // contiguous kilobytes across the wave) and the same neighbour swap of Philox halves; the last
    // partial block and unaligned arrays go element by element under an index guard.
    constexpr uint64_t kBlock = (uint64_t)kThreads * kVec;
    constexpr uint32_t kHalf = 64 * kVec / 2;
    const uint64_t n_blocks = (n + kBlock - 1) / kBlock;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const bool odd = (lane & 1u) != 0u;
    for (uint64_t b = blockIdx.x; b < n_blocks; b += gridDim.x) {
        const uint64_t base = b * kBlock;
        if (aligned && base + kBlock <= n) {
            const uint64_t blk = base + (uint64_t)wave * (64 * kVec);
            u32x4 raw[2];
            u32x2 z[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint64_t e = blk + (uint64_t)h * kHalf + lane * 4u;
                raw[h] = ldg128(source + e * 4);
                if constexpr (NOISE == RT_NOISE_EXPLICIT) z[h] = ldg64(noise + e * 2);
            }
            if constexpr (NOISE == RT_NOISE_PHILOX) {
                const uint64_t first = (blk >> 3) + (lane >> 1);
                const uint64_t mine = odd ? first + (kHalf >> 3) : first;
                const u32x4 r = philox4x32_10((uint32_t)mine, (uint32_t)(mine >> 32), 3u, 0u, seed_lo, seed_hi);
                const uint32_t g0 = swap_neighbour(odd ? r.x : r.z);
                const uint32_t g1 = swap_neighbour(odd ? r.y : r.w);
                z[0].x = odd ? g0 : r.x; z[0].y = odd ? g1 : r.y;
                z[1].x = odd ? r.z : g0; z[1].y = odd ? r.w : g1;
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint64_t e = blk + (uint64_t)h * kHalf + lane * 4u;
                float x[4];
                decode4<RT_DT_F32>(raw[h], x);
                store_out4<RT_DT_BF16>(target, e, x, z[h]);
            }
        } else {
            const uint64_t i = base + (uint64_t)threadIdx.x * kVec;
            if (i >= n) continue;
            const Raw8<RT_DT_F32> r = load_raw_guarded<RT_DT_F32>(source, i, n);
            float x[8];
            decode<RT_DT_F32>(r, x);
            u32x4 z;
            if constexpr (NOISE == RT_NOISE_EXPLICIT) {
                z = load_raw_guarded<RT_DT_BF16>(noise, i, n).a;
            } else {
                const uint64_t blk = i >> 3;
                z = philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), 3u, 0u, seed_lo, seed_hi);
            }
            store_out_guarded<RT_DT_BF16>(target, i, n, x, z);
        }
    }
}

// ---------------------------------------------------------------------------
// Self-test: sqrt_rn_from_2m96 against the compiler's sqrtf on every float of its domain
// [2^-96, +inf) -- 1 879 048 192 bit patterns.  Counts the patterns whose results differ.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void sqrt_selftest_kernel(unsigned long long* __restrict__ mismatches) {
    constexpr uint32_t kLo = 0x0F800000u, kHi = 0x7F800000u;
    uint32_t bad = 0;
    for (uint64_t u = (uint64_t)kLo + (uint64_t)blockIdx.x * kThreads + threadIdx.x; u < kHi;
         u += (uint64_t)gridDim.x * kThreads) {
        float x = u2f((uint32_t)u);
        asm volatile("" : "+v"(x));  // keep the two evaluations apart
        const float a = sqrt_rn_from_2m96(x);
        const float b = __builtin_sqrtf(x);
        bad += f2u(a) != f2u(b) ? 1u : 0u;
    }
    if (bad) atomicAdd(mismatches, (unsigned long long)bad);
}

// ---------------------------------------------------------------------------
// Wavefront / workgroup sum in a fixed order (deterministic run to run).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x = x + __shfl_xor(x, off, 64);
    return x;
}

__device__ __forceinline__ float block_sum(float x, float* lds) {
    x = wave_sum(x);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = x;
    __syncthreads();
    float r = 0.0f;
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 0; w < kThreads / 64; ++w) r = r + lds[w];
    }
    __syncthreads();
    return r;  // valid in thread 0
}

// Sum of squares of one chunk of one gradient tensor (per-lane partial).
// Whole chunk of an aligned gradient: every load is 16 bytes per lane and contiguous across the
// wave whatever the element type (a sum does not care which lane gets which element), all loads
// of the chunk are in flight together.
template <int GDT>
__device__ __forceinline__ float chunk_sumsq_full(uint64_t g_addr, uint32_t chunk, float inv_loss_scale) {
    constexpr int kLoads = (int)(kChunkElems * esize<GDT>() / 16 / kThreads);  // 4 (16-bit) or 8 (fp32)
    const uint64_t base = g_addr + (uint64_t)chunk * kChunkElems * esize<GDT>() + (uint64_t)threadIdx.x * 16;
    u32x4 r[kLoads];
#pragma unroll
    for (int k = 0; k < kLoads; ++k) r[k] = ldg128(base + (uint64_t)k * (kThreads * 16));
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
        if constexpr (GDT == RT_DT_F32) {
            const float x[4] = {u2f(r[k].x), u2f(r[k].y), u2f(r[k].z), u2f(r[k].w)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float y = x[j] * inv_loss_scale;
                acc = __builtin_fmaf(y, y, acc);
            }
        } else {
            Raw8<GDT> raw;
            raw.a = r[k];
            float x[8];
            decode<GDT>(raw, x);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float y = x[j] * inv_loss_scale;
                acc = __builtin_fmaf(y, y, acc);
            }
        }
    }
    return acc;
}

template <int GDT>
__device__ __forceinline__ float chunk_sumsq(uint64_t g_addr, uint64_t n, uint32_t chunk, float inv_loss_scale) {
    const uint64_t chunk_base = (uint64_t)chunk * kChunkElems;
    const bool aligned = (g_addr & 15u) == 0;
    if (aligned && chunk_base + kChunkElems <= n) return chunk_sumsq_full<GDT>(g_addr, chunk, inv_loss_scale);
    float acc = 0.0f;
#pragma unroll 1
    for (int it = 0; it < kItersPerChunk; ++it) {
        const uint64_t i = chunk_base + (uint64_t)(it * kThreads + (int)threadIdx.x) * kVec;
        if (i >= n) break;
        const bool full = aligned && (i + kVec <= n);
        const Raw8<GDT> r = full ? load_raw<GDT>(g_addr, i) : load_raw_guarded<GDT>(g_addr, i, n);
        float g[8];
        decode<GDT>(r, g);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float x = g[j] * inv_loss_scale;
            acc = __builtin_fmaf(x, x, acc);
        }
    }
    return acc;
}

__device__ __forceinline__ float chunk_sumsq_dt(int dt, uint64_t g_addr, uint64_t n, uint32_t chunk,
                                                float inv_loss_scale) {
    if (dt == RT_DT_BF16) return chunk_sumsq<RT_DT_BF16>(g_addr, n, chunk, inv_loss_scale);
    if (dt == RT_DT_F32) return chunk_sumsq<RT_DT_F32>(g_addr, n, chunk, inv_loss_scale);
    return chunk_sumsq<RT_DT_F16>(g_addr, n, chunk, inv_loss_scale);
}

// ---------------------------------------------------------------------------
// Pass 1 of the global grad norm: workgroup b accumulates the chunks
// b, b + gridDim.x, ... and writes one partial sum of squares.  The only table
// is one NormEntry per gradient (small enough to live in a fixed device array
// for the entry point that allocates nothing); a chunk finds its gradient by
// binary search.  Chunks are numbered in two sequences -- first every whole
// chunk of the 16-byte aligned gradients, then everything else, each in tensor
// order -- so that most workgroups see nothing but whole chunks.
// ---------------------------------------------------------------------------
struct alignas(16) NormEntry {
    uint64_t g;
    uint64_t numel;
    uint32_t first_whole;  // number of the gradient's first whole chunk among the whole chunks
    uint32_t first_rest;   // number of its first other chunk among the other chunks
    uint32_t n_whole;      // whole chunks it contributes to the first sequence
    uint32_t dtype;
};
static_assert(sizeof(NormEntry) == 32, "NormEntry layout");

// A slice of the table travels to the device array as a kernel argument (no copy engine, no
// staging memory): at most kNormEntriesPerWrite entries per launch.
constexpr uint32_t kNormEntriesPerWrite = 64;
struct NormEntrySlice {
    NormEntry e[kNormEntriesPerWrite];
};
__global__ __launch_bounds__(kNormEntriesPerWrite) void norm_table_write_kernel(NormEntry* __restrict__ table,
                                                                                uint32_t first, uint32_t count,
                                                                                const NormEntrySlice slice) {
    if (threadIdx.x < count) table[first + threadIdx.x] = slice.e[threadIdx.x];
}

__global__ __launch_bounds__(kThreads) void grad_sumsq_table_kernel(const NormEntry* __restrict__ table, uint32_t n,
                                                                    uint32_t total_whole, uint32_t n_chunks,
                                                                    float inv_loss_scale,
                                                                    double* __restrict__ partials) {
    __shared__ float lds[kThreads / 64];
    double total = 0.0;
    for (uint32_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const bool whole = c < total_whole;
        const uint32_t key = whole ? c : c - total_whole;
        uint32_t lo = 0, hi = n;  // last entry whose first chunk number in this sequence is <= key
        while (hi - lo > 1u) {
            const uint32_t mid = (lo + hi) >> 1;
            const uint32_t f = whole ? table[mid].first_whole : table[mid].first_rest;
            if (f <= key) lo = mid; else hi = mid;
        }
        const NormEntry e = table[lo];
        const uint32_t chunk = whole ? key - e.first_whole : e.n_whole + (key - e.first_rest);
        const float acc = chunk_sumsq_dt((int)e.dtype, e.g, e.numel, chunk, inv_loss_scale);
        const float bs = block_sum(acc, lds);
        total += (double)bs;  // meaningful in thread 0 only
    }
    if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

// Pass 2: one workgroup folds the partials in index order and derives the
// clip coefficient with torch.nn.utils.clip_grad_norm_'s formula.
__global__ __launch_bounds__(kThreads) void grad_norm_finish_kernel(const double* __restrict__ partials,
                                                                    uint32_t n_partials, float max_norm,
                                                                    float* __restrict__ out) {
    __shared__ double lds[kThreads];
    double acc = 0.0;
    for (uint32_t i = threadIdx.x; i < n_partials; i += kThreads) acc += partials[i];
    lds[threadIdx.x] = acc;
    __syncthreads();
    for (int w = kThreads / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) lds[threadIdx.x] += lds[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float total = (float)__builtin_sqrt(lds[0]);
        const bool finite = (f2u(total) & 0x7F800000u) != 0x7F800000u;
        const float c = max_norm / (total + 1e-6f);
        out[0] = total;
        // a non-finite norm must never scale anything: the skip flag stops the update
        out[1] = (finite && c < 1.0f) ? c : 1.0f;
        ((uint32_t*)out)[2] = finite ? 0u : 1u;
    }
}

// ---------------------------------------------------------------------------
// Row means for centralization (adamw.py:179-184).  A pure read of the gradients, 2 or 4 bytes per
// element, so what matters is how many loads are in flight:
//  * rows of at most kWaveRowMax elements (every matrix of a transformer) are summed by ONE
//    wavefront each.  A lane issues up to eight 128-bit loads (sixteen for fp32) before its first
//    add, each load instruction contiguous across the wave; no LDS, no barrier, and the four waves
//    of a workgroup work on four rows independently;
//  * longer rows (a huge 1-D tensor is a single row) take one workgroup per row, four vectors per
//    thread in flight, and one LDS reduction per row.
// Which of the two a row takes depends on its length alone, and both entry points (one gradient, or
// the gradients of a whole step through a table) use the same two functions, so the same row
// gives the same bits through either.
// ---------------------------------------------------------------------------
constexpr uint32_t kWaveRowMax = 32768;
constexpr int kRowVecs = 8;   // vectors of 8 elements per lane and batch of the wave path

template <int GDT>
__device__ __forceinline__ float add_vec(float acc, const Raw8<GDT>& r, float inv_loss_scale) {
    float x[8];
    decode<GDT>(r, x);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = acc + x[j] * inv_loss_scale;
    return acc;
}

template <int DT>
__device__ __forceinline__ float load_elem(uint64_t base, uint64_t idx) {
    if constexpr (DT == RT_DT_BF16) return u2f(ldg16(base + idx * 2) << 16);
    else if constexpr (DT == RT_DT_F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)ldg16(base + idx * 2));
    else return ldg32f(base + idx * 4);
}

// Sum of row [base, base + row_len) of g by the calling wavefront; the result is in every lane.
// A row that starts on a 16-byte boundary (every row of a matrix whose rows are a multiple of 8
// elements long) moves as whole vectors, 32 registers of them in flight per lane, and at most 7
// single elements at its end; any other row goes element by element.
// KEEP: the row is read again right away (by the update that takes its own row means), so its
// lines are loaded the ordinary way and stay in the L2; the values and their order are the same.
template <int DT>
__device__ __forceinline__ Raw8<DT> load_raw_cached(uint64_t base, uint64_t i) {
    Raw8<DT> r;
    const uint64_t addr = base + i * esize<DT>();
    r.a = *(const RT_GLOBAL u32x4*)addr;
    if constexpr (DT == RT_DT_F32) r.b = *(const RT_GLOBAL u32x4*)(addr + 16);
    return r;
}

template <int GDT, bool KEEP = false>
__device__ __forceinline__ float row_sum_wave(uint64_t g, uint64_t base, uint32_t row_len, float inv_loss_scale) {
    constexpr int kB = GDT == RT_DT_F32 ? kRowVecs / 2 : kRowVecs;   // an fp32 vector of 8 elements is two loads
    const uint32_t lane = threadIdx.x & 63u;
    float acc = 0.0f;
    if (((g + base * esize<GDT>()) & 15u) == 0) {
        const uint32_t n_vec = row_len / kVec;
        for (uint32_t v0 = 0; v0 < n_vec; v0 += 64u * kB) {
            Raw8<GDT> r[kB];
#pragma unroll
            for (int k = 0; k < kB; ++k) {
                const uint32_t v = v0 + (uint32_t)k * 64u + lane;
                if (v < n_vec)
                    r[k] = KEEP ? load_raw_cached<GDT>(g, base + (uint64_t)v * kVec) : load_raw<GDT>(g, base + (uint64_t)v * kVec);
            }
#pragma unroll
            for (int k = 0; k < kB; ++k) {
                const uint32_t v = v0 + (uint32_t)k * 64u + lane;
                if (v < n_vec) acc = add_vec<GDT>(acc, r[k], inv_loss_scale);
            }
        }
        const uint32_t t = n_vec * kVec + lane;
        if (t < row_len) acc = acc + load_elem<GDT>(g, base + t) * inv_loss_scale;
    } else {
        for (uint32_t e = lane; e < row_len; e += 64u) acc = acc + load_elem<GDT>(g, base + e) * inv_loss_scale;
    }
    return wave_sum(acc);
}

// Sum of one (long) row by the calling workgroup; valid in thread 0.
template <int GDT>
__device__ __forceinline__ float row_sum_block(uint64_t g, uint64_t base, uint64_t row_len, float inv_loss_scale,
                                               float* lds) {
    constexpr int kInFlight = 4;
    const bool aligned = ((g + base * esize<GDT>()) & 15u) == 0;
    float acc = 0.0f;
    for (uint64_t c0 = 0; c0 < row_len; c0 += (uint64_t)kThreads * kVec * kInFlight) {
        Raw8<GDT> r[kInFlight];
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const uint64_t e = c0 + ((uint64_t)k * kThreads + threadIdx.x) * kVec;
            if (e < row_len)
                r[k] = (aligned && e + kVec <= row_len) ? load_raw<GDT>(g, base + e)
                                                        : load_raw_guarded<GDT>(g, base + e, base + row_len);
        }
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const uint64_t e = c0 + ((uint64_t)k * kThreads + threadIdx.x) * kVec;
            if (e < row_len) acc = add_vec<GDT>(acc, r[k], inv_loss_scale);
        }
    }
    return block_sum(acc, lds);
}

__device__ __forceinline__ float row_sum_wave_dt(uint32_t dt, uint64_t g, uint64_t base, uint32_t row_len, float inv) {
    if (dt == RT_DT_BF16) return row_sum_wave<RT_DT_BF16>(g, base, row_len, inv);
    if (dt == RT_DT_F32) return row_sum_wave<RT_DT_F32>(g, base, row_len, inv);
    return row_sum_wave<RT_DT_F16>(g, base, row_len, inv);
}
__device__ __forceinline__ float row_sum_block_dt(uint32_t dt, uint64_t g, uint64_t base, uint64_t row_len, float inv,
                                                  float* lds) {
    if (dt == RT_DT_BF16) return row_sum_block<RT_DT_BF16>(g, base, row_len, inv, lds);
    if (dt == RT_DT_F32) return row_sum_block<RT_DT_F32>(g, base, row_len, inv, lds);
    return row_sum_block<RT_DT_F16>(g, base, row_len, inv, lds);
}

// One gradient.  Rows of at most kWaveRowMax elements: workgroup b takes rows 4b .. 4b+3, one per wave.
__global__ __launch_bounds__(kThreads) void row_mean_kernel(uint64_t g, uint32_t dtype, uint64_t rows, uint32_t row_len,
                                                            float inv_loss_scale, float* __restrict__ out) {
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint64_t row = (uint64_t)blockIdx.x * (kThreads / 64) + wave;
    if (row >= rows) return;
    const float sum = row_sum_wave_dt(dtype, g, row * row_len, row_len, inv_loss_scale);
    if ((threadIdx.x & 63u) == 0) out[row] = sum / (float)row_len;
}
// Longer rows: one workgroup per row.
__global__ __launch_bounds__(kThreads) void row_mean_long_kernel(uint64_t g, uint32_t dtype, uint64_t row_len,
                                                                 float inv_loss_scale, float* __restrict__ out) {
    __shared__ float lds[kThreads / 64];
    const uint64_t row = blockIdx.x;
    const float sum = row_sum_block_dt(dtype, g, row * row_len, row_len, inv_loss_scale, lds);
    if (threadIdx.x == 0) out[row] = sum / (float)row_len;
}

// The same for many gradients in one launch.  Rows are counted through all gradients of the launch;
// `first` holds every gradient's first row number (ascending), `table` its record at the same index.
struct alignas(16) RowMeanEntry {
    uint64_t g;
    uint64_t out;        // fp32[rows] of this gradient
    uint64_t row_len;
    uint32_t first_row;  // number of this gradient's first row in the launch
    uint32_t dtype;
    uint32_t rows;       // rows of this gradient
    uint32_t pad[3];
};
static_assert(sizeof(RowMeanEntry) == 48, "RowMeanEntry layout");

// Workgroup b takes rows 4b .. 4b+3, one per wave.  (A fixed number of workgroups whose waves walk rows
// a launch-width apart, looking their gradient up only when it changes, measured 8 % slower: a wave
// then has nothing in flight while it reduces a row.)
__global__ __launch_bounds__(kThreads) void row_mean_table_kernel(const uint32_t* __restrict__ first,
                                                                  const RowMeanEntry* __restrict__ table, uint32_t n,
                                                                  uint32_t rows_total, float inv_loss_scale) {
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t row = blockIdx.x * (kThreads / 64) + wave;
    if (row >= rows_total) return;
    const uint32_t idx = find_range(first, n, row);   // each wave searches on its own
    const RowMeanEntry e = load_const(&table[idx]);
    const uint64_t r = row - e.first_row;
    const float sum = row_sum_wave_dt(e.dtype, e.g, r * e.row_len, (uint32_t)e.row_len, inv_loss_scale);
    if ((threadIdx.x & 63u) == 0) ((RT_GLOBAL float*)e.out)[r] = sum / (float)e.row_len;
}

__global__ __launch_bounds__(kThreads) void row_mean_table_long_kernel(const uint32_t* __restrict__ first,
                                                                       const RowMeanEntry* __restrict__ table, uint32_t n,
                                                                       float inv_loss_scale) {
    __shared__ float lds[kThreads / 64];
    const uint32_t row = blockIdx.x;
    const uint32_t idx = find_range(first, n, row);
    const RowMeanEntry e = load_const(&table[idx]);
    const uint64_t r = row - e.first_row;
    const float sum = row_sum_block_dt(e.dtype, e.g, r * e.row_len, e.row_len, inv_loss_scale, lds);
    if (threadIdx.x == 0) ((RT_GLOBAL float*)e.out)[r] = sum / (float)e.row_len;
}

// ---------------------------------------------------------------------------
// Update with centralization (adamw.py:179-184) that takes the row means itself.  One wavefront per
// row: it sums the row exactly as the row-mean kernels above do (row_sum_wave: same loads, same
// order, same bits), keeps the mean in a register, and then updates the row, four vectors per lane
// at a time with all their loads issued first, as the fast kernel does.  The gradient is read twice,
// but the second time out of the L2 it was loaded into a few microseconds before: the separate
// row-mean pass (2 bytes per element more from HBM, one launch more) is not needed for such tensors.
// For whole 16-byte-aligned tensors of 16-bit arrays with Philox noise whose rows are a multiple of 8
// and between 512 and kWaveRowMax elements long -- every matrix of a transformer; the host sends
// everything else through precomputed means.  `first` lists every tensor's first row number in the
// launch (ascending), `fast_tensors` its record at the same index; workgroup b takes rows 4b .. 4b+3.
// Two instances, launched apart: rows of at most kRowwiseShortMax elements keep their gradient in
// registers (158 registers, three waves per SIMD: 2 % faster on such rows than reading it again, 1.4 %
// slower on long rows if they shared the instance), longer rows read it again (128 registers, four waves).
// ---------------------------------------------------------------------------
constexpr uint32_t kRowwiseMinLen = 64 * kVec;   // one vector per lane at least
constexpr uint32_t kRowwiseShortMax = 64 * kVec * kRowVecs;   // 4096: a row that one batch of row_sum_wave covers
static_assert(kRowVecs == 2 * kFastIters, "the short-row path updates a row in two halves");

template <int PDT, int GDT, int MDT, int VDT, bool SHORT>
__global__ __launch_bounds__(kThreads) void sr_adamw_rowwise_kernel(const LaunchArgs a) {
    if (a.skip != nullptr && load_const(a.skip) != 0u) return;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t row = blockIdx.x * (kThreads / 64) + wave;
    if (row >= a.n_rows) return;
    const uint32_t ri = find_range(a.first, a.n_ranges, row);   // each wave searches on its own
    const DevTensor t = load_const(&a.fast_tensors[ri]);
    const uint32_t r = row - load_const(&a.first[ri]);
    UpdateCtx c;
    make_ctx(a, t.set_idx, c);
    const uint32_t row_len = (uint32_t)t.row_len;
    const uint64_t e0 = (uint64_t)r * row_len;
    const uint64_t tp = t.p, tg = t.g, tm = t.m, tv = t.v;

    if constexpr (SHORT) {
        // Rows of at most kRowwiseShortMax elements: the gradient stays in registers between the sum and the
        // update (eight vectors per lane), and the other loads of the row's first half are on the way
        // while the row is summed.  The sum adds the same values in the same order as row_sum_wave.
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t n_vec = row_len / kVec;   // <= 64 * kRowVecs
        Raw8<GDT> gr[kRowVecs];
#pragma unroll
        for (int k = 0; k < kRowVecs; ++k) {
            const uint32_t vi = (uint32_t)k * 64u + lane;
            if (vi < n_vec) gr[k] = load_raw<GDT>(tg, e0 + (uint64_t)vi * kVec);
        }
        struct In3 { Raw8<PDT> p; Raw8<MDT> m; Raw8<VDT> v; };
        In3 q[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t vi = (uint32_t)k * 64u + lane;
            if (vi < n_vec) {
                const uint64_t i = e0 + (uint64_t)vi * kVec;
                q[k].p = load_raw<PDT>(tp, i); q[k].m = load_raw<MDT>(tm, i); q[k].v = load_raw<VDT>(tv, i);
            }
        }
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < kRowVecs; ++k) {
            const uint32_t vi = (uint32_t)k * 64u + lane;
            if (vi < n_vec) acc = add_vec<GDT>(acc, gr[k], c.s.inv_loss_scale);
        }
        const float mc = cen_term(wave_sum(acc) / (float)row_len, c.s, c.do_clip, c.coef);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            if (half == 1) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t vi = (uint32_t)(4 + k) * 64u + lane;
                    if (vi < n_vec) {
                        const uint64_t i = e0 + (uint64_t)vi * kVec;
                        q[k].p = load_raw<PDT>(tp, i); q[k].m = load_raw<MDT>(tm, i); q[k].v = load_raw<VDT>(tv, i);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t vi = (uint32_t)(half * 4 + k) * 64u + lane;
                if (vi < n_vec) {
                    const uint64_t i = e0 + (uint64_t)vi * kVec;
                    float p[8], g[8], m[8], v[8];
                    decode<PDT>(q[k].p, p);
                    decode<GDT>(gr[half * 4 + k], g);
                    decode<MDT>(q[k].m, m);
                    decode<VDT>(q[k].v, v);
                    u32x4 zp = 0, zm = 0, zv = 0;
                    philox_noise3<PDT, MDT, VDT>(t, c, i, zp, zm, zv);
                    scale_grads(g, c);
#pragma unroll
                    for (int j = 0; j < 8; ++j) g[j] = g[j] - mc;
                    update_n<8>(p, g, m, v, c.s);
                    store_out<PDT>(tp, i, p, zp);
                    store_out<MDT>(tm, i, m, zm);
                    store_out<VDT>(tv, i, v, zv);
                }
            }
        }
        return;
    }
    // (sixteen vectors per lane on the way at once instead of eight -- a lane adds its vectors in ascending
    // order whatever the batch, so no bit changes -- measured the same time on the 8B set)
    const float sum = row_sum_wave<GDT, true>(tg, e0, row_len, c.s.inv_loss_scale);
    const float mc = cen_term(sum / (float)row_len, c.s, c.do_clip, c.coef);

    struct In {
        Raw8<PDT> p;
        Raw8<GDT> g;
        Raw8<MDT> m;
        Raw8<VDT> v;
    };
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t n_vec = row_len / kVec;
    for (uint32_t v0 = 0; v0 < n_vec; v0 += 64u * kFastIters) {
        In q[kFastIters];
#pragma unroll
        for (int k = 0; k < kFastIters; ++k) {
            const uint32_t vi = v0 + (uint32_t)k * 64u + lane;
            if (vi < n_vec) {
                const uint64_t i = e0 + (uint64_t)vi * kVec;
                q[k].p = load_raw<PDT>(tp, i);
                q[k].g = load_raw<GDT>(tg, i);
                q[k].m = load_raw<MDT>(tm, i);
                q[k].v = load_raw<VDT>(tv, i);
            }
        }
#pragma unroll
        for (int k = 0; k < kFastIters; ++k) {
            const uint32_t vi = v0 + (uint32_t)k * 64u + lane;
            if (vi < n_vec) {
                const uint64_t i = e0 + (uint64_t)vi * kVec;
                float p[8], g[8], m[8], v[8];
                decode<PDT>(q[k].p, p);
                decode<GDT>(q[k].g, g);
                decode<MDT>(q[k].m, m);
                decode<VDT>(q[k].v, v);
                u32x4 zp = 0, zm = 0, zv = 0;
                philox_noise3<PDT, MDT, VDT>(t, c, i, zp, zm, zv);
                scale_grads(g, c);
#pragma unroll
                for (int j = 0; j < 8; ++j) g[j] = g[j] - mc;   // grad.sub_(mean.mul_(c)): the product is rounded, then subtracted
                update_n<8>(p, g, m, v, c.s);
                store_out<PDT>(tp, i, p, zp);
                store_out<MDT>(tm, i, m, zm);
                store_out<VDT>(tv, i, v, zv);
            }
        }
    }
}

}  // namespace rt
