/*
 * CPU oracle for the stochastic-rounding AdamW step.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain scalar C, the
 * algorithm of the reference's ramtorch/stochastic_optimizers/adamw.py so the
 * HIP kernels can be checked against it.  Only tests/, the smoke check and the
 * benchmark's cpu_baseline leg may load it; the shipped library never does.
 *
 * The reference's arithmetic is executed by torch's elementwise kernels, whose
 * rounding sequence (which products are fused into an FMA, whether the scalar
 * division is a reciprocal multiply, operand association) is a property of the
 * torch build.  Every such choice is a bit of `flavour`, so that one setting
 * can be pinned against the torch kernels that the reference would run.
 *
 * Parity pins (see tests/): the 8-element known-answer vector, the Random123
 * Philox4x32-10 vectors, the brute-force count of round-ups over all 65536
 * noises, the closed-form cases of the update (zero grad, zero state), and
 * torch's own GPU kernels run op by op on the GPU box (committed as golden
 * vectors), torch's CPU kernels for the CPU flavour, numpy's and torch's
 * fp32 -> fp16 conversion for orc_f32_to_f16_rne.
 * Parity unpinned: orc_grad_sumsq and orc_row_means.  They are sums, whose value
 * depends on the order of addition; nothing in the reference fixes an order
 * (it has no clipping at all, and its row mean is whatever torch's reduction
 * does), so they are checked against a float64 evaluation to 1e-6 relative and
 * the kernels are compared with them to that tolerance, not bit for bit.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see oracle/Makefile).
 * Contraction must stay off: every fused operation below is an explicit fmaf.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- flavour bits --------------------------------------------------------- */
#define ORC_FMA_ADD 1u          /* adamw.py:190  m' = fma(a1, g, m*b1)  else two roundings   */
#define ORC_FMA_ADDCMUL 2u      /* adamw.py:191  v' = fma(., ., v*b2)   else two roundings   */
#define ORC_FMA_ADDCDIV 4u      /* adamw.py:200  p' = fma(., ., p1)     else two roundings   */
#define ORC_DIV_RECIP 8u        /* adamw.py:193  sqrt(v)*fl(1/bcs)      else sqrt(v)/bcs     */
#define ORC_ADDCMUL_AG_FIRST 16u /* adamw.py:191 (a2*g)*g               else a2*(g*g)        */
#define ORC_ADDCDIV_AM_FIRST 32u /* adamw.py:200 (-ss*m)/den            else -ss*(m/den)     */

#define ORC_DT_BF16 0
#define ORC_DT_F32 1
#define ORC_DT_F16 2
#define ORC_DT_F64 3

#define ORC_NOISE_PHILOX 0
#define ORC_NOISE_EXPLICIT 1

/* Per-(group, step) constants, already rounded to float32 the way each ATen
 * call rounds its Python-double scalar at the point of use (adamw.py:186-200). */
typedef struct orc_scalars {
    float beta1;          /* float32(beta1)                         adamw.py:190 */
    float one_m_beta1;    /* float32(1 - beta1)                     adamw.py:190 */
    float beta2;          /* float32(beta2)                         adamw.py:191 */
    float one_m_beta2;    /* float32(1 - beta2)                     adamw.py:191 */
    float bcs;            /* float32((1 - beta2**step) ** 0.5)      adamw.py:187 */
    float inv_bcs;        /* float32(1.0 / bcs), reciprocal in double  adamw.py:193 */
    float eps;            /* float32(eps)                           adamw.py:194 */
    float decay;          /* float32(1 - (lr/bc) * wd)              adamw.py:198 */
    float neg_step_size;  /* float32(-(lr/bc))                      adamw.py:200 */
    float inv_loss_scale; /* extension: grads are multiplied by this first (1.0f = off) */
    int32_t apply_decay;  /* weight_decay != 0                      adamw.py:197 */
    int32_t apply_clip;   /* extension: multiply grads by a clip coefficient */
} orc_scalars;

static inline float bits_to_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static inline uint32_t f32_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* bf16 -> fp32 is exact: the 16 bits become the high half (adamw.py:160-170). */
float orc_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* IEEE binary16 -> fp32, exact. */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * bits_to_f32(0x33800000u); /* 2^-24 */
        return bits_to_f32(f32_to_bits(v) | sign);
    }
    if (exp == 31) return bits_to_f32(sign | 0x7F800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/*
 * fp32 -> IEEE binary16, round to nearest even with gradual underflow: the
 * conversion Tensor.copy_ performs when a param or state is kept in fp16
 * (adamw.py:208,214,221-222).  NaN payloads are not part of the contract
 * (a quiet NaN of the same sign is returned).
 */
uint16_t orc_f32_to_f16_rne(float x) {
    uint32_t b = f32_to_bits(x);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    uint32_t a = b & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    if (a == 0x7F800000u) return (uint16_t)(sign | 0x7C00u);
    int32_t exp = (int32_t)(a >> 23) - 127 + 15; /* biased binary16 exponent */
    uint32_t man = a & 0x7FFFFFu;
    if (exp >= 31) return (uint16_t)(sign | 0x7C00u);
    if (exp <= 0) {
        /* subnormal result: the 24-bit significand moves right by 14 - exp */
        int32_t shift = 14 - exp;
        if (shift > 25 || a == 0) return sign;
        uint32_t sig = man | 0x800000u;
        uint32_t half = sig >> shift;
        uint32_t rem = sig & ((1u << shift) - 1u);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) ++half;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) ++half; /* may carry up to infinity */
    return (uint16_t)(sign | half);
}

void orc_f32_to_f16_array(const float* x, uint16_t* out, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16_rne(x[i]);
}

/*
 * Stochastic rounding of one fp32 value to bf16 (adamw.py:14-30):
 *   result = noise(int32 in [0,65536)) + bits(source)     :24  (wrapping add)
 *   result &= 0xFFFF0000                                  :27
 *   target <- result viewed as fp32                       :30  (exact in bf16)
 * so the stored 16 bits are the high half of the 32-bit sum.
 */
uint16_t orc_sr_bf16(float x, uint16_t noise) {
    uint32_t r = f32_to_bits(x) + (uint32_t)noise;
    return (uint16_t)(r >> 16);
}

/* ---- Philox4x32-10 (Salmon et al., SC'11; Random123 reference constants) -- */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
    const uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)M0 * c0;
        uint64_t p1 = (uint64_t)M1 * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += W0; k1 += W1;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/*
 * Rounding noise in Philox mode.  The reference draws torch.randint from a
 * generator reseeded with step+42 / +69 / +420 (adamw.py:206-218), which gives
 * every tensor of one shape the same noise; that stream is deliberately not
 * reproduced.  Here each aligned block of 8 elements of one array of one tensor
 * at one step owns one Philox call:
 *   counter = (block_lo, block_hi, tensor_id*4 + which, step)   which: 0=p 1=m 2=v
 *   key     = (seed_lo, seed_hi)
 * and element e of the tensor takes 16-bit field (e & 7) of the 128-bit output
 * (little-endian: word (e&7)>>1, low half for even e).
 */
uint16_t orc_philox_noise(uint64_t seed, uint32_t step, uint32_t tensor_id, uint32_t which,
                          uint64_t elem) {
    uint64_t block = elem >> 3;
    uint32_t ctr[4] = {(uint32_t)block, (uint32_t)(block >> 32), tensor_id * 4u + which, step};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t out[4];
    orc_philox4x32_10(ctr, key, out);
    uint32_t w = out[(elem & 7u) >> 1];
    return (uint16_t)((elem & 1u) ? (w >> 16) : (w & 0xFFFFu));
}

/*
 * One element of adamw.py:190-200 in float32.  p, g, m, v are the upcast
 * inputs (adamw.py:160-170); clip_coef is used only when s->apply_clip.
 */
void orc_update_elem(float p, float g, float m, float v, const orc_scalars* s, float clip_coef,
                     uint32_t flavour, float* p_out, float* m_out, float* v_out) {
    /* extensions ahead of the reference's math: unscale, then clip */
    if (s->inv_loss_scale != 1.0f) g = g * s->inv_loss_scale;
    if (s->apply_clip) g = g * clip_coef;

    /* ema.mul_(beta1).add_(grad, alpha=1-beta1)                     adamw.py:190 */
    float t = m * s->beta1;
    float m1;
    if (flavour & ORC_FMA_ADD) {
        m1 = fmaf(s->one_m_beta1, g, t);
    } else {
        float ag = s->one_m_beta1 * g;
        m1 = t + ag;
    }

    /* ema_squared.mul_(beta2).addcmul_(grad, grad, value=1-beta2)   adamw.py:191 */
    float u = v * s->beta2;
    float v1;
    if (flavour & ORC_ADDCMUL_AG_FIRST) {
        float ag = s->one_m_beta2 * g;
        if (flavour & ORC_FMA_ADDCMUL) {
            v1 = fmaf(ag, g, u);
        } else {
            float agg = ag * g;
            v1 = u + agg;
        }
    } else {
        float gg = g * g;
        if (flavour & ORC_FMA_ADDCMUL) {
            v1 = fmaf(s->one_m_beta2, gg, u);
        } else {
            float agg = s->one_m_beta2 * gg;
            v1 = u + agg;
        }
    }

    /* denom = (ema_squared.sqrt() / bias_correction_sqrt).add_(eps) adamw.py:193-195 */
    float sq = sqrtf(v1);
    float d;
    if (flavour & ORC_DIV_RECIP) {
        d = sq * s->inv_bcs;
    } else {
        d = sq / s->bcs;
    }
    float den = d + s->eps;

    /* p.mul_(1 - step_size * weight_decay)                          adamw.py:197-198 */
    float p1 = s->apply_decay ? p * s->decay : p;

    /* p.addcdiv_(ema, denom, value=-step_size)                      adamw.py:200 */
    float p2;
    if (flavour & ORC_ADDCDIV_AM_FIRST) {
        float am = s->neg_step_size * m1;
        float q = am / den;
        p2 = p1 + q; /* a + (alpha*b)/c has no product left to fuse */
    } else {
        float q = m1 / den;
        if (flavour & ORC_FMA_ADDCDIV) {
            p2 = fmaf(s->neg_step_size, q, p1);
        } else {
            float aq = s->neg_step_size * q;
            p2 = p1 + aq;
        }
    }
    *p_out = p2;
    *m_out = m1;
    *v_out = v1;
}

static inline float load_as_f32(const void* base, int dtype, uint64_t i) {
    switch (dtype) {
        case ORC_DT_BF16: return orc_bf16_to_f32(((const uint16_t*)base)[i]);
        case ORC_DT_F16: return orc_f16_to_f32(((const uint16_t*)base)[i]);
        case ORC_DT_F64: return (float)((const double*)base)[i]; /* .to(float32): round to nearest even */
        default: return ((const float*)base)[i];
    }
}

/* Write-back of one element of p / ema / ema_squared (adamw.py:204-222): bf16 is
 * stochastically rounded, every other dtype takes a plain copy_ (round to nearest). */
static inline void store_from_f32(void* base, int dtype, uint64_t i, float x, uint16_t noise) {
    switch (dtype) {
        case ORC_DT_BF16: ((uint16_t*)base)[i] = orc_sr_bf16(x, noise); break;
        case ORC_DT_F16: ((uint16_t*)base)[i] = orc_f32_to_f16_rne(x); break;
        case ORC_DT_F64: ((double*)base)[i] = (double)x; break;
        default: ((float*)base)[i] = x; break;
    }
}

/*
 * Whole-tensor step: upcast (adamw.py:160-170), update (:190-200), write back
 * (:204-222: bf16 targets are stochastically rounded, fp32 / fp16 / fp64 targets
 * take a plain copy_).  `elem_offset` is the index, within the logical tensor, of the
 * first element passed in (a multiple of 8), so that a tensor processed in
 * pieces draws the same noise as one processed whole.  dbg_* (optional) get
 * the fp32 values before rounding.  Returns 0, or a negative argument error.
 */
int orc_step_tensor(void* p, int p_dtype, const void* g, int g_dtype, void* m, int m_dtype,
                    void* v, int v_dtype, uint64_t numel, const orc_scalars* s, float clip_coef,
                    int noise_mode, const uint16_t* noise_p, const uint16_t* noise_m,
                    const uint16_t* noise_v, uint64_t seed, uint32_t step, uint32_t tensor_id,
                    uint64_t elem_offset, uint32_t flavour, float* dbg_p, float* dbg_m,
                    float* dbg_v) {
    if (p_dtype < 0 || p_dtype > 3 || m_dtype < 0 || m_dtype > 3 || v_dtype < 0 || v_dtype > 3) return -1;
    if (g_dtype < 0 || g_dtype > 3) return -1;
    if (elem_offset & 7u) return -2;
    if (noise_mode == ORC_NOISE_EXPLICIT) {
        if (p_dtype == ORC_DT_BF16 && !noise_p) return -3;
        if (m_dtype == ORC_DT_BF16 && !noise_m) return -3;
        if (v_dtype == ORC_DT_BF16 && !noise_v) return -3;
    }
    for (uint64_t i = 0; i < numel; ++i) {
        float pf = load_as_f32(p, p_dtype, i);
        float gf = load_as_f32(g, g_dtype, i);
        float mf = load_as_f32(m, m_dtype, i);
        float vf = load_as_f32(v, v_dtype, i);
        float po, mo, vo;
        orc_update_elem(pf, gf, mf, vf, s, clip_coef, flavour, &po, &mo, &vo);
        if (dbg_p) dbg_p[i] = po;
        if (dbg_m) dbg_m[i] = mo;
        if (dbg_v) dbg_v[i] = vo;
        uint64_t e = elem_offset + i;
        uint16_t np16 = 0, nm16 = 0, nv16 = 0;
        if (p_dtype == ORC_DT_BF16)
            np16 = noise_mode == ORC_NOISE_EXPLICIT ? noise_p[i] : orc_philox_noise(seed, step, tensor_id, 0, e);
        if (m_dtype == ORC_DT_BF16)
            nm16 = noise_mode == ORC_NOISE_EXPLICIT ? noise_m[i] : orc_philox_noise(seed, step, tensor_id, 1, e);
        if (v_dtype == ORC_DT_BF16)
            nv16 = noise_mode == ORC_NOISE_EXPLICIT ? noise_v[i] : orc_philox_noise(seed, step, tensor_id, 2, e);
        store_from_f32(p, p_dtype, i, po, np16);
        store_from_f32(m, m_dtype, i, mo, nm16);
        store_from_f32(v, v_dtype, i, vo, nv16);
    }
    return 0;
}

/*
 * copy_stochastic_(target, source, seed) (adamw.py:6-30) on its own: fp32
 * source -> bf16 target.  Explicit noise, or Philox with counter
 * (block_lo, block_hi, 3, 0) and key = seed ("which" 3 is never used by a step).
 */
void orc_sr_copy(uint16_t* target, const float* source, uint64_t numel, int noise_mode,
                 const uint16_t* noise, uint64_t seed) {
    for (uint64_t i = 0; i < numel; ++i) {
        uint16_t n = noise_mode == ORC_NOISE_EXPLICIT ? noise[i] : orc_philox_noise(seed, 0, 0, 3, i);
        target[i] = orc_sr_bf16(source[i], n);
    }
}

/*
 * Sum of squares of the unscaled gradient in float64: the yardstick for the
 * device-side reduction of the global-norm clip (semantics of
 * torch.nn.utils.clip_grad_norm_: total = sqrt(sum over tensors of ||g||^2),
 * coef = min(1, max_norm / (total + 1e-6))).  Not in the reference.
 */
double orc_grad_sumsq(const void* g, int g_dtype, uint64_t numel, float inv_loss_scale) {
    double acc = 0.0;
    for (uint64_t i = 0; i < numel; ++i) {
        float gf = load_as_f32(g, g_dtype, i);
        if (inv_loss_scale != 1.0f) gf = gf * inv_loss_scale;
        acc += (double)gf * (double)gf;
    }
    return acc;
}

/*
 * Row means for gradient centralization (adamw.py:179-184):
 *   grad.sub_(grad.mean(dim=1.., keepdim=True).mul_(c))
 * computed in float64 and rounded once (torch reduces in float32 with its own
 * summation order, so the mean is a yardstick within tolerance, not bit-exact).
 */
void orc_row_means(const void* g, int g_dtype, uint64_t rows, uint64_t row_len, float* out) {
    for (uint64_t r = 0; r < rows; ++r) {
        double acc = 0.0;
        for (uint64_t c = 0; c < row_len; ++c) acc += (double)load_as_f32(g, g_dtype, r * row_len + c);
        out[r] = (float)(acc / (double)row_len);
    }
}
