/*
 * CPU oracle for the ElixirOptimizer.step path -- TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic the reference performs
 * on the optimizer-step path.  It is the checker for the HIP kernels: only
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may build,
 * load or call it.  Nothing in the shipped package links or falls back to it.
 *
 * Build with -ffp-contract=off so that every fused multiply-add below is one
 * that is written out with fmaf().
 *
 * Reference files each function follows (paths relative to the reference tree):
 *   orc_overflow        elixir/chunk/core/chunk.py:214-216   (isinf.any | isnan.any)
 *   orc_sumsq           float64 brute force used to check the norm
 *   orc_l2norm_sq_ref   elixir/chunk/core/chunk.py:218-221   (float().norm(2).item()**2)
 *   orc_writeback       elixir/chunk/core/chunk.py:403-414   (shard.copy_(fp32 shard): RNE cast)
 *   orc_land            elixir/chunk/core/chunk.py:299,309-315,484-489  (reduce_buffer /= pg_size on
 *                       the device, then shard.copy_(reduce_buffer[shard_begin:shard_end]))
 *   orc_adam            elixir/wrapper/optimizer.py:211-216 -> inner optimizer step with
 *                       div_scale.  The inner optimizer (ColossalAI HybridAdam) is not part
 *                       of the reference tree; its published update rule is
 *                         g = float(g); if div_scale > 0: g /= div_scale
 *                         AdamW: m,v moments; p -= lr*(mhat/(sqrt(vhat)+eps) + wd*p)
 *                         L2:    g += wd*p first
 *                       The op order and the float64 host scalars follow torch.optim.Adam's
 *                       single-tensor path (torch/optim/adam.py:414-419, 457, 476, 528-545),
 *                       which is the semantics the parity target names.
 *
 * dtype codes: 0 = fp32, 1 = fp16, 2 = bf16.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---------- low-precision codecs, written on the bit patterns ---------- */

static inline float bits_to_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t f32_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* IEEE binary16 -> binary32, exact. */
static float half_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0x1Fu) /* inf / nan: keep payload in the top mantissa bits */
        return bits_to_f32(sign | 0x7F800000u | (man << 13));
    if (exp == 0) {
        if (man == 0)
            return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return (sign ? -v : v);
    }
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even, overflow to inf, NaN stays NaN. */
static uint16_t f32_to_half_bits(float f) {
    uint32_t x = f32_to_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax > 0x7F800000u) /* NaN -> quiet NaN */
        return (uint16_t)(sign | 0x7E00u);
    if (ax >= 0x47800000u) /* |f| >= 65536 (also inf) -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (ax >= 0x38800000u) { /* normal half range: |f| >= 2^-14 */
        uint32_t man = ax & 0x7FFFFFu;
        uint32_t exp = (ax >> 23) - 112u;
        uint32_t h = (exp << 10) | (man >> 13);
        uint32_t rem = man & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u)))
            h += 1u; /* carry may roll into the exponent, up to inf: that is right */
        return (uint16_t)(sign | h);
    }
    if (ax < 0x33000000u) /* |f| < 2^-25 -> rounds to zero (2^-25 itself ties to even = 0) */
        return sign;
    {
        /* subnormal half: result = round(|f| / 2^-24) as an integer in [0, 1024] */
        uint32_t e = ax >> 23;                       /* biased exponent, 102..112 */
        uint32_t man = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
        uint32_t shift = 126u - e;                   /* 14..24 */
        uint32_t h = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (h & 1u)))
            h += 1u;
        return (uint16_t)(sign | h);
    }
}

static float bf16_bits_to_f32(uint16_t b) { return bits_to_f32((uint32_t)b << 16); }

/* binary32 -> bfloat16, round to nearest even, NaN stays a quiet NaN. */
static uint16_t f32_to_bf16_bits(float f) {
    uint32_t x = f32_to_bits(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

float orc_lowp_to_f32(uint16_t bits, int dtype) {
    return dtype == 1 ? half_bits_to_f32(bits) : bf16_bits_to_f32(bits);
}

uint16_t orc_f32_to_lowp(float x, int dtype) {
    return dtype == 1 ? f32_to_half_bits(x) : f32_to_bf16_bits(x);
}

void orc_lowp_to_f32_array(const uint16_t *bits, float *out, int dtype, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i)
        out[i] = orc_lowp_to_f32(bits[i], dtype);
}

static inline float load_grad(const void *g, int dtype, uint64_t i) {
    if (dtype == 0)
        return ((const float *)g)[i];
    return orc_lowp_to_f32(((const uint16_t *)g)[i], dtype);
}

/* ---------- stage 2: overflow flag (chunk.py:214-216) ---------- */

int orc_overflow(const void *g, int dtype, uint64_t n) {
    int found = 0;
#pragma omp parallel for reduction(| : found) schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        float x = load_grad(g, dtype, (uint64_t)i);
        found |= (isinf(x) || isnan(x)) ? 1 : 0;
    }
    return found;
}

/* ---------- stage 3: squared L2 norm ---------- */

/* float64 brute force: sum of double(g)^2, accumulated in input order per thread. */
double orc_sumsq(const void *g, int dtype, uint64_t n) {
    double s = 0.0;
#pragma omp parallel for reduction(+ : s) schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        double x = (double)load_grad(g, dtype, (uint64_t)i);
        s += x * x;
    }
    return s;
}

/* chunk.py:218-221: the norm is an fp32 scalar; the square is taken in float64 on the host. */
double orc_l2norm_sq_ref(const void *g, int dtype, uint64_t n) {
    float nrm = (float)sqrt(orc_sumsq(g, dtype, n));
    return (double)nrm * (double)nrm;
}

/* ---------- stage 5: low-precision writeback (chunk.py:403-414) ---------- */

void orc_writeback(const float *master, void *lowp, int dtype, uint64_t n) {
    if (dtype == 0) {
        memcpy(lowp, master, n * sizeof(float));
        return;
    }
    uint16_t *out = (uint16_t *)lowp;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i)
        out[i] = orc_f32_to_lowp(master[i], dtype);
}

/* ---------- gradient landing (chunk.py:299, 309-315, 484-489) ---------- */

/*
 * dst[i] = cast_dd(src[i]) for i in [0, n).  With mul != 1 the element is first scaled the way an
 * in-place `payload /= pg_size` scales it on the device: the tensor is multiplied by the fp32
 * reciprocal of the host scalar (mul = 1.0f / pg_size) in fp32 and rounded back to the payload's
 * own type; the cast to the shard's type follows.  Equal types and mul == 1: the bits move
 * untouched (a copy does not canonicalise NaN payloads).  Allowed pairs: sd == dd, or sd == fp32.
 */
void orc_land(const void *src, int sd, void *dst, int dd, uint64_t n, float mul) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        if (sd == dd && mul == 1.0f) {
            if (sd == 0)
                ((uint32_t *)dst)[i] = ((const uint32_t *)src)[i];
            else
                ((uint16_t *)dst)[i] = ((const uint16_t *)src)[i];
            continue;
        }
        float v = load_grad(src, sd, (uint64_t)i);
        if (mul != 1.0f) {
            v = v * mul;
            if (sd != 0)
                v = orc_lowp_to_f32(orc_f32_to_lowp(v, sd), sd);
        }
        if (dd == 0)
            ((float *)dst)[i] = v;
        else
            ((uint16_t *)dst)[i] = orc_f32_to_lowp(v, dd);
    }
}

/* ---------- stages 1+4: unscale and Adam / AdamW ---------- */

/*
 * One optimizer step over n elements.  Scalars arrive as float64, exactly as the Python
 * optimizer holds them, and are narrowed to fp32 at the same places a tensor op would
 * narrow a Python scalar.
 *
 *   step            the step count AFTER the increment (1 for the first update)
 *   adamw_mode      1: decoupled decay  p *= 1 - lr*wd   (adam.py:414-417)
 *                   0: L2               g += wd*p         (adam.py:418-430)
 *   bias_correction 0 freezes both corrections at 1
 *   div_scale       <= 0 means "do not unscale" (the wrapper passes -1, optimizer.py:180-183)
 *   g == NULL       gradient is zero everywhere (the allocation step, optimizer.py:94-113)
 */
void orc_adam(const void *g, int g_dtype, float *p, float *m, float *v, uint64_t n, double lr,
              double beta1, double beta2, double eps, double weight_decay, int64_t step,
              int adamw_mode, int bias_correction, float div_scale) {
    double bc1 = 1.0, bc2 = 1.0;
    if (bias_correction) {
        bc1 = 1.0 - pow(beta1, (double)step);
        bc2 = 1.0 - pow(beta2, (double)step);
    }
    const double step_size = lr / bc1;
    const double bc2_sqrt = sqrt(bc2);

    const float decay_mul = (float)(1.0 - lr * weight_decay);
    const float wd_f = (float)weight_decay;
    const float w1 = (float)(1.0 - beta1);
    /* the coefficient of the second lerp form as torch's vectorised CPU kernel computes it: weight - 1
     * (not -(1 - weight): the two differ in the sign of zero when beta1 = 0, and with it the sign of a
     * zero exp_avg) */
    const float w1_minus_one = w1 - 1.0f;
    const float beta2_f = (float)beta2;
    const float omb2 = (float)(1.0 - beta2);
    const float bc2_sqrt_f = (float)bc2_sqrt;
    const float eps_f = (float)eps;
    const float neg_step = (float)(-step_size);

#pragma omp parallel for schedule(static)
    for (int64_t ii = 0; ii < (int64_t)n; ++ii) {
        uint64_t i = (uint64_t)ii;
        float gi = g ? load_grad(g, g_dtype, i) : 0.0f;
        if (div_scale > 0.0f)
            gi = gi / div_scale;
        float pi = p[i], mi = m[i], vi = v[i];

        if (weight_decay != 0.0) {
            if (adamw_mode)
                pi = pi * decay_mul;
            else
                gi = fmaf(wd_f, pi, gi); /* grad.add(param, alpha=wd): fused on the CPU kernels */
        }
        /* m.lerp_(g, 1-beta1): one fused multiply-add on the difference (adam.py:457) */
        float diff = gi - mi;
        if (w1 < 0.5f)
            mi = fmaf(w1, diff, mi);
        else
            mi = fmaf(w1_minus_one, diff, gi);
        /* v.mul_(beta2).addcmul_(g, g, value=1-beta2) (adam.py:476): the product v*beta2 is
         * rounded, (1-beta2)*g is rounded, and the last multiply-add is fused -- the form that
         * reproduces torch's CPU kernels bit for bit. */
        vi = fmaf(omb2 * gi, gi, vi * beta2_f);
        /* denom = sqrt(v)/sqrt(bc2) + eps; p += (-step_size*m)/denom (adam.py:528-545) */
        float denom = sqrtf(vi) / bc2_sqrt_f + eps_f;
        pi = pi + (neg_step * mi) / denom;

        p[i] = pi;
        m[i] = mi;
        v[i] = vi;
    }
}

/* Same step in float64 throughout, from fp32 inputs: the closed form the fp32 paths are
 * measured against.  Outputs are float64 arrays. */
void orc_adam_f64(const void *g, int g_dtype, const float *p, const float *m, const float *v,
                  double *p_out, double *m_out, double *v_out, uint64_t n, double lr, double beta1,
                  double beta2, double eps, double weight_decay, int64_t step, int adamw_mode,
                  int bias_correction, double div_scale) {
    double bc1 = 1.0, bc2 = 1.0;
    if (bias_correction) {
        bc1 = 1.0 - pow(beta1, (double)step);
        bc2 = 1.0 - pow(beta2, (double)step);
    }
    for (uint64_t i = 0; i < n; ++i) {
        double gi = g ? (double)load_grad(g, g_dtype, i) : 0.0;
        if (div_scale > 0.0)
            gi /= div_scale;
        double pi = p[i], mi = m[i], vi = v[i];
        if (weight_decay != 0.0) {
            if (adamw_mode)
                pi *= 1.0 - lr * weight_decay;
            else
                gi += weight_decay * pi;
        }
        mi = beta1 * mi + (1.0 - beta1) * gi;
        vi = beta2 * vi + (1.0 - beta2) * gi * gi;
        pi -= (lr / bc1) * mi / (sqrt(vi / bc2) + eps);
        p_out[i] = pi;
        m_out[i] = mi;
        v_out[i] = vi;
    }
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
