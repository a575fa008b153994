/*
 * TEST INFRASTRUCTURE — CPU restatement ("oracle") of the arithmetic of the
 * BMTrain hot path.  Nothing shipped links or calls this file; only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may use it, and only
 * as the checker.
 *
 * Every function is a scalar, single-threaded, plain-C restatement of one
 * reference routine, with the expression tree spelled out (this file must be
 * compiled with -ffp-contract=off so that the only fused multiply-adds are the
 * explicit fmaf() calls).  Citations are relative to the reference checkout.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   - half/bf16 converters: exhaustive over all 65,536 16-bit patterns and
 *     boundary/random fp32 values against torch's .half()/.bfloat16()/.float().
 *   - has_inf_nan: exhaustive over all 65,536 patterns per dtype against
 *     torch.isinf|torch.isnan.
 *   - adam_cpu_* (trees A3/A4 below): bit-for-bit against the reference's own
 *     compiled adam_cpu.hpp (oracle/_ref, and the committed vectors under
 *     tests/golden/ that were produced from it).
 *   - adam_gpu_bf16: same expression as the reference's scalar CPU bf16 path,
 *     so fp32 state is pinned bit-for-bit by the same compiled reference; the
 *     bf16 copy is pinned by torch's round-to-nearest-even .bfloat16().
 *   - adam_gpu_fp16: no compiled reference exists for it (CUDA only).  Pinned
 *     by the exact power-of-two scaling identity against adam_gpu_bf16, by
 *     torch.optim.AdamW in float64, and by the lr = 0 special case.
 *   - cross-entropy: torch log_softmax / cross_entropy in fp32 and a float64
 *     brute force; closed forms on tiny rows.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

/* ------------------------------------------------------------------------- */
/* 16-bit <-> fp32 converters                                                 */
/* ------------------------------------------------------------------------- */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE binary16 -> binary32, exact (subnormals, inf and NaN payload kept). */
static inline float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return u2f(f2u(v) | sign);
    }
    if (exp == 31) return u2f(sign | 0x7F800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even; NaN -> quiet NaN. */
static inline uint16_t float_to_half_rne(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);   /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);  /* >= 65536 (incl. inf) */
    if (a < 0x38800000u) {
        /* |f| < 2^-14: result is subnormal (or zero): round |f| / 2^-24 to integer, RNE */
        if (a < 0x33000000u) return sign;                    /* < 2^-25 -> 0 */
        uint32_t e = a >> 23;                                /* biased exponent, 102..112 */
        uint32_t m = (a & 0x7FFFFFu) | 0x800000u;            /* 24-bit significand */
        uint32_t shift = 126u - e;                           /* 14..24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    /* normal range: drop 13 mantissa bits with RNE; the carry may bump the exponent (up to inf) */
    uint32_t r = a - 0x38000000u;                            /* rebias 127 -> 15 */
    uint32_t q = r >> 13;
    uint32_t rem = r & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

static inline float bf16_to_float(uint16_t h) { return u2f((uint32_t)h << 16); }

/* binary32 -> bfloat16, round to nearest even (what a GPU store does,
 * adam_cuda.cu:66 `__float2bfloat16`); NaN -> quiet NaN. */
static inline uint16_t float_to_bf16_rne(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

/* binary32 -> bfloat16 by truncation (reference CPU path, adam_cpu.hpp:135-137). */
static inline uint16_t float_to_bf16_trunc(float f) { return (uint16_t)(f2u(f) >> 16); }

void oracle_half_to_float(int64_t n, const uint16_t *src, float *dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = half_to_float(src[i]);
}
/* adam_cpu.hpp:83-112,158-175 (`fp16_from_fp32_value_launcher`): RNE. */
void oracle_to_fp16_from_fp32(int64_t n, const float *src, uint16_t *dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = float_to_half_rne(src[i]);
}
/* adam_cpu.hpp:135-156 (`bf16_from_fp32_value_launcher`): truncation. */
void oracle_to_bf16_from_fp32(int64_t n, const float *src, uint16_t *dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = float_to_bf16_trunc(src[i]);
}
void oracle_to_bf16_from_fp32_rne(int64_t n, const float *src, uint16_t *dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = float_to_bf16_rne(src[i]);
}

/* ------------------------------------------------------------------------- */
/* has_inf_nan  (has_inf_nan.cu:35-67, 70-97, 101-138)                         */
/* out[0] = 1 iff some element is +-inf or NaN; otherwise out[0] is untouched  */
/* (sticky flag).  n <= 0 is a no-op (:108,:128).                              */
/* ------------------------------------------------------------------------- */
void oracle_has_inf_nan_fp16(int64_t n, const uint16_t *g, uint8_t *out) {
    if (n <= 0) return;
    for (int64_t i = 0; i < n; i++)
        if ((g[i] & 0x7FFFu) >= 0x7C00u) { out[0] = 1; return; }
}
void oracle_has_inf_nan_bf16(int64_t n, const uint16_t *g, uint8_t *out) {
    if (n <= 0) return;
    for (int64_t i = 0; i < n; i++)
        if ((g[i] & 0x7FFFu) >= 0x7F80u) { out[0] = 1; return; }
}

/* ------------------------------------------------------------------------- */
/* Adam                                                                        */
/* ------------------------------------------------------------------------- */

/* Tree selectors for the scalar expression.
 *   TREE_PLAIN  : every operation rounded separately, exactly as written.
 *   TREE_FMA_MV : m' = fma(b1, m, (1-b1)*g); v' = fma(b2, v, ((1-b2)*g)*g);
 *                 p' as written.
 *   TREE_FMA_MVP: as TREE_FMA_MV and p' = fma(-(lr*wd), p, p - upd).  This is
 *                 what g++ -O3 makes of the reference's scalar CPU loops (it
 *                 contracts every a*b+c it finds; measured bit-for-bit against
 *                 oracle/_ref over millions of elements), and it is the tree the
 *                 HIP kernels implement. */
enum { TREE_PLAIN = 0, TREE_FMA_MV = 1, TREE_FMA_MVP = 2 };

/* One element of the "unscaled state" update shared by the GPU bf16 kernel
 * (adam_cuda.cu:60-64) and the scalar CPU loops (adam_cpu.hpp:207-218,265-276):
 *   g  = g16 / scale
 *   m' = b1*m + (1-b1)*g
 *   v' = b2*v + (1-b2)*g*g
 *   p' = p - lr*m'/bc1/(sqrtf(v'/bc2)+eps) - lr*wd*p          (old p in the decay term)
 */
static inline void adam_scalar_elem(float g, float *m, float *v, float *p,
                                    float b1, float b2, float eps, float lr, float wd,
                                    float bc1, float bc2, int tree,
                                    float *delta /* may be NULL */) {
    float omb1 = 1.0f - b1, omb2 = 1.0f - b2;
    float mm, vv;
    if (tree != TREE_PLAIN) {
        mm = fmaf(b1, *m, omb1 * g);
        vv = fmaf(b2, *v, (omb2 * g) * g);
    } else {
        mm = (b1 * *m) + (omb1 * g);
        vv = (b2 * *v) + ((omb2 * g) * g);
    }
    float pp = *p;
    float den = sqrtf(vv / bc2) + eps;
    if (delta) *delta = ((mm / bc1) / den) + (wd * pp);   /* adam_cpu.hpp:213-217 */
    float upd = ((lr * mm) / bc1) / den;
    float np = (tree == TREE_FMA_MVP) ? fmaf(-(lr * wd), pp, pp - upd)
                                      : (pp - upd) - ((lr * wd) * pp);
    *m = mm; *v = vv; *p = np;
}

/* GPU bf16 kernel, adam_cuda.cu:39-72 (launcher :103-126).  bf16 copy is RNE. */
void oracle_adam_gpu_bf16(int64_t n, float *p32, uint16_t *p16, const uint16_t *g16,
                          float *m, float *v, float b1, float b2, float eps, float lr,
                          float scale, float wd, float bc1, float bc2, int tree) {
    for (int64_t i = 0; i < n; i++) {
        float g = bf16_to_float(g16[i]) / scale;
        adam_scalar_elem(g, &m[i], &v[i], &p32[i], b1, b2, eps, lr, wd, bc1, bc2, tree, NULL);
        p16[i] = float_to_bf16_rne(p32[i]);
    }
}

/* GPU fp16 kernel, adam_cuda.cu:8-37 (launcher :76-101).  The moments are kept
 * multiplied by `scale`:
 *   g  = float(g16)                          (not divided)
 *   m' = b1*float(m16) + (1-b1)*g
 *   v' = b2*v + (1-b2)*g*g/scale
 *   p' = p - lr*m'/bc1/(sqrtf(v'*scale/bc2) + eps*scale) - lr*wd*p
 *   store half(p'), p', v', half(m')         (the update uses the un-rounded m')
 */
void oracle_adam_gpu_fp16(int64_t n, float *p32, uint16_t *p16, const uint16_t *g16,
                          uint16_t *m16, float *v, float b1, float b2, float eps, float lr,
                          float scale, float wd, float bc1, float bc2, int tree) {
    float omb1 = 1.0f - b1, omb2 = 1.0f - b2;
    for (int64_t i = 0; i < n; i++) {
        float g = half_to_float(g16[i]);
        float mm, vv;
        if (tree != TREE_PLAIN) {
            mm = fmaf(b1, half_to_float(m16[i]), omb1 * g);
            vv = fmaf(b2, v[i], ((omb2 * g) * g) / scale);
        } else {
            mm = (b1 * half_to_float(m16[i])) + (omb1 * g);
            vv = (b2 * v[i]) + (((omb2 * g) * g) / scale);
        }
        float pp = p32[i];
        float den = sqrtf((vv * scale) / bc2) + (eps * scale);
        float upd = ((lr * mm) / bc1) / den;
        float np = (tree == TREE_FMA_MVP) ? fmaf(-(lr * wd), pp, pp - upd)
                                          : (pp - upd) - ((lr * wd) * pp);
        p16[i] = float_to_half_rne(np);
        p32[i] = np;
        v[i] = vv;
        m16[i] = float_to_half_rne(mm);
    }
}

/* Vector-lane tree of the AVX / AVX-512 CPU loops (adam_cpu.hpp:353-382, 454-486):
 *   g  = g16 / scale
 *   m' = fma(b1, m, (1-b1)*g)
 *   v' = fma(b2, v, (1-b2)*(g*g))           (g*g first, unlike the scalar loop)
 *   p1 = fma(-lr, wd*p, p)
 *   p' = fma(-lr, (m'/bc1)/(sqrt(v'/bc2)+eps), p1)
 */
static inline void adam_vector_elem(float g, float *m, float *v, float *p,
                                    float b1, float b2, float eps, float lr, float wd,
                                    float bc1, float bc2, float *delta) {
    float omb1 = 1.0f - b1, omb2 = 1.0f - b2;
    float mm = fmaf(b1, *m, omb1 * g);
    float vv = fmaf(b2, *v, omb2 * (g * g));
    float pp = *p;
    float q = (mm / bc1) / (sqrtf(vv / bc2) + eps);
    if (delta) *delta = q + (wd * pp);
    float p1 = fmaf(-lr, wd * pp, pp);
    float np = fmaf(-lr, q, p1);
    *m = mm; *v = vv; *p = np;
}

/* CPU offload Adam, fp16 gradients: adam_cpu_fp16_launcher (adam_cpu.hpp:504-533)
 * dispatching to adam_cpu_0 (:183-239, level 0), adam_cpu_1 (:299-398, level 1,
 * 8 lanes) or adam_cpu_2 (:400-502, level 2, 16 lanes).  `threads` reproduces
 * parallel_for (:42-80): chunk = max(ceil(n/threads),1), thread t owns
 * [t*chunk, min((t+1)*chunk, n)); inside a chunk whole vectors take the vector
 * tree and the remaining < lanes elements take the scalar tree.
 * delta_info (may be NULL) = {mean, var, sum, sumsq} of the per-element update
 * (:226-238); its float accumulation order here is chunk by chunk, element by
 * element, which the threaded reference does not fix — compare it with a
 * tolerance, not bit-for-bit. */
void oracle_adam_cpu_fp16(int64_t n, float *p32, uint16_t *p16, float *delta_info,
                          const uint16_t *g16, float *m, float *v,
                          float b1, float b2, float eps, float lr, float scale, float wd,
                          float bc1, float bc2, int level, int64_t threads, int scalar_tree) {
    int64_t lanes = level == 0 ? 1 : (level == 1 ? 8 : 16);
    if (threads < 1) threads = 1;
    int64_t chunk = (n + threads - 1) / threads;
    if (chunk < 1) chunk = 1;
    float sum = 0.f, sumsq = 0.f;
    for (int64_t t = 0; t < threads; t++) {
        int64_t lo = t * chunk; if (lo > n) lo = n;
        int64_t hi = (t + 1) * chunk; if (hi > n) hi = n;
        float s_i = 0.f, q_i = 0.f;
        int64_t j = lo;
        if (lanes > 1) {
            for (; j + lanes <= hi; j += lanes) {
                float d[16];
                for (int64_t k = 0; k < lanes; k++) {
                    int64_t i = j + k;
                    float g = half_to_float(g16[i]) / scale;
                    adam_vector_elem(g, &m[i], &v[i], &p32[i], b1, b2, eps, lr, wd, bc1, bc2,
                                     delta_info ? &d[k] : NULL);
                    p16[i] = float_to_half_rne(p32[i]);
                }
                if (delta_info) for (int64_t k = 0; k < lanes; k++) { s_i += d[k]; q_i += d[k] * d[k]; }
            }
        }
        for (int64_t i = j; i < hi; i++) {
            float g = half_to_float(g16[i]) / scale;
            float d;
            adam_scalar_elem(g, &m[i], &v[i], &p32[i], b1, b2, eps, lr, wd, bc1, bc2,
                             scalar_tree, delta_info ? &d : NULL);
            p16[i] = float_to_half_rne(p32[i]);
            if (delta_info) { s_i += d; q_i += d * d; }
        }
        sum += s_i; sumsq += q_i;
    }
    if (delta_info) {
        delta_info[0] = sum / n;
        delta_info[1] = sumsq / n - sum * sum / ((float)n * (float)n);
        delta_info[2] = sum;
        delta_info[3] = sumsq;
    }
}

/* CPU offload Adam, bf16 gradients: adam_cpu_bf16_launcher (adam_cpu.hpp:535-557)
 * -> adam_cpu_bf16_0 (:241-297): always the scalar tree; bf16 copy truncated. */
void oracle_adam_cpu_bf16(int64_t n, float *p32, uint16_t *p16, float *delta_info,
                          const uint16_t *g16, float *m, float *v,
                          float b1, float b2, float eps, float lr, float scale, float wd,
                          float bc1, float bc2, int64_t threads, int scalar_tree) {
    (void)threads; /* every element takes the same tree: chunking cannot matter */
    float sum = 0.f, sumsq = 0.f;
    for (int64_t i = 0; i < n; i++) {
        float g = bf16_to_float(g16[i]) / scale;
        float d;
        adam_scalar_elem(g, &m[i], &v[i], &p32[i], b1, b2, eps, lr, wd, bc1, bc2,
                         scalar_tree, delta_info ? &d : NULL);
        p16[i] = float_to_bf16_trunc(p32[i]);
        if (delta_info) { sum += d; sumsq += d * d; }
    }
    if (delta_info) {
        delta_info[0] = sum / n;
        delta_info[1] = sumsq / n - sum * sum / ((float)n * (float)n);
        delta_info[2] = sum;
        delta_info[3] = sumsq;
    }
}

/* ------------------------------------------------------------------------- */
/* Cross-entropy                                                               */
/* ------------------------------------------------------------------------- */

/* Block sum in the reference's order (reduce.cuh:55-83 `block_allreduce_sum`
 * with 1024 threads, 32-lane warps): partial[t] holds thread t's strided sum;
 * each warp folds with offsets 16,8,4,2,1; the 32 warp results fold the same way. */
static float ref_block_sum_1024(float *partial /* 1024, clobbered */) {
    float warp[32];
    for (int w = 0; w < 32; w++) {
        float *x = partial + 32 * w;
        for (int off = 16; off > 0; off >>= 1)
            for (int l = 0; l < off; l++) x[l] += x[l + off];
        warp[w] = x[0];
    }
    for (int off = 16; off > 0; off >>= 1)
        for (int l = 0; l < off; l++) warp[l] += warp[l + off];
    return warp[0];
}

typedef float (*cvt_in_fn)(uint16_t);
typedef uint16_t (*cvt_out_fn)(float);

/* cross_entropy.cu:9-43 (fp16) / :63-101 (bf16):
 *   M = fmaxf(max_i x_i, -1e6)           (fmaxf ignores NaN operands)
 *   S = sum_i expf(x_i - M) + 1e-10       (sum: stride-1024 partials, then tree;
 *                                          the 1e-10 literal is a double, :28,:86)
 *   softmax_i = to16(expf(x_i - M) / S)
 *   out_r = t_r != ignore ? -x[t_r] + M + logf(S) : 0
 * With m == 0 the reference would issue an invalid launch; here it is a no-op. */
static void ce_forward(int64_t m, int64_t n, const uint16_t *x, const int32_t *target,
                       uint16_t *softmax, float *out, int32_t ignore_index,
                       cvt_in_fn in, cvt_out_fn outc) {
    float partial[1024];
    for (int64_t r = 0; r < m; r++) {
        const uint16_t *row = x + r * n;
        float mx = -INFINITY;
        for (int64_t i = 0; i < n; i++) mx = fmaxf(in(row[i]), mx);
        mx = fmaxf(mx, -1e6f);
        for (int t = 0; t < 1024; t++) {
            float s = 0.f;
            for (int64_t i = t; i < n; i += 1024) s += expf(in(row[i]) - mx);
            partial[t] = s;
        }
        float S = (float)((double)ref_block_sum_1024(partial) + 1e-10);
        for (int64_t i = 0; i < n; i++) softmax[r * n + i] = outc(expf(in(row[i]) - mx) / S);
        if (target[r] != ignore_index)
            out[r] = (-in(row[target[r]]) + mx) + logf(S);
        else
            out[r] = 0.f;
    }
}
void oracle_ce_forward_fp16(int64_t m, int64_t n, const uint16_t *x, const int32_t *target,
                            uint16_t *softmax, float *out, int32_t ignore_index) {
    ce_forward(m, n, x, target, softmax, out, ignore_index, half_to_float, float_to_half_rne);
}
void oracle_ce_forward_bf16(int64_t m, int64_t n, const uint16_t *x, const int32_t *target,
                            uint16_t *softmax, float *out, int32_t ignore_index) {
    ce_forward(m, n, x, target, softmax, out, ignore_index, bf16_to_float, float_to_bf16_rne);
}

/* The forward expression of cross_entropy.cu:17-42 evaluated in other ways that are equally faithful to the
 * source: nothing in it fixes which expf the compiler links or how many lanes a warp has.
 *   exp_kind 0: this host's libm expf (what ce_forward above uses);
 *            1: exp in double precision, rounded to float (the correctly rounded value but for double rounding);
 *            2: that value moved by one float ulp down, not at all, not at all or up, chosen by a fixed hash of
 *               the argument's bits: a stand-in for any expf that is accurate to 1 ulp.  The reference's own expf
 *               is the CUDA library's, whose documented maximum error is 2 ulp, so an evaluation that is 1 ulp
 *               away from this host's libm on some arguments is as faithful to the source as libm's;
 *            3: the same with steps of -2, -1, 0, 0, 0, 0, +1, +2 ulps: the full width that documented bound allows.
 *   sum_kind 0: reduce.cuh's order on 32-lane warps (ce_forward above);
 *            1: the same source on 64-lane wavefronts: 1024 strided partials, each wave folds with offsets
 *               32..1, the 16 wave results fold with offsets 8..1;
 *            2: the sum in double precision, rounded once.
 * Used by tests to measure how far two faithful evaluations of the reference lie apart in 16-bit units. */
static float alt_exp(float t, int exp_kind) {
    if (exp_kind == 0) return expf(t);
    float e = (float)exp((double)t);
    if (exp_kind >= 2 && e > 0.f && isfinite(e)) {
        uint32_t u, h;
        memcpy(&u, &t, 4);
        h = u * 2654435761u;
        if (exp_kind == 2) {
            h >>= 30;
            if (h == 0) e = nextafterf(e, 0.f);
            else if (h == 3) e = nextafterf(e, INFINITY);
        } else {
            h >>= 29;
            if (h <= 1) e = nextafterf(e, 0.f);
            if (h == 0) e = nextafterf(e, 0.f);
            if (h >= 6) e = nextafterf(e, INFINITY);
            if (h == 7) e = nextafterf(e, INFINITY);
        }
    }
    return e;
}
void oracle_alt_exp(int64_t n, const float *t, float *out, int32_t exp_kind) {
    for (int64_t i = 0; i < n; i++) out[i] = alt_exp(t[i], exp_kind);
}
static float block_sum_wave64(float *partial /* 1024, clobbered */) {
    float wave[16];
    for (int w = 0; w < 16; w++) {
        float *x = partial + 64 * w;
        for (int off = 32; off > 0; off >>= 1)
            for (int l = 0; l < off; l++) x[l] += x[l + off];
        wave[w] = x[0];
    }
    for (int off = 8; off > 0; off >>= 1)
        for (int l = 0; l < off; l++) wave[l] += wave[l + off];
    return wave[0];
}
static void ce_forward_alt(int64_t m, int64_t n, const uint16_t *x, const int32_t *target, uint16_t *softmax,
                           float *out, int32_t ignore_index, cvt_in_fn in, cvt_out_fn outc, int exp_kind, int sum_kind) {
    float partial[1024];
    for (int64_t r = 0; r < m; r++) {
        const uint16_t *row = x + r * n;
        float mx = -INFINITY;
        for (int64_t i = 0; i < n; i++) mx = fmaxf(in(row[i]), mx);
        mx = fmaxf(mx, -1e6f);
        float sum;
        if (sum_kind == 2) {
            double acc = 0.0;
            for (int64_t i = 0; i < n; i++) acc += (double)alt_exp(in(row[i]) - mx, exp_kind);
            sum = (float)acc;
        } else {
            for (int t = 0; t < 1024; t++) {
                float s = 0.f;
                for (int64_t i = t; i < n; i += 1024) s += alt_exp(in(row[i]) - mx, exp_kind);
                partial[t] = s;
            }
            sum = sum_kind == 1 ? block_sum_wave64(partial) : ref_block_sum_1024(partial);
        }
        float S = (float)((double)sum + 1e-10);
        for (int64_t i = 0; i < n; i++) softmax[r * n + i] = outc(alt_exp(in(row[i]) - mx, exp_kind) / S);
        out[r] = target[r] != ignore_index ? (-in(row[target[r]]) + mx) + logf(S) : 0.f;
    }
}
void oracle_ce_forward_alt_fp16(int64_t m, int64_t n, const uint16_t *x, const int32_t *target, uint16_t *softmax,
                                float *out, int32_t ignore_index, int32_t exp_kind, int32_t sum_kind) {
    ce_forward_alt(m, n, x, target, softmax, out, ignore_index, half_to_float, float_to_half_rne, exp_kind, sum_kind);
}
void oracle_ce_forward_alt_bf16(int64_t m, int64_t n, const uint16_t *x, const int32_t *target, uint16_t *softmax,
                                float *out, int32_t ignore_index, int32_t exp_kind, int32_t sum_kind) {
    ce_forward_alt(m, n, x, target, softmax, out, ignore_index, bf16_to_float, float_to_bf16_rne, exp_kind, sum_kind);
}

/* cross_entropy.cu:46-60 (fp16) / :104-121 (bf16): in place on the stored softmax,
 *   x_i = to16( i == t_r ? (x_i - 1) * v : x_i * v ),  v = grad_output[r].
 * ignore_index is not read: an ignored row (t_r = -100) simply never matches i. */
static void ce_backward(int64_t m, int64_t n, const float *grad_output, const int32_t *target,
                        uint16_t *x, cvt_in_fn in, cvt_out_fn outc) {
    for (int64_t r = 0; r < m; r++) {
        int32_t t = target[r];
        float v = grad_output[r];
        for (int64_t i = 0; i < n; i++) {
            float s = in(x[r * n + i]);
            x[r * n + i] = outc(i == (int64_t)t ? (s - 1.f) * v : s * v);
        }
    }
}
void oracle_ce_backward_fp16(int64_t m, int64_t n, const float *grad_output,
                             const int32_t *target, uint16_t *x, int32_t ignore_index) {
    (void)ignore_index;
    ce_backward(m, n, grad_output, target, x, half_to_float, float_to_half_rne);
}
void oracle_ce_backward_bf16(int64_t m, int64_t n, const float *grad_output,
                             const int32_t *target, uint16_t *x, int32_t ignore_index) {
    (void)ignore_index;
    ce_backward(m, n, grad_output, target, x, bf16_to_float, float_to_bf16_rne);
}

/* cross_entropy.cu:124-164 `fused_sumexp_*`: sum_i expf(x_i - max_r), reference
 * summation order, no 1e-10 term. */
static void sumexp(int64_t m, int64_t n, const uint16_t *x, const float *gmax, float *gsum,
                   cvt_in_fn in) {
    float partial[1024];
    for (int64_t r = 0; r < m; r++) {
        float mx = gmax[r];
        for (int t = 0; t < 1024; t++) {
            float s = 0.f;
            for (int64_t i = t; i < n; i += 1024) s += expf(in(x[r * n + i]) - mx);
            partial[t] = s;
        }
        gsum[r] = ref_block_sum_1024(partial);
    }
}
void oracle_fused_sumexp_fp16(int64_t m, int64_t n, const uint16_t *x, const float *gmax, float *gsum) {
    sumexp(m, n, x, gmax, gsum, half_to_float);
}
void oracle_fused_sumexp_bf16(int64_t m, int64_t n, const uint16_t *x, const float *gmax, float *gsum) {
    sumexp(m, n, x, gmax, gsum, bf16_to_float);
}

/* cross_entropy.cu:167-199 `fused_softmax_inplace_*`: x_i = to16(expf(x_i - max_r) / sum_r). */
static void softmax_inplace(int64_t m, int64_t n, uint16_t *x, const float *gmax, const float *gsum,
                            cvt_in_fn in, cvt_out_fn outc) {
    for (int64_t r = 0; r < m; r++)
        for (int64_t i = 0; i < n; i++)
            x[r * n + i] = outc(expf(in(x[r * n + i]) - gmax[r]) / gsum[r]);
}
void oracle_fused_softmax_inplace_fp16(int64_t m, int64_t n, uint16_t *x, const float *gmax, const float *gsum) {
    softmax_inplace(m, n, x, gmax, gsum, half_to_float, float_to_half_rne);
}
void oracle_fused_softmax_inplace_bf16(int64_t m, int64_t n, uint16_t *x, const float *gmax, const float *gsum) {
    softmax_inplace(m, n, x, gmax, gsum, bf16_to_float, float_to_bf16_rne);
}

/* ------------------------------------------------------------------------- */
/* Gradient statistics                                                         */
/* ------------------------------------------------------------------------- */
/* What OptimManager.clip_grad_norm accumulates per tensor for norm_type 2
 * (optim_manager.py:186-190: `g.float().norm(2) ** 2`), i.e. sum_i g_i^2, here in
 * double precision; the overflow flag is oracle_has_inf_nan_*. */
double oracle_grad_sumsq_fp16(int64_t n, const uint16_t *g) {
    double s = 0.0;
    for (int64_t i = 0; i < n; i++) { double x = (double)half_to_float(g[i]); s += x * x; }
    return s;
}
double oracle_grad_sumsq_bf16(int64_t n, const uint16_t *g) {
    double s = 0.0;
    for (int64_t i = 0; i < n; i++) { double x = (double)bf16_to_float(g[i]); s += x * x; }
    return s;
}
