/*
 * CPU oracle for the DNNKernels dense-contraction path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's
 * KernelAbstractions-CPU forms (the scalar kernels every plan declines to on a
 * device without cooperative matrices).  It is the checker the HIP kernels are
 * compared against and the timed CPU baseline; nothing in the product path may
 * call it.  Each function cites the reference source it follows
 * (paths relative to DNNKernels/src/).
 *
 * Layout convention (reference safetensors.jl:7-12, graph.jl:161-167): a Julia
 * column-major array (a,b,c,d) is the row-major C array [d][c][b][a].  All
 * "element strides" below are in elements, not bytes.
 *
 * Parity pinning (what fixes each function besides its own formula):
 *   orc_erf / gelu       A&S 7.1.26 closed form vs libm erf in fp64, and the
 *                        reference's own thresholds (test_activation_width.jl:70-107)
 *   orc_gemm_f16         fp64 matmul over the fp16-rounded inputs (numpy), the
 *                        reference's criterion (tools/gemm_bench.jl:134-148)
 *   orc_sdpa_*           textbook softmax(QK^T)V in fp64 (test_flash.jl:13-24),
 *                        torch.nn.functional.scaled_dot_product_attention (fp32),
 *                        row-sum / masked-row / split-merge invariants
 *   orc_conv2d_f16       torch.nn.functional.conv2d in fp32/fp64; im2col map by
 *                        brute force on tiny shapes
 *   orc_convtranspose2d_f16  torch.nn.functional.conv_transpose2d in fp64 (stride, padding,
 *                        dilation, output_padding, groups) and the pixel-shuffle identity of
 *                        the non-overlapping case (conv.jl:204-222)
 *   orc_layernorm_f16    torch.nn.functional.layer_norm in fp32
 *   orc_softmax_f16      numpy float64 exp / sum (rows sum to 1, shift invariance, a row of
 *                        -inf gives zeros); composed with two orc_gemm_f16 it reproduces
 *                        orc_sdpa_threepass (the two-GEMM attention, attention.jl:675-705)
 *   unpinned             bit-level accumulation order of Lava.coopmat_gemm!/gemv!
 *                        (third-party, source absent); irrelevant at the 1e-2 /
 *                        cosine 0.9999 gate.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#if defined(__F16C__)
#include <immintrin.h>
#endif
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ fp16 <-> fp32 */

static inline float h2f(uint16_t h) {
#if defined(__F16C__)
    return _cvtsh_ss(h);
#else
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu, u;
    if (e == 0) {
        if (m == 0) u = s;
        else { int sh = 0; while (!(m & 0x400u)) { m <<= 1; sh++; }
               u = s | ((uint32_t)(113 - sh) << 23) | ((m & 0x3ffu) << 13); }
    } else if (e == 31) u = s | 0x7f800000u | (m << 13);
    else u = s | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &u, 4); return f;
#endif
}

static inline uint16_t f2h(float f) {          /* round to nearest even */
#if defined(__F16C__)
    return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
#else
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t s = (x >> 16) & 0x8000u; x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(s | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
    if (x >= 0x477ff000u) return (uint16_t)(s | 0x7c00u);      /* rounds to inf */
    if (x < 0x38800000u) {                                     /* subnormal / zero */
        if (x < 0x33000000u) return (uint16_t)s;
        int e = (int)(x >> 23); uint32_t m = (x & 0x7fffffu) | 0x800000u;
        int sh = 126 - e;                                      /* 14..24 */
        uint32_t r = m >> sh, rem = m & ((1u << sh) - 1), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1))) r++;
        return (uint16_t)(s | r);
    }
    uint32_t r = x - 0x38000000u, rem = r & 0x1fffu; r >>= 13;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) r++;
    return (uint16_t)(s | r);
#endif
}

ORC_API void orc_f16_to_f32(float *o, const uint16_t *a, int64_t n) { for (int64_t i = 0; i < n; i++) o[i] = h2f(a[i]); }
ORC_API void orc_f32_to_f16(uint16_t *o, const float *a, int64_t n) { for (int64_t i = 0; i < n; i++) o[i] = f2h(a[i]); }
ORC_API int orc_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ portable seeded inputs
 * Counter-based SplitMix64 -> Box-Muller.  Element i of a tensor with seed s
 * depends on (s, i) only, so a tensor's values do not depend on how it is
 * generated (threads, chunking).  This is the one generator every test and the
 * benchmark use: "identical seeded inputs" means this function. */
static inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline double rng_u01(uint64_t seed, uint64_t ctr) {   /* (0,1] */
    uint64_t z = mix64(seed * 0xD1342543DE82EF95ull + (ctr + 1) * 0x9E3779B97F4A7C15ull);
    return (double)((z >> 11) + 1) * (1.0 / 9007199254740992.0);
}
static inline double rng_normal(uint64_t seed, uint64_t i) {
    double u1 = rng_u01(seed, 2 * i), u2 = rng_u01(seed, 2 * i + 1);
    return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
}
ORC_API void orc_randn_f32(float *o, int64_t n, uint64_t seed, double mean, double std) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) o[i] = (float)(mean + std * rng_normal(seed, (uint64_t)i));
}
ORC_API void orc_randn_f16(uint16_t *o, int64_t n, uint64_t seed, double mean, double std) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) o[i] = f2h((float)(mean + std * rng_normal(seed, (uint64_t)i)));
}
ORC_API void orc_uniform_f16(uint16_t *o, int64_t n, uint64_t seed, double lo, double hi) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) o[i] = f2h((float)(lo + (hi - lo) * rng_u01(seed, (uint64_t)i)));
}

/* ------------------------------------------------------------------ activations
 * ops.jl:161-169 (erf: Abramowitz & Stegun 7.1.26 evaluated in fp32),
 * ops.jl:1665-1669 (geluexact), ops.jl:1677-1682 (gelutanh), ops.jl:1683 (relu_epi).
 * Each takes the fp16 value, evaluates in fp32, rounds once. */
static inline float erf_as(float x) {
    float a = fabsf(x);
    float t = 1.0f / (1.0f + 0.3275911f * a);
    float y = 1.0f - (((((1.061405429f * t - 1.453152027f) * t) + 1.421413741f) * t - 0.284496736f) * t + 0.254829592f) * t * expf(-a * a);
    return x < 0.0f ? -y : y;
}
static inline float gelu_exact(float x) { return 0.5f * x * (1.0f + erf_as(x / sqrtf(2.0f))); }
static inline float gelu_tanh(float x)  { return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x))); }

enum { EPI_NONE = 0, EPI_GELU_ERF = 1, EPI_GELU_TANH = 2, EPI_RELU = 3 };

static inline float apply_epi(float v, int epi) {
    switch (epi) {
    case EPI_GELU_ERF:  return gelu_exact(v);
    case EPI_GELU_TANH: return gelu_tanh(v);
    case EPI_RELU:      return v > 0.0f ? v : 0.0f;
    default:            return v;
    }
}
ORC_API float orc_erf(float x) { return erf_as(x); }
/* out[i] = fp16(f(fp32(in[i]))), kind: 0 erf, 1 gelu exact, 2 gelu tanh, 3 relu */
ORC_API void orc_act_f16(uint16_t *o, const uint16_t *a, int64_t n, int kind) {
    for (int64_t i = 0; i < n; i++) {
        float x = h2f(a[i]);
        o[i] = f2h(kind == 0 ? erf_as(x) : apply_epi(x, kind));
    }
}

/* ------------------------------------------------------------------ GEMM
 * kernels/extern/matmul.jl:17-27 (mm2): acc = fp32(bias), muladd over k in
 * fp32, ONE rounding to the output type; matmul.jl:210-214: the activation is
 * applied to the *rounded* value.  Row-major restatement of the reversed
 * layout (ops.jl:1345-1356):  Y[T][F] = X[T][K] . W + bias[F].
 *   w_layout 0: W is [K][F] (the reference's hoisted weight, hoistcasts.jl:47-112)
 *   w_layout 1: W is [F][K]
 *   bias_mode 0 none, 1 per output column (F), 2 per output row (T)
 *   out_f32   0: Y is fp16 (rounded, then epi, then optional residual add rounded
 *                again: the graph's separate add.Tensor, ops.jl:186-197); 1: Y is fp32
 * Batched (mm3, matmul.jl:29-39): batch strides in elements, 0 = shared. */
ORC_API void orc_gemm_f16(void *Y, const uint16_t *X, const uint16_t *W, const uint16_t *bias,
                          const uint16_t *residual,
                          int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                          int w_layout, int bias_mode, int epi, int out_f32,
                          int64_t nbatch, int64_t sY, int64_t sX, int64_t sW) {
    if (nbatch < 1) nbatch = 1;
    for (int64_t b = 0; b < nbatch; b++) {
        const uint16_t *Xb = X + b * sX, *Wb = W + b * sW;
        #pragma omp parallel for schedule(static)
        for (int64_t t = 0; t < T; t++) {
            float *xr = (float *)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
            for (int64_t k = 0; k < K; k++) xr[k] = h2f(Xb[t * ldX + k]);
            for (int64_t f = 0; f < F; f++) {
                float acc = bias_mode == 1 ? h2f(bias[f]) : bias_mode == 2 ? h2f(bias[t]) : 0.0f;
                if (w_layout == 0) for (int64_t k = 0; k < K; k++) acc = fmaf(xr[k], h2f(Wb[k * ldW + f]), acc);
                else               for (int64_t k = 0; k < K; k++) acc = fmaf(xr[k], h2f(Wb[f * ldW + k]), acc);
                if (out_f32) {
                    ((float *)Y)[b * sY + t * ldY + f] = apply_epi(acc, epi);
                } else {
                    uint16_t y = f2h(apply_epi(h2f(f2h(acc)), epi));
                    if (residual) y = f2h(h2f(y) + h2f(residual[b * sY + t * ldY + f]));
                    ((uint16_t *)Y)[b * sY + t * ldY + f] = y;
                }
            }
            free(xr);
        }
    }
}

/* ------------------------------------------------------------------ attention
 * Operands are (E, L, H, B) with element strides (sE, sL, sH, sB)
 * (attention.jl:1-22).  out is dense (E, Lq, H, B).
 * bias (optional) is laid out (Lk, Lq, H, B) with element strides; a stride of
 * 0 broadcasts that axis (attention.jl:55-59, launch.jl:72-75).  bias_f32
 * selects its element type.  kv_len (optional, int32[B]) excludes keys
 * >= kv_len[b]: equivalent to the decoder's additive 0 / finfo.min mask
 * (tools/export_whisper_decoder.py:158-165). */
typedef struct { int64_t e, l, h, b; } str4;

static inline float bias_at(const void *bias, int bias_f32, const int64_t *bs, int64_t lk, int64_t lq, int64_t h, int64_t b) {
    int64_t o = lk * bs[0] + lq * bs[1] + h * bs[2] + b * bs[3];
    return bias_f32 ? ((const float *)bias)[o] : h2f(((const uint16_t *)bias)[o]);
}

/* Three-pass form, attention.jl:46-112 and 790-834: scores are stored in the
 * operand type (fp16) after scale and bias; the softmax stores fp16(exp(s-m))
 * UNNORMALISED and sums the unrounded exponentials in fp32; apply accumulates
 * fp32(p16)*v in fp32 and divides by the sum.  An all-masked row (max not
 * finite) gives zeros, sum 1. */
ORC_API void orc_sdpa_threepass_f16(void *out, int out_f32,
                                    const uint16_t *q, const int64_t *qs,
                                    const uint16_t *k, const int64_t *ks,
                                    const uint16_t *v, const int64_t *vs,
                                    const void *bias, int bias_f32, const int64_t *bs,
                                    const int32_t *kv_len,
                                    int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale) {
    #pragma omp parallel for collapse(3) schedule(static)
    for (int64_t b = 0; b < B; b++)
    for (int64_t h = 0; h < H; h++)
    for (int64_t lq = 0; lq < Lq; lq++) {
        int64_t n = Lk > 0 ? Lk : 1;
        uint16_t *sc = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)n);
        int64_t klim = kv_len ? (kv_len[b] < Lk ? kv_len[b] : Lk) : Lk;
        for (int64_t lk = 0; lk < Lk; lk++) {                       /* attn_scores */
            float acc = 0.0f;
            for (int64_t e = 0; e < E; e++)
                acc = fmaf(h2f(q[e * qs[0] + lq * qs[1] + h * qs[2] + b * qs[3]]),
                           h2f(k[e * ks[0] + lk * ks[1] + h * ks[2] + b * ks[3]]), acc);
            acc *= scale;
            if (bias) acc += bias_at(bias, bias_f32, bs, lk, lq, h, b);
            if (lk >= klim) acc = -INFINITY;
            sc[lk] = f2h(acc);
        }
        float m = -INFINITY, s = 0.0f;                              /* attn_softmax */
        for (int64_t lk = 0; lk < Lk; lk++) m = fmaxf(m, h2f(sc[lk]));
        if (!isfinite(m)) {
            for (int64_t lk = 0; lk < Lk; lk++) sc[lk] = 0;
            s = 1.0f;
        } else {
            for (int64_t lk = 0; lk < Lk; lk++) {
                float e = expf(h2f(sc[lk]) - m);
                sc[lk] = f2h(e);
                s += e;
            }
        }
        for (int64_t e = 0; e < E; e++) {                           /* attn_apply */
            float acc = 0.0f;
            for (int64_t lk = 0; lk < Lk; lk++)
                acc = fmaf(h2f(sc[lk]), h2f(v[e * vs[0] + lk * vs[1] + h * vs[2] + b * vs[3]]), acc);
            float r = acc / s;
            int64_t o = e + E * (lq + Lq * (h + H * b));
            if (out_f32) ((float *)out)[o] = r; else ((uint16_t *)out)[o] = f2h(r);
        }
        free(sc);
    }
}

/* Composed Float32 reference for the cpu=false fused kernels: softmax(QK^T
 * scale + bias) V with nothing rounded between the stages (the in-file host
 * references of the reference's tests: test_flash.jl:13-24 attnref,
 * test_coopmat_attention.jl:28-39 threepass).  Accumulation in double so that
 * it is a reference for, not a copy of, any fp32 summation order. */
ORC_API void orc_sdpa_ref_f32(float *out,
                              const uint16_t *q, const int64_t *qs,
                              const uint16_t *k, const int64_t *ks,
                              const uint16_t *v, const int64_t *vs,
                              const void *bias, int bias_f32, const int64_t *bs,
                              const int32_t *kv_len,
                              int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale) {
    #pragma omp parallel for collapse(3) schedule(static)
    for (int64_t b = 0; b < B; b++)
    for (int64_t h = 0; h < H; h++)
    for (int64_t lq = 0; lq < Lq; lq++) {
        int64_t n = Lk > 0 ? Lk : 1;
        double *sc = (double *)malloc(sizeof(double) * (size_t)n);
        int64_t klim = kv_len ? (kv_len[b] < Lk ? kv_len[b] : Lk) : Lk;
        double m = -INFINITY;
        for (int64_t lk = 0; lk < Lk; lk++) {
            double acc = 0.0;
            for (int64_t e = 0; e < E; e++)
                acc += (double)h2f(q[e * qs[0] + lq * qs[1] + h * qs[2] + b * qs[3]]) *
                       (double)h2f(k[e * ks[0] + lk * ks[1] + h * ks[2] + b * ks[3]]);
            acc *= (double)scale;
            if (bias) acc += (double)bias_at(bias, bias_f32, bs, lk, lq, h, b);
            if (lk >= klim) acc = -INFINITY;
            sc[lk] = acc;
            if (acc > m) m = acc;
        }
        double s = 0.0;
        if (!isfinite(m)) { for (int64_t lk = 0; lk < Lk; lk++) sc[lk] = 0.0; s = 1.0; }
        else for (int64_t lk = 0; lk < Lk; lk++) { sc[lk] = exp(sc[lk] - m); s += sc[lk]; }
        for (int64_t e = 0; e < E; e++) {
            double acc = 0.0;
            for (int64_t lk = 0; lk < Lk; lk++)
                acc += sc[lk] * (double)h2f(v[e * vs[0] + lk * vs[1] + h * vs[2] + b * vs[3]]);
            out[e + E * (lq + Lq * (h + H * b))] = (float)(acc / s);
        }
        free(sc);
    }
}

/* The online-softmax recurrence of the fused kernels in scalar fp32,
 * flash.jl:25-38 (m' = max(m,rowmax); c = exp(m-m'); l' = l*c + sum exp(s-m');
 * acc' = acc*c + sum exp(s-m') v; out = acc/l), walked in key blocks of `bk`,
 * optionally split into `nsplit` key ranges merged as flash.jl:1385-1421
 * (m = max m_s; L = sum e^{m_s-m} l_s; O = sum e^{m_s-m} O_s / L).
 * Dense operands only.  Used to check that block size and split count do not
 * change the result beyond fp32 rounding. */
ORC_API void orc_sdpa_flash_f32(float *out, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B,
                                float scale, int64_t bk, int64_t nsplit) {
    if (nsplit < 1) nsplit = 1;
    if (bk < 1) bk = 32;
    int64_t nblk = (Lk + bk - 1) / bk, per = (nblk + nsplit - 1) / nsplit;
    #pragma omp parallel for collapse(3) schedule(static)
    for (int64_t b = 0; b < B; b++)
    for (int64_t h = 0; h < H; h++)
    for (int64_t lq = 0; lq < Lq; lq++) {
        const uint16_t *qr = q + E * (lq + Lq * (h + H * b));
        float *O = (float *)calloc((size_t)(E * nsplit), sizeof(float));
        float *ms = (float *)malloc(sizeof(float) * (size_t)nsplit), *ls = (float *)malloc(sizeof(float) * (size_t)nsplit);
        float *sb = (float *)malloc(sizeof(float) * (size_t)bk);
        for (int64_t s = 0; s < nsplit; s++) {
            float m = -INFINITY, l = 0.0f; float *acc = O + s * E;
            int64_t k0 = s * per * bk, k1 = (s + 1) * per * bk; if (k1 > Lk) k1 = Lk;
            for (int64_t kb = k0; kb < k1; kb += bk) {
                int64_t ke = kb + bk < k1 ? kb + bk : k1;
                float rm = -INFINITY;
                for (int64_t lk = kb; lk < ke; lk++) {
                    const uint16_t *kr = k + E * (lk + Lk * (h + H * b));
                    float a = 0.0f;
                    for (int64_t e = 0; e < E; e++) a = fmaf(h2f(qr[e]), h2f(kr[e]), a);
                    sb[lk - kb] = a * scale; rm = fmaxf(rm, sb[lk - kb]);
                }
                float mn = fmaxf(m, rm), c = isfinite(mn) ? expf(m - mn) : 1.0f;
                l *= c; for (int64_t e = 0; e < E; e++) acc[e] *= c;
                for (int64_t lk = kb; lk < ke; lk++) {
                    float p = isfinite(mn) ? expf(sb[lk - kb] - mn) : 0.0f;
                    const uint16_t *vr = v + E * (lk + Lk * (h + H * b));
                    l += p; for (int64_t e = 0; e < E; e++) acc[e] = fmaf(p, h2f(vr[e]), acc[e]);
                }
                m = mn;
            }
            ms[s] = m; ls[s] = l;
        }
        float m = -INFINITY; for (int64_t s = 0; s < nsplit; s++) m = fmaxf(m, ms[s]);
        float L = 0.0f;
        for (int64_t s = 0; s < nsplit; s++) if (isfinite(ms[s])) L += expf(ms[s] - m) * ls[s];
        for (int64_t e = 0; e < E; e++) {
            float o = 0.0f;
            for (int64_t s = 0; s < nsplit; s++) if (isfinite(ms[s])) o += expf(ms[s] - m) * O[s * E + e];
            out[e + E * (lq + Lq * (h + H * b))] = L > 0.0f ? o / L : 0.0f;
        }
        free(O); free(ms); free(ls); free(sb);
    }
}

/* ------------------------------------------------------------------ convolution
 * kernels/extern/conv.jl:26-51 (conv2d, direct form): x (W,H,Cin,N) =
 * row-major [N][Cin][H][W]; w (KW,KH,Cin/groups,Cout) = [Cout][Cin/g][KH][KW];
 * out (OW,OH,Cout,N).  acc = fp32(bias[co]); loops ci, ky, kx (kx innermost);
 * fp32 muladd; one rounding; relu on the rounded value (conv_coopmat.jl:307-333). */
ORC_API int64_t orc_convsize(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d) {   /* conv.jl:309 */
    return (n + 2 * p - d * (k - 1) - 1) / s + 1;
}
ORC_API void orc_conv2d_f16(void *out, int out_f32, const uint16_t *x, const uint16_t *w, const uint16_t *bias,
                            int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                            int64_t KW, int64_t KH, int64_t Cout,
                            int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy,
                            int64_t groups, int relu) {
    int64_t OW = orc_convsize(Wi, KW, sx, px, dx), OH = orc_convsize(Hi, KH, sy, py, dy);
    int64_t cing = Cin / groups, coutg = Cout / groups;
    #pragma omp parallel for collapse(2) schedule(static)
    for (int64_t n = 0; n < N; n++)
    for (int64_t co = 0; co < Cout; co++) {
        int64_t g = co / coutg;
        for (int64_t oy = 0; oy < OH; oy++)
        for (int64_t ox = 0; ox < OW; ox++) {
            float acc = bias ? h2f(bias[co]) : 0.0f;
            for (int64_t ci = 0; ci < cing; ci++) {
                int64_t xc = g * cing + ci;
                for (int64_t ky = 0; ky < KH; ky++) {
                    int64_t iy = oy * sy - py + ky * dy;
                    if (iy < 0 || iy >= Hi) continue;
                    for (int64_t kx = 0; kx < KW; kx++) {
                        int64_t ix = ox * sx - px + kx * dx;
                        if (ix < 0 || ix >= Wi) continue;
                        acc = fmaf(h2f(x[((n * Cin + xc) * Hi + iy) * Wi + ix]),
                                   h2f(w[((co * cing + ci) * KH + ky) * KW + kx]), acc);
                    }
                }
            }
            int64_t o = ((n * Cout + co) * OH + oy) * OW + ox;
            if (out_f32) { ((float *)out)[o] = relu && acc < 0 ? 0.0f : acc; }
            else { float r = h2f(f2h(acc)); ((uint16_t *)out)[o] = f2h(relu && r < 0 ? 0.0f : r); }
        }
    }
}

/* conv.jl:201 (convtransposesize) */
ORC_API int64_t orc_convtransposesize(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d, int64_t op) {
    return (n - 1) * s - 2 * p + d * (k - 1) + op + 1;
}
/* conv.jl:149-191 (convtranspose2d): the gather form -- every output element is computed from the inputs
 * that reach it (stride divisibility), fp32 accumulator seeded with the bias, one rounding.  w is torch's
 * transposed-convolution weight [Cin][Cout/groups][KH][KW]. */
ORC_API void orc_convtranspose2d_f16(void *out, int out_f32, const uint16_t *x, const uint16_t *w, const uint16_t *bias,
                                     int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                                     int64_t KW, int64_t KH, int64_t Cout,
                                     int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy,
                                     int64_t opx, int64_t opy, int64_t groups) {
    int64_t OW = orc_convtransposesize(Wi, KW, sx, px, dx, opx), OH = orc_convtransposesize(Hi, KH, sy, py, dy, opy);
    int64_t cing = Cin / groups, coutg = Cout / groups;
    #pragma omp parallel for collapse(2) schedule(static)
    for (int64_t n = 0; n < N; n++)
    for (int64_t co = 0; co < Cout; co++) {
        int64_t g = co / coutg, cog = co % coutg;
        for (int64_t oy = 0; oy < OH; oy++)
        for (int64_t ox = 0; ox < OW; ox++) {
            float acc = bias ? h2f(bias[co]) : 0.0f;
            int64_t bx = ox + px, by = oy + py;
            for (int64_t ci = g * cing; ci < (g + 1) * cing; ci++) {
                for (int64_t ky = 0; ky < KH; ky++) {
                    int64_t ty = by - ky * dy;
                    if (ty < 0 || ty % sy != 0) continue;
                    int64_t iy = ty / sy;
                    if (iy >= Hi) continue;
                    for (int64_t kx = 0; kx < KW; kx++) {
                        int64_t tx = bx - kx * dx;
                        if (tx < 0 || tx % sx != 0) continue;
                        int64_t ix = tx / sx;
                        if (ix >= Wi) continue;
                        acc = fmaf(h2f(x[((n * Cin + ci) * Hi + iy) * Wi + ix]),
                                   h2f(w[((ci * coutg + cog) * KH + ky) * KW + kx]), acc);
                    }
                }
            }
            int64_t o = ((n * Cout + co) * OH + oy) * OW + ox;
            if (out_f32) ((float *)out)[o] = acc;
            else ((uint16_t *)out)[o] = f2h(acc);
        }
    }
}

/* conv_coopmat.jl:259-286 (im2col_kernel!): col is column-major MP x CRSP, i.e.
 * row-major [CRSP][MP]; row m = pixel (n, oh, ow) with ow fastest; column
 * c = (cin, kh, kw) with kw fastest; zero for m >= NPQ, c >= CRS and for taps
 * that fall in the padding. */
ORC_API void orc_im2col_f16(uint16_t *col, const uint16_t *x,
                            int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH,
                            int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy,
                            int64_t MP, int64_t CRSP) {
    int64_t OW = orc_convsize(Wi, KW, sx, px, dx), OH = orc_convsize(Hi, KH, sy, py, dy);
    int64_t NPQ = N * OH * OW, CRS = Cin * KH * KW;
    for (int64_t c = 0; c < CRSP; c++)
    for (int64_t m = 0; m < MP; m++) {
        uint16_t val = 0;
        if (m < NPQ && c < CRS) {
            int64_t ow = m % OW, oh = (m / OW) % OH, n = m / (OW * OH);
            int64_t kw = c % KW, kh = (c / KW) % KH, ci = c / (KW * KH);
            int64_t ix = ow * sx - px + kw * dx, iy = oh * sy - py + kh * dy;
            if (ix >= 0 && ix < Wi && iy >= 0 && iy < Hi) val = x[((n * Cin + ci) * Hi + iy) * Wi + ix];
        }
        col[c * MP + m] = val;
    }
}

/* ------------------------------------------------------------------ layer norm
 * kernels/layernorm.jl:53-113: mean in fp32, variance about that mean in fp32
 * (two passes), r = 1/sqrt(var + eps); out = (x-mu)*r*gamma + beta, stored in
 * the operand type; mean and rstd returned in fp32.  The reference reduces
 * with a 128-lane strided partial sum and a tree; the summation order is not
 * part of the contract (ops.jl:586-597 "the two forms do not produce identical
 * bits"), so this uses a double accumulator rounded to fp32. */
ORC_API void orc_layernorm_f16(uint16_t *out, float *mean, float *rstd, const uint16_t *a,
                               const uint16_t *gamma, const uint16_t *beta,
                               int64_t C, int64_t groups, float eps) {
    #pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < groups; g++) {
        const uint16_t *r = a + g * C;
        double s = 0.0; for (int64_t i = 0; i < C; i++) s += h2f(r[i]);
        float mu = (float)(s / (double)C);
        double s2 = 0.0; for (int64_t i = 0; i < C; i++) { float d = h2f(r[i]) - mu; s2 += (double)(d * d); }
        float rs = 1.0f / sqrtf((float)(s2 / (double)C) + eps);
        for (int64_t i = 0; i < C; i++) {
            float x = (h2f(r[i]) - mu) * rs;
            if (gamma) x *= h2f(gamma[i]);
            if (beta) x += h2f(beta[i]);
            out[g * C + i] = f2h(x);
        }
        if (mean) mean[g] = mu;
        if (rstd) rstd[g] = rs;
    }
}

/* ops.jl:474-555 softmax_kernel!: per slice m = max, s = sum exp(x - m), out = T(exp(x - m) / s), all in fp32
 * (the 64-lane strided partial sums are a reduction order, not part of the contract: a double accumulator here).
 * `scale` multiplies x first, as attn_softmax_rows! does (attention.jl:528-560); 1 for aten::_softmax.
 * A slice of -inf gives zeros, the attention convention (attention.jl:82-87). */
ORC_API void orc_softmax_f16(uint16_t *out, const uint16_t *a, int64_t n, int64_t rows, float scale) {
    #pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < rows; g++) {
        const uint16_t *r = a + g * n;
        float m = -INFINITY;
        for (int64_t i = 0; i < n; i++) { float x = h2f(r[i]) * scale; if (x > m) m = x; }
        if (m == -INFINITY) { for (int64_t i = 0; i < n; i++) out[g * n + i] = 0; continue; }
        double s = 0.0;
        for (int64_t i = 0; i < n; i++) s += (double)expf(h2f(r[i]) * scale - m);
        float den = (float)s;
        for (int64_t i = 0; i < n; i++) out[g * n + i] = f2h(expf(h2f(r[i]) * scale - m) / den);
    }
}

/* out = fp16(fp32(a) * c): mul.Tensor / div.Tensor with a constant in the operand type. */
ORC_API void orc_scale_f16(uint16_t *o, const uint16_t *a, float c, int64_t n) {
    for (int64_t i = 0; i < n; i++) o[i] = f2h(h2f(a[i]) * c);
}

/* out = fp16(fp32(a) + fp32(b)): the graph's residual add.Tensor in the operand
 * type (ops.jl:186-197 broadcast emit; Julia Float16 '+' rounds once). */
ORC_API void orc_add_f16(uint16_t *o, const uint16_t *a, const uint16_t *b, int64_t n) {
    for (int64_t i = 0; i < n; i++) o[i] = f2h(h2f(a[i]) + h2f(b[i]));
}
