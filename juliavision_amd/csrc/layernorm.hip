// Layer norm, the residual add, row softmax and scaling by a constant: the HBM-bound
// glue between the contractions of an encoder block.  One wavefront per row or
// normalisation group, the row held in registers between the passes so that it
// is read from memory once; fp32 statistics (layernorm.jl:53-113, ops.jl:474-555).
#include "common.hpp"

namespace {

// A row of C <= 64 * 8 * NCH halves lives in NCH 16-byte chunks per lane.
template <int NCH>
__global__ __launch_bounds__(256) void layernorm_vec_kernel(half_t *out, float *mean, float *rstd, const half_t *a,
                                                            const half_t *gamma, const half_t *beta, int C, long groups, float eps) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long g = (long)blockIdx.x * 4 + wave;
    if (g >= groups) return;
    const half_t *row = a + g * C;
    float x[NCH][8];
    float s = 0.0f;
    // gamma and beta are requested together with the row: one trip to memory for the kernel, not two
    u32x4 graw[NCH], braw[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        const u32x4 z = {0u, 0u, 0u, 0u};
        graw[i] = (gamma && e0 < C) ? ldg16(gamma + e0) : z;
        braw[i] = (beta && e0 < C) ? ldg16(beta + e0) : z;
    }
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < C) {
            half8v t = as_half8(ldg16(row + e0));
#pragma unroll
            for (int j = 0; j < 8; j++) { x[i][j] = (float)t[j]; s += x[i][j]; }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) x[i][j] = 0.0f;
        }
    }
    s = wave_sum(s);
    const float mu = s / (float)C;
    float s2 = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < C) {
#pragma unroll
            for (int j = 0; j < 8; j++) { const float d = x[i][j] - mu; s2 = fmaf(d, d, s2); }
        }
    }
    s2 = wave_sum(s2);
    const float r = 1.0f / sqrtf(s2 / (float)C + eps);
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < C) {
            const half8v gv = as_half8(graw[i]), bv = as_half8(braw[i]);
            half8v o;
#pragma unroll
            for (int j = 0; j < 8; j++)
                o[j] = ln_norm1(x[i][j], mu, r, gamma != nullptr, gamma ? (float)gv[j] : 0.0f, beta != nullptr, beta ? (float)bv[j] : 0.0f);
            *reinterpret_cast<half8v *>(out + g * C + e0) = o;
        }
    }
    if (lane == 0) {
        if (mean) mean[g] = mu;
        if (rstd) rstd[g] = r;
    }
}

// Any C, any alignment: the same three passes reading memory each time.
__global__ __launch_bounds__(256) void layernorm_any_kernel(half_t *out, float *mean, float *rstd, const half_t *a,
                                                            const half_t *gamma, const half_t *beta, int C, long groups, float eps) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long g = (long)blockIdx.x * 4 + wave;
    if (g >= groups) return;
    const half_t *row = a + g * C;
    float s = 0.0f;
    for (int i = lane; i < C; i += 64) s += (float)row[i];
    s = wave_sum(s);
    const float mu = s / (float)C;
    float s2 = 0.0f;
    for (int i = lane; i < C; i += 64) { const float d = (float)row[i] - mu; s2 = fmaf(d, d, s2); }
    s2 = wave_sum(s2);
    const float r = 1.0f / sqrtf(s2 / (float)C + eps);
    for (int i = lane; i < C; i += 64) {
        float y = ((float)row[i] - mu) * r;
        if (gamma) y *= (float)gamma[i];
        if (beta) y += (float)beta[i];
        out[g * C + i] = (half_t)y;
    }
    if (lane == 0) {
        if (mean) mean[g] = mu;
        if (rstd) rstd[g] = r;
    }
}

// Softmax over rows of n elements (the last, contiguous axis): m = max, s = sum exp(c x - m), out = exp(c x - m) / s in
// fp32, one rounding (softmax_kernel!, ops.jl:474-555; c = 1 there -- a constant scale ahead of the softmax rides along
// here).  A row whose maximum is -inf (every element masked) gives zeros, as the attention kernels do.
template <int NCH>
__global__ __launch_bounds__(256) void softmax_vec_kernel(half_t *out, const half_t *a, int n, long rows, float c) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long g = (long)blockIdx.x * 4 + wave;
    if (g >= rows) return;
    const half_t *row = a + g * n;
    float x[NCH][8];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < n) {
            half8v t = as_half8(ldg16(row + e0));
#pragma unroll
            for (int j = 0; j < 8; j++) { x[i][j] = (float)t[j] * c; m = fmaxf(m, x[i][j]); }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) x[i][j] = -INFINITY;
        }
    }
    m = wave_max(m);
    const float mm = m == -INFINITY ? 0.0f : m;
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) { x[i][j] = __expf(x[i][j] - mm); s += x[i][j]; }
    s = wave_sum(s);
    const float inv = s > 0.0f ? 1.0f / s : 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < n) {
            half8v o;
#pragma unroll
            for (int j = 0; j < 8; j++) o[j] = (half_t)(x[i][j] * inv);
            *reinterpret_cast<half8v *>(out + g * n + e0) = o;
        }
    }
}

// Any n, any alignment, fp16 or fp32 rows: three passes over memory.
template <typename T>
__global__ __launch_bounds__(256) void softmax_any_kernel(T *out, const T *a, int n, long rows, float c) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long g = (long)blockIdx.x * 4 + wave;
    if (g >= rows) return;
    const T *row = a + g * n;
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, (float)row[i] * c);
    m = wave_max(m);
    const float mm = m == -INFINITY ? 0.0f : m;
    float s = 0.0f;
    for (int i = lane; i < n; i += 64) s += __expf((float)row[i] * c - mm);
    s = wave_sum(s);
    const float inv = s > 0.0f ? 1.0f / s : 0.0f;
    for (int i = lane; i < n; i += 64) out[g * n + i] = (T)(__expf((float)row[i] * c - mm) * inv);
}

__global__ void scale_kernel(half_t *o, const half_t *a, float c, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) o[i] = (half_t)((float)a[i] * c);
}

// A stand-alone activation (the same functions the GEMM and convolution epilogues apply) and clamp.
__global__ void act_kernel(half_t *o, const half_t *a, int epi, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) o[i] = (half_t)apply_epi((float)a[i], epi);
}
__global__ void clamp_kernel(half_t *o, const half_t *a, float lo, float hi, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) o[i] = (half_t)fminf(fmaxf((float)a[i], lo), hi);
}

__global__ void add_vec_kernel(half_t *o, const half_t *a, const half_t *b, long n8) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    half8v x = as_half8(ldg16(a + i * 8)), y = as_half8(ldg16(b + i * 8)), r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = (half_t)((float)x[j] + (float)y[j]);
    *reinterpret_cast<half8v *>(o + i * 8) = r;
}
__global__ void add_any_kernel(half_t *o, const half_t *a, const half_t *b, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) o[i] = (half_t)((float)a[i] + (float)b[i]);
}


// Row statistics for a layer norm that is folded into the GEMM reading the rows (mi_lnfold_gemm_f16): for every
// 32-column segment of a row, (sum, squares about the segment's own mean) -- what the GEMM stores leave when they
// produce the rows themselves -- stored segment-major.  A thread owns one segment of one row (64 bytes, four 16-byte
// loads, no exchange between lanes); the lanes of a wave take consecutive rows, so its result is one contiguous store.
__global__ __launch_bounds__(256) void rowstats_kernel(float *stats, const half_t *a, long ld, int C, long rows) {
    const long g = (long)blockIdx.x * 256 + threadIdx.x;      // row
    const int seg = blockIdx.y;
    if (g >= rows) return;
    const half_t *src = a + g * ld + 32 * seg;
    const int chunks = min(4, (C - 32 * seg) / 8);             // C % 8 == 0
    half8v t[4];
#pragma unroll
    for (int i = 0; i < 4; i++) if (i < chunks) t[i] = as_half8(ldg16(src + 8 * i));
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (i < chunks) {
#pragma unroll
            for (int j = 0; j < 8; j++) sum += (float)t[i][j];
        }
    const float mean = sum / (float)(8 * chunks);
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (i < chunks) {
#pragma unroll
            for (int j = 0; j < 8; j++) { const float d = (float)t[i][j] - mean; sq = fmaf(d, d, sq); }
        }
    const float2v o = {sum, sq};
    *reinterpret_cast<float2v *>(stats + ((long)seg * rows + g) * 2) = o;
}

// Load-time preparation of a folded norm: Wp = fp16(gamma[k] W[k][n]), colsum[n] = sum_k Wp[k][n] (of the ROUNDED
// values: what the matrix units will multiply), biasp[n] = bias[n] + sum_k beta[k] W[k][n], both in fp32; run once per
// weight.  A thread moves sixteen bytes of W at a time; the sums over k are partial sums of fixed k-subsets combined
// in a fixed order (the same bits on every run).
//   [K][F] weights: a workgroup owns 64 columns, its thread (chunk c of 8 columns, k-group g of 32) walks k = g, g + 32, ...
//   [F][K] weights: a workgroup owns 8 columns, a group of 32 lanes walks one of them 256 k at a time
template <bool B_KN>
__global__ __launch_bounds__(256) void lnfold_prepare_kernel(half_t *Wp, float *colsum, float *biasp, const half_t *W, const half_t *gamma,
                                                             const half_t *beta, const half_t *bias, int K, int F, long ldW) {
    __shared__ float part[2][32][64];
    const int tid = threadIdx.x;
    if constexpr (B_KN) {
        const int c = tid & 7, g = tid >> 3, n0 = blockIdx.x * 64 + c * 8;
        float cs[8], bp[8];
#pragma unroll
        for (int e = 0; e < 8; e++) cs[e] = bp[e] = 0.0f;
        if (n0 < F) {
            for (int k = g; k < K; k += 32) {
                const long at = (long)k * ldW + n0;
                const half8v w = as_half8(ldg16(W + at));
                const float gk = gamma ? (float)gamma[k] : 1.0f, bk = beta ? (float)beta[k] : 0.0f;
                half8v o;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    o[e] = (half_t)(gamma ? gk * (float)w[e] : (float)w[e]);
                    cs[e] += (float)o[e];
                    bp[e] = fmaf(bk, (float)w[e], bp[e]);
                }
                *reinterpret_cast<half8v *>(Wp + at) = o;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; e++) { part[0][g][c * 8 + e] = cs[e]; part[1][g][c * 8 + e] = bp[e]; }
        __syncthreads();
        if (tid < 64 && blockIdx.x * 64 + tid < F) {
            const int n = blockIdx.x * 64 + tid;
            float a = 0.0f, b = bias ? (float)bias[n] : 0.0f;
            for (int q = 0; q < 32; q++) { a += part[0][q][tid]; b += part[1][q][tid]; }
            colsum[n] = a;
            biasp[n] = b;
        }
    } else {
        const int l = tid & 31, n = blockIdx.x * 8 + (tid >> 5);
        float cs = 0.0f, bp = 0.0f;
        if (n < F) {
            for (int k0 = l * 8; k0 < K; k0 += 256) {
                const long at = (long)n * ldW + k0;
                const half8v w = as_half8(ldg16(W + at));
                half8v o;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    o[e] = (half_t)(gamma ? (float)gamma[k0 + e] * (float)w[e] : (float)w[e]);
                    cs += (float)o[e];
                    if (beta) bp = fmaf((float)beta[k0 + e], (float)w[e], bp);
                }
                *reinterpret_cast<half8v *>(Wp + at) = o;
            }
        }
        part[0][tid >> 5][l] = cs;
        part[1][tid >> 5][l] = bp;
        __syncthreads();
        if (l == 0 && n < F) {
            float a = 0.0f, b = bias ? (float)bias[n] : 0.0f;
            for (int q = 0; q < 32; q++) { a += part[0][tid >> 5][q]; b += part[1][tid >> 5][q]; }
            colsum[n] = a;
            biasp[n] = b;
        }
    }
}

// The same, an element at a time: weights whose rows do not start on sixteen bytes or whose extents are not multiples of 8.
__global__ __launch_bounds__(256) void lnfold_prepare_any_kernel(half_t *Wp, float *colsum, float *biasp, const half_t *W, const half_t *gamma,
                                                                 const half_t *beta, const half_t *bias, int K, int F, long ldW, int b_kn) {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= F) return;
    float cs = 0.0f, bp = bias ? (float)bias[n] : 0.0f;
    for (int k = 0; k < K; k++) {
        const long at = b_kn ? (long)k * ldW + n : (long)n * ldW + k;
        const float w = (float)W[at];
        const half_t wp = (half_t)(gamma ? (float)gamma[k] * w : w);
        Wp[at] = wp;
        cs += (float)wp;
        if (beta) bp = fmaf((float)beta[k], w, bp);
    }
    colsum[n] = cs;
    biasp[n] = bp;
}

}  // namespace

extern "C" {

int mi_layernorm_f16(void *out, float *mean, float *rstd, const void *a, const void *gamma, const void *beta,
                     int64_t C, int64_t groups, float eps, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !a) return MI_DECLINE_OPERANDS;
    if (C < 1 || C > INT32_MAX || groups < 0) return MI_DECLINE_EXTENT;
    if (groups == 0) return MI_OK;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)ceil_div(groups, 4)), block(256);
    half_t *o = (half_t *)out;
    const half_t *x = (const half_t *)a, *g = (const half_t *)gamma, *b = (const half_t *)beta;
    const bool vec = C % 8 == 0 && aligned_to(a, 16) && aligned_to(out, 16) && (!g || aligned_to(g, 16)) && (!b || aligned_to(b, 16));
    if (vec && C <= 512)       hipLaunchKernelGGL(layernorm_vec_kernel<1>, grid, block, 0, st, o, mean, rstd, x, g, b, (int)C, (long)groups, eps);
    else if (vec && C <= 1024) hipLaunchKernelGGL(layernorm_vec_kernel<2>, grid, block, 0, st, o, mean, rstd, x, g, b, (int)C, (long)groups, eps);
    else if (vec && C <= 2048) hipLaunchKernelGGL(layernorm_vec_kernel<4>, grid, block, 0, st, o, mean, rstd, x, g, b, (int)C, (long)groups, eps);
    else if (vec && C <= 4096) hipLaunchKernelGGL(layernorm_vec_kernel<8>, grid, block, 0, st, o, mean, rstd, x, g, b, (int)C, (long)groups, eps);
    else                       hipLaunchKernelGGL(layernorm_any_kernel, grid, block, 0, st, o, mean, rstd, x, g, b, (int)C, (long)groups, eps);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_softmax_f16(void *out, const void *a, int dtype, int64_t n, int64_t rows, float scale, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !a) return MI_DECLINE_OPERANDS;
    if (dtype != MI_F16 && dtype != MI_F32) return MI_DECLINE_OPERANDS;
    if (n < 1 || n > INT32_MAX || rows < 0) return MI_DECLINE_EXTENT;
    if (rows == 0) return MI_OK;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)ceil_div(rows, 4)), block(256);
    if (dtype == MI_F32) {
        hipLaunchKernelGGL(softmax_any_kernel<float>, grid, block, 0, st, (float *)out, (const float *)a, (int)n, (long)rows, scale);
        return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
    }
    half_t *o = (half_t *)out;
    const half_t *x = (const half_t *)a;
    const bool vec = n % 8 == 0 && aligned_to(a, 16) && aligned_to(out, 16);
    if (vec && n <= 512)       hipLaunchKernelGGL(softmax_vec_kernel<1>, grid, block, 0, st, o, x, (int)n, (long)rows, scale);
    else if (vec && n <= 1024) hipLaunchKernelGGL(softmax_vec_kernel<2>, grid, block, 0, st, o, x, (int)n, (long)rows, scale);
    else if (vec && n <= 2048) hipLaunchKernelGGL(softmax_vec_kernel<4>, grid, block, 0, st, o, x, (int)n, (long)rows, scale);
    else if (vec && n <= 4096) hipLaunchKernelGGL(softmax_vec_kernel<8>, grid, block, 0, st, o, x, (int)n, (long)rows, scale);
    else                       hipLaunchKernelGGL(softmax_any_kernel<half_t>, grid, block, 0, st, o, x, (int)n, (long)rows, scale);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_scale_f16(void *out, const void *a, float c, int64_t n, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !a) return MI_DECLINE_OPERANDS;
    if (n < 0) return MI_DECLINE_EXTENT;
    if (n == 0) return MI_OK;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, (half_t *)out, (const half_t *)a, c, (long)n);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_act_f16(void *out, const void *a, int epi, int64_t n, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !a) return MI_DECLINE_OPERANDS;
    if (epi < MI_EPI_NONE || epi > MI_EPI_RELU) return MI_DECLINE_UNSUPPORTED;
    if (n < 0) return MI_DECLINE_EXTENT;
    if (n == 0) return MI_OK;
    hipLaunchKernelGGL(act_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, (half_t *)out, (const half_t *)a, epi, (long)n);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_clamp_f16(void *out, const void *a, float lo, float hi, int64_t n, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !a) return MI_DECLINE_OPERANDS;
    if (n < 0 || is_nan_arg(lo) || is_nan_arg(hi) || lo > hi) return MI_DECLINE_EXTENT;
    if (n == 0) return MI_OK;
    hipLaunchKernelGGL(clamp_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, (half_t *)out, (const half_t *)a, lo, hi, (long)n);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_add_f16(void *out, const void *a, const void *b, int64_t n, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !a || !b) return MI_DECLINE_OPERANDS;
    if (n < 0) return MI_DECLINE_EXTENT;
    if (n == 0) return MI_OK;
    hipStream_t st = (hipStream_t)stream;
    if (n % 8 == 0 && aligned_to(out, 16) && aligned_to(a, 16) && aligned_to(b, 16))
        hipLaunchKernelGGL(add_vec_kernel, dim3((unsigned)ceil_div(n / 8, 256)), dim3(256), 0, st, (half_t *)out, (const half_t *)a, (const half_t *)b, (long)(n / 8));
    else
        hipLaunchKernelGGL(add_any_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, (half_t *)out, (const half_t *)a, (const half_t *)b, (long)n);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_rowstats_f16(float *stats, const void *a, int64_t ld, int64_t C, int64_t rows, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!stats || !a || !aligned_to(stats, 8) || !aligned_to(a, 16)) return MI_DECLINE_OPERANDS;
    if (C < 8 || C % 8 || ld < C || ld % 8 || rows < 0 || C > INT32_MAX) return MI_DECLINE_EXTENT;
    if (rows == 0) return MI_OK;
    if (ceil_div(C, 32) > 65535) return MI_DECLINE_EXTENT;
    hipLaunchKernelGGL(rowstats_kernel, dim3((unsigned)ceil_div(rows, 256), (unsigned)ceil_div(C, 32)), dim3(256), 0, (hipStream_t)stream,
                       stats, (const half_t *)a, (long)ld, (int)C, (long)rows);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_lnfold_prepare_f16(void *Wp, float *colsum, float *biasp, const void *W, const void *gamma, const void *beta, const void *bias,
                          int64_t K, int64_t F, int64_t ldW, int w_layout, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!Wp || !colsum || !biasp || !W || (w_layout != MI_W_KF && w_layout != MI_W_FK)) return MI_DECLINE_OPERANDS;
    if (K < 1 || F < 1 || K > INT32_MAX || F > INT32_MAX || ldW < (w_layout == MI_W_KF ? F : K)) return MI_DECLINE_EXTENT;
    hipStream_t st = (hipStream_t)stream;
    half_t *o = (half_t *)Wp;
    const half_t *w = (const half_t *)W, *g = (const half_t *)gamma, *be = (const half_t *)beta, *bi = (const half_t *)bias;
    const bool kn = w_layout == MI_W_KF;
    const bool vec = aligned_to(W, 16) && aligned_to(Wp, 16) && ldW % 8 == 0 && (kn ? F % 8 == 0 : K % 8 == 0);
    if (!vec)    hipLaunchKernelGGL(lnfold_prepare_any_kernel, dim3((unsigned)ceil_div(F, 256)), dim3(256), 0, st, o, colsum, biasp, w, g, be, bi, (int)K, (int)F, (long)ldW, kn ? 1 : 0);
    else if (kn) hipLaunchKernelGGL(lnfold_prepare_kernel<true>, dim3((unsigned)ceil_div(F, 64)), dim3(256), 0, st, o, colsum, biasp, w, g, be, bi, (int)K, (int)F, (long)ldW);
    else         hipLaunchKernelGGL(lnfold_prepare_kernel<false>, dim3((unsigned)ceil_div(F, 8)), dim3(256), 0, st, o, colsum, biasp, w, g, be, bi, (int)K, (int)F, (long)ldW);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

}  // extern "C"
