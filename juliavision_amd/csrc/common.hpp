// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/mi355dnn.h"

typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

#define MI_DEVICE static __device__ __forceinline__

MI_DEVICE u32x4 ldg16(const half_t *p) { return *reinterpret_cast<const u32x4 *>(p); }
MI_DEVICE u32x2 ldg8(const half_t *p) { return *reinterpret_cast<const u32x2 *>(p); }

// lo16(x) | lo16(y) << 16   and   hi16(x) | hi16(y) << 16
MI_DEVICE uint32_t pack_lo(uint32_t x, uint32_t y) { return __builtin_amdgcn_perm(y, x, 0x05040100u); }
MI_DEVICE uint32_t pack_hi(uint32_t x, uint32_t y) { return __builtin_amdgcn_perm(y, x, 0x07060302u); }

MI_DEVICE half8v as_half8(u32x4 v) { return __builtin_bit_cast(half8v, v); }

// Lane exchanges without the LDS crossbar.  lane_xor<O>(v) is v of lane (lane ^ O) for O = 1, 2, 4, 8: data-parallel
// primitives riding on the consuming VALU instruction (quad permutes, a rotation by 8 inside each row of 16, and for 4
// the mirror of 8 lanes followed by the mirror of 4: lane ^ 7 ^ 3).  Across rows gfx950 has v_permlane16_swap /
// v_permlane32_swap, which exchange the odd rows of one register with the even rows of another: from two copies of v
// they leave (even rows twice, odd rows twice), whose sum or maximum is op(v[lane], v[lane ^ 16]) in every lane.
// wave_sum / wave_max are the butterflies over 32, 16, 8, 4, 2, 1 built from these: the pairs, the order and therefore
// the bits are those of the same butterfly written with __shfl_xor (six ds_bpermute round trips).
template <int CTRL>
MI_DEVICE float dpp_mov(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true)); }
template <int O>
MI_DEVICE float lane_xor(float v) {
    static_assert(O == 1 || O == 2 || O == 4 || O == 8, "inside a row of 16 lanes");
    if constexpr (O == 1) return dpp_mov<0xB1>(v);             // quad_perm [1,0,3,2]
    else if constexpr (O == 2) return dpp_mov<0x4E>(v);        // quad_perm [2,3,0,1]
    else if constexpr (O == 4) return dpp_mov<0x1B>(dpp_mov<0x141>(v));   // row_half_mirror, then quad_perm [3,2,1,0]
    else return dpp_mov<0x128>(v);                              // row_ror:8
}
// (x, y) <- (even 32-lane halves of both, odd halves of both); the instruction is written out because the builtin's
// second result is miscompiled when both operands hold the same value.
MI_DEVICE void swap_rows32(float &x, float &y) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y)); }
MI_DEVICE void swap_rows16(float &x, float &y) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y)); }
MI_DEVICE float wave_sum(float a) {
    float x = a, y = a;
    swap_rows32(x, y); a = x + y;
    x = a; y = a;
    swap_rows16(x, y); a = x + y;
    a += lane_xor<8>(a);
    a += lane_xor<4>(a);
    a += lane_xor<2>(a);
    a += lane_xor<1>(a);
    return a;
}
MI_DEVICE float wave_max(float a) {
    float x = a, y = a;
    swap_rows32(x, y); a = fmaxf(x, y);
    x = a; y = a;
    swap_rows16(x, y); a = fmaxf(x, y);
    a = fmaxf(a, lane_xor<8>(a));
    a = fmaxf(a, lane_xor<4>(a));
    a = fmaxf(a, lane_xor<2>(a));
    a = fmaxf(a, lane_xor<1>(a));
    return a;
}

// Abramowitz & Stegun 7.1.26 in fp32: the same expression as the reference's
// `erf` (DNNKernels/src/ops.jl:161-169), so a folded gelu is the graph's gelu.
MI_DEVICE float erf_as(float x) {
    float a = fabsf(x);
    float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * a);
    float y = 1.0f - (((((1.061405429f * t - 1.453152027f) * t) + 1.421413741f) * t - 0.284496736f) * t + 0.254829592f) * t * __expf(-a * a);
    return x < 0.0f ? -y : y;
}
// geluexact (DNNKernels/src/ops.jl:1665-1669) = 0.5 v (1 + erf(v / sqrt 2)) with the erf above, written so that it
// costs 11 vector instructions and two transcendentals instead of 17 and two (the GEMM store is bound by them: 32 768
// outputs per workgroup).  With u = |v|, t = 1 / (1 + p u / sqrt 2) and q = 0.5 P(t) exp(-v^2 / 2):
//   v >= 0:  0.5 v (2 - P e) = v - v q        v < 0:  0.5 v (P e) = v q        both:  max(v, 0) - u q.
// Same polynomial, same coefficients; the difference from the textbook order is rounding in the last fp32 place
// (and, for v < -3, none of the cancellation in 1 - (1 - P e)), far below the fp16 result's resolution.
// u is capped at 64: beyond |v| = 14 the exponential is exactly 0 in fp32 and the result max(v, 0) either way, and
// with the cap v = +inf gives +inf as the reference's expression does (uncapped, -inf * 0 + inf would be NaN).  At
// v = -inf the reference's 0.5 v (1 + erf) is -inf * 0 = NaN; this form gives -0.
MI_DEVICE float gelu_erf(float v) {
    const float u = fminf(fabsf(v), 64.0f);
    const float t = __builtin_amdgcn_rcpf(fmaf(u, 0.3275911f * 0.70710678118654752440f, 1.0f));
    float pl = fmaf(0.5f * 1.061405429f, t, -0.5f * 1.453152027f);
    pl = fmaf(pl, t, 0.5f * 1.421413741f);
    pl = fmaf(pl, t, -0.5f * 0.284496736f);
    pl = fmaf(pl, t, 0.5f * 0.254829592f);
    pl *= t;
    const float e = __builtin_amdgcn_exp2f((v * v) * (-0.5f * 1.44269504088896340736f));
    return fmaf(-u, pl * e, fmaxf(v, 0.0f));
}
// ops.jl:1665-1669 (geluexact), 1677-1682 (gelutanh), 1683 (relu_epi)
MI_DEVICE float apply_epi(float v, int epi) {
    switch (epi) {
    case MI_EPI_GELU_ERF: return gelu_erf(v);
    case MI_EPI_GELU_TANH: return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    case MI_EPI_RELU: return fmaxf(v, 0.0f);
    default: return v;
    }
}

template <int EPI>
MI_DEVICE float apply_epi_c(float v) {
    if constexpr (EPI == MI_EPI_GELU_ERF) return gelu_erf(v);
    else if constexpr (EPI == MI_EPI_GELU_TANH) return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    else if constexpr (EPI == MI_EPI_RELU) return fmaxf(v, 0.0f);
    else return v;
}

// One layer-normalised element, rounded to fp16: shared by the layer-norm kernels and the GEMV that folds
// the norm into its prologue, so that the two produce the same bits.
MI_DEVICE half_t ln_norm1(float x, float mu, float r, bool has_g, float g, bool has_b, float b) {
    float y = (x - mu) * r;
    if (has_g) y *= g;
    if (has_b) y += b;
    return (half_t)y;
}

static inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t round_up(size_t a, size_t b) { return (a + b - 1) / b * b; }
// NaN by its bits: the build tells the compiler that no NaNs occur, which folds comparisons with one away.
static inline bool is_nan_arg(float x) { uint32_t u; __builtin_memcpy(&u, &x, 4); return (u & 0x7fffffffu) > 0x7f800000u; }

// Implicit-GEMM convolution: how the GEMM finds its [K][N] operand (the im2col matrix) in a
// zero-padded copy of the input instead of in memory.  The K axis is ordered (kh, kw, ci) with ci
// fastest (the weights are re-laid to match), so a 64-deep tile is 64 consecutive channels of one
// tap: row k of the tile and column n = (oh, ow) is xp[img][ci0 + k][oh*sy + kh*dy][ow + kw*dx],
// and eight consecutive columns of a row are eight consecutive halves of xp (stride 1 along x).
struct ConvGather {
    const half_t *xp;      // padded input [img][Cin][Hp][Wp]; nullptr = ordinary GEMM
    long img;              // elements per image
    long odd;              // xp[i] for odd i is also stored at xp[odd + i], a 4-byte aligned address: a second copy of
                           // the padded input, one element to the left, follows the first
    int HpWp, Wp, OW, sy, dyWp, dx, KW;
    int cpt;               // 64-channel tiles per tap: Cin / 64
    int split;             // 1: the launch's planes are K-slices of one image, 0: they are images
};

// Implicit-GEMM convolution over a channels-last input x[N][H][W][C]: how the GEMM finds its [M][K] operand
// (the patch matrix: row m = output pixel (n, oh, ow), K ordered (kh, kw, ci) with ci fastest) in x itself.
// A 64-deep tile is 64 consecutive channels of one tap, i.e. 128 contiguous bytes of x per row, at an offset
// from the row's pixel that is the same for every row; rows whose tap falls outside the image read zeros.
struct NhwcGather {
    const half_t *x;       // nullptr = ordinary GEMM
    int H, W, C, OH, OW;
    int sx, sy, px, py, dx, dy, KW;
    int cpt;               // 64-channel tiles per tap: C / 64
    int split;             // 1: the launch's planes are K-slices
};

// True once mi_init has run successfully on this process (defined in gemm.hip).
bool mi_ready();
int mi_num_cus();
// Planning for a device other than the current one (mi_*_plan_caps): between begin and end, on this thread,
// mi_num_cus() and mi_plan_mfma() answer for caps (the six values of mi_device_caps); caps == nullptr changes nothing.
bool mi_plan_mfma();
void mi_plan_caps_begin(const int64_t *caps);
void mi_plan_caps_end();
// True if the current device deals workgroups to its XCDs round robin by workgroup id (ids that differ by a multiple
// of 8 share an L2), as a probe launch at mi_init showed; kernels whose workgroups exchange data through one L2 ask.
bool mi_xcd_round_robin();
int mi_sdpa_init();
// Y[M x N] = A[M x K] . B (+bias) (+ residual, fp16, addressed like Y) with B either [K][NB-padded N] (b_kn) or [N][K]; defined in gemm.hip.
int mi_internal_gemm(void *Y, const void *A, const void *B, const void *bias, int M, int N, int NB, int K,
                     long ldY, long ldA, long ldB, int b_kn, int bias_mode, int epi, int out_f32,
                     long nbatch, long sY, long sA, long sB, void *ws, size_t ws_bytes, hipStream_t st,
                     const ConvGather *gather = nullptr, const NhwcGather *agather = nullptr, const void *residual = nullptr);
// Workspace bytes such a call needs (fp32 planes when it splits K); T > 8 rows.
size_t mi_internal_gemm_workspace(int64_t T, int64_t K, int64_t F, int64_t nbatch);
