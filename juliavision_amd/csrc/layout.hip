// Layout helpers: the strided (E,L,H,B) -> dense (L,E,H,B) transpose the reference keeps for
// operands whose contraction axis is not the contiguous one (transposeLE / toLE_tiled,
// attention.jl:342-396).  The GEMM and attention kernels here read strided operands in
// place, so nothing on the hot path calls this; it serves callers that need the other
// order in memory: channel-major convolution output as token-major rows, a [F][K] weight
// hoisted to [K][F].
#include "common.hpp"

namespace {

struct LeArgs {
    half_t *out;
    const half_t *in;
    long sE, sL, sH, sB;       // element strides of the source
    long oE, oH, oB;           // element strides of the destination (its L axis is contiguous)
    int E, L, H;
};

// 32 x 32 tiles through LDS: reads run along e (the source's contiguous axis), writes along l.
// 33 columns: a 32-wide tile would put a whole column into one bank.
__global__ void le_tiled_kernel(LeArgs a) {
    __shared__ half_t tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int e0 = blockIdx.x * 32, l0 = blockIdx.y * 32;
    const int h = blockIdx.z % a.H, b = blockIdx.z / a.H;
    const half_t *src = a.in + h * a.sH + b * a.sB;
    half_t *dst = a.out + h * a.oH + b * a.oB;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int e = e0 + tx, l = l0 + ty + 8 * j;
        tile[ty + 8 * j][tx] = (e < a.E && l < a.L) ? src[e * a.sE + l * a.sL] : (half_t)0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int l = l0 + tx, e = e0 + ty + 8 * j;
        if (l < a.L && e < a.E) dst[e * a.oE + l] = tile[tx][ty + 8 * j];
    }
}

// The source already runs along l: a strided copy, reads and writes both along l.
__global__ void le_copy_kernel(LeArgs a) {
    const int l = blockIdx.x * 64 + (threadIdx.x & 63);
    const int e = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int h = blockIdx.z % a.H, b = blockIdx.z / a.H;
    if (l >= a.L || e >= a.E) return;
    a.out[h * a.oH + b * a.oB + e * a.oE + l] = a.in[h * a.sH + b * a.sB + e * a.sE + l * a.sL];
}

}  // namespace

extern "C" int mi_transpose_le_f16(void *out, const int64_t out_strides[4], const void *in, const int64_t in_strides[4],
                                   int64_t E, int64_t L, int64_t H, int64_t B, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !in || !in_strides) return MI_DECLINE_OPERANDS;
    if (E < 0 || L < 0 || H < 0 || B < 0 || E > INT32_MAX || L > INT32_MAX || H * B > 65535) return MI_DECLINE_EXTENT;
    if (E == 0 || L == 0 || H == 0 || B == 0) return MI_OK;
    LeArgs a;
    a.out = (half_t *)out; a.in = (const half_t *)in;
    a.sE = in_strides[0]; a.sL = in_strides[1]; a.sH = in_strides[2]; a.sB = in_strides[3];
    if (out_strides) {
        if (out_strides[0] != 1 || out_strides[1] < L) return MI_DECLINE_OPERANDS;      // (L,E,H,B): L contiguous
        a.oE = out_strides[1]; a.oH = out_strides[2]; a.oB = out_strides[3];
    } else {
        a.oE = L; a.oH = L * E; a.oB = L * E * H;
    }
    if (a.sE < 0 || a.sL < 0 || a.sH < 0 || a.sB < 0) return MI_DECLINE_OPERANDS;
    a.E = (int)E; a.L = (int)L; a.H = (int)H;
    hipStream_t st = (hipStream_t)stream;
    if (a.sL == 1 && a.sE != 1) {
        if (ceil_div(E, 4) > 65535) return MI_DECLINE_EXTENT;
        hipLaunchKernelGGL(le_copy_kernel, dim3((unsigned)ceil_div(L, 64), (unsigned)ceil_div(E, 4), (unsigned)(H * B)), dim3(256), 0, st, a);
    } else {
        if (ceil_div(L, 32) > 65535) return MI_DECLINE_EXTENT;
        hipLaunchKernelGGL(le_tiled_kernel, dim3((unsigned)ceil_div(E, 32), (unsigned)ceil_div(L, 32), (unsigned)(H * B)), dim3(256), 0, st, a);
    }
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

// A hoisted [K][F] weight re-laid as [F][K], once at model load: the 2-D case of the transpose above.
extern "C" int mi_relayout_weight_f16(void *w_fk, int64_t ld_fk, const void *w_kf, int64_t ld_kf, int64_t K, int64_t F, void *stream) {
    if (ld_kf < F || ld_fk < K) return MI_DECLINE_EXTENT;
    const int64_t in_strides[4] = {1, ld_kf, 0, 0}, out_strides[4] = {1, ld_fk, 0, 0};
    return mi_transpose_le_f16(w_fk, out_strides, w_kf, in_strides, F, K, 1, 1, stream);
}
