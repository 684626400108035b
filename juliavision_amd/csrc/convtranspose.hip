// Transposed convolution for gfx950, in the reference's layout:
//   x (W,H,Cin,N) = [N][Cin][H][W],  w (KW,KH,Cout/g,Cin) = [Cin][Cout/g][KH][KW] (torch's
//   conv_transpose2d weight),  out (OW,OH,Cout,N) = [N][Cout][OH][OW].
// Two routes, as the reference has them (conv.jl:204-294):
//   kernel == stride, no padding / dilation / output padding, one group:
//       every output pixel has exactly one source pixel and one tap, so per image
//           y[(co,ky,kx)][H*W] = w2[(co,ky,kx)][Cin] . x[Cin][H*W]        (one GEMM, MFMA)
//           out[co][iy*KH+ky][ix*KW+kx] = y[(co,ky,kx)][iy*W+ix]          (pixel shuffle)
//       The bias is expanded to one value per GEMM row, so y is already the rounded result and
//       the shuffle only moves bits.
//   anything else: one thread per output gathers the inputs that reach it (conv.jl:149-191).
#include "common.hpp"

namespace {

struct CtArgs {
    const half_t *x, *w, *bias;
    half_t *out;
    int Wi, Hi, Cin, N, KW, KH, Cout, OW, OH;
    int sx, sy, px, py, dx, dy, groups;
};

// w2[(co,ky,kx)][ci] = w[ci][(co,ky,kx)] (a 2-D transpose through LDS, 32x32 tiles) and, from the
// blocks past the transpose, bias2[(co,ky,kx)] = bias[co].
__global__ void ct_prepare_kernel(half_t *w2, half_t *bias2, const half_t *w, const half_t *bias, int Cin, int M, int taps,
                                  int tiles_m, int tile_blocks) {
    if ((int)blockIdx.x >= tile_blocks) {
        const int r = ((int)blockIdx.x - tile_blocks) * 256 + threadIdx.x;
        if (r < M) bias2[r] = bias ? bias[r / taps] : (half_t)0.0f;
        return;
    }
    __shared__ half_t tile[32][33];
    const int tm = ((int)blockIdx.x % tiles_m) * 32, tk = ((int)blockIdx.x / tiles_m) * 32;
    const int lx = threadIdx.x & 31, ly = threadIdx.x >> 5;       // 256 threads: 8 rows a pass
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int k = tk + ly + 8 * p, m = tm + lx;
        tile[ly + 8 * p][lx] = (k < Cin && m < M) ? w[(long)k * M + m] : (half_t)0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int m = tm + ly + 8 * p, k = tk + lx;
        if (m < M && k < Cin) w2[(long)m * Cin + k] = tile[lx][ly + 8 * p];
    }
}

// out[n][co][iy*KH+ky][ix*KW+kx] = y[n][(co,ky,kx)][iy*W+ix].  A thread produces VEC consecutive
// outputs of one output row (one 16-byte store when VEC is 8).
template <int VEC>
__global__ void ct_shuffle_kernel(half_t *out, const half_t *y, int Wi, int Hi, int KW, int KH, int Cout) {
    const int OW = Wi * KW, OH = Hi * KH;
    const int per_row = OW / VEC;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)Cout * OH * per_row;
    if (idx >= total) return;
    const int n = blockIdx.y;
    const int ox0 = (int)(idx % per_row) * VEC;
    long t = idx / per_row;
    const int oy = (int)(t % OH), co = (int)(t / OH);
    const int iy = oy / KH, ky = oy % KH;
    const long HW = (long)Hi * Wi;
    const half_t *src = y + ((long)n * Cout * KH * KW + ((long)co * KH + ky) * KW) * HW + (long)iy * Wi;
    half_t *dst = out + (((long)n * Cout + co) * OH + oy) * OW + ox0;
    if constexpr (VEC == 8) {
        half8v v;
        int ix = ox0 / KW, kx = ox0 % KW;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            v[j] = src[kx * HW + ix];
            if (++kx == KW) { kx = 0; ix++; }
        }
        *reinterpret_cast<half8v *>(dst) = v;
    } else {
        dst[0] = src[(ox0 % KW) * HW + ox0 / KW];
    }
}

// The gather form: the loop order and the fp32 accumulator (seeded with the bias) of the reference's
// convtranspose2d (conv.jl:149-191).
__global__ void ct_gather_kernel(CtArgs a) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)a.N * a.Cout * a.OH * a.OW;
    if (idx >= total) return;
    const int ox = (int)(idx % a.OW);
    long t = idx / a.OW;
    const int oy = (int)(t % a.OH); t /= a.OH;
    const int co = (int)(t % a.Cout);
    const int n = (int)(t / a.Cout);
    const int cing = a.Cin / a.groups, coutg = a.Cout / a.groups;
    const int g = co / coutg, cog = co % coutg;
    float acc = a.bias ? (float)a.bias[co] : 0.0f;
    const int bx = ox + a.px, by = oy + a.py;
    for (int ci = g * cing; ci < (g + 1) * cing; ci++) {
        const half_t *xc = a.x + ((long)n * a.Cin + ci) * a.Hi * a.Wi;
        const half_t *wc = a.w + ((long)ci * coutg + cog) * a.KH * a.KW;
        for (int ky = 0; ky < a.KH; ky++) {
            const int ty = by - ky * a.dy;
            if (ty < 0 || ty % a.sy != 0) continue;
            const int iy = ty / a.sy;
            if (iy >= a.Hi) continue;
            for (int kx = 0; kx < a.KW; kx++) {
                const int tx = bx - kx * a.dx;
                if (tx < 0 || tx % a.sx != 0) continue;
                const int ix = tx / a.sx;
                if (ix >= a.Wi) continue;
                acc = fmaf((float)xc[iy * a.Wi + ix], (float)wc[ky * a.KW + kx], acc);
            }
        }
    }
    a.out[idx] = (half_t)acc;
}

int fill(CtArgs &a, void *out, const void *x, const void *w, const void *bias,
         int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
         int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy, int64_t opx, int64_t opy, int64_t groups) {
    if (Wi < 1 || Hi < 1 || Cin < 1 || N < 0 || KW < 1 || KH < 1 || Cout < 1) return MI_DECLINE_EXTENT;
    if (sx < 1 || sy < 1 || dx < 1 || dy < 1 || px < 0 || py < 0 || opx < 0 || opy < 0 || groups < 1) return MI_DECLINE_EXTENT;
    if (Cin % groups || Cout % groups) return MI_DECLINE_EXTENT;
    // ATen's rule: the output padding fills the gap a stride (or dilation) leaves, no more
    if ((opx >= sx && opx >= dx) || (opy >= sy && opy >= dy)) return MI_DECLINE_EXTENT;
    const int64_t OW = mi_convtransposesize(Wi, KW, sx, px, dx, opx), OH = mi_convtransposesize(Hi, KH, sy, py, dy, opy);
    if (OW < 1 || OH < 1) return MI_DECLINE_EXTENT;
    if (Wi * Hi * Cin > INT32_MAX || OW * OH * Cout > INT32_MAX || Cin * (Cout / groups) * KW * KH > INT32_MAX || N > 65535) return MI_DECLINE_EXTENT;
    a.x = (const half_t *)x; a.w = (const half_t *)w; a.bias = (const half_t *)bias; a.out = (half_t *)out;
    a.Wi = (int)Wi; a.Hi = (int)Hi; a.Cin = (int)Cin; a.N = (int)N; a.KW = (int)KW; a.KH = (int)KH; a.Cout = (int)Cout;
    a.OW = (int)OW; a.OH = (int)OH;
    a.sx = (int)sx; a.sy = (int)sy; a.px = (int)px; a.py = (int)py; a.dx = (int)dx; a.dy = (int)dy; a.groups = (int)groups;
    return MI_OK;
}

// shufflecase, conv.jl:204-209; the output padding is zero by the caller's check
bool shuffle_ok(const CtArgs &a, int64_t opx, int64_t opy) {
    return a.groups == 1 && a.px == 0 && a.py == 0 && a.dx == 1 && a.dy == 1 && opx == 0 && opy == 0 && a.KW == a.sx && a.KH == a.sy;
}

struct CtScratch { size_t w2, bias2, y, gemm; };

CtScratch scratch_of(const CtArgs &a) {
    const int64_t M = (int64_t)a.Cout * a.KH * a.KW, HW = (int64_t)a.Hi * a.Wi;
    CtScratch s;
    s.w2 = round_up((size_t)M * a.Cin * 2, 256);
    s.bias2 = round_up((size_t)M * 2, 256);
    s.y = round_up((size_t)a.N * M * HW * 2, 256);
    s.gemm = mi_internal_gemm_workspace(M, a.Cin, HW, a.N);
    return s;
}

}  // namespace

extern "C" {

int64_t mi_convtransposesize(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d, int64_t op) {
    return (n - 1) * s - 2 * p + d * (k - 1) + op + 1;
}

int mi_convtranspose2d_f16_plan(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                                int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy,
                                int64_t opx, int64_t opy, int64_t groups) {
    CtArgs a;
    if (fill(a, nullptr, nullptr, nullptr, nullptr, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, opx, opy, groups) != MI_OK)
        return MI_CONVT_DECLINE;
    return shuffle_ok(a, opx, opy) ? MI_CONVT_GEMM_SHUFFLE : MI_CONVT_GATHER;
}

size_t mi_convtranspose2d_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                                        int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy,
                                        int64_t opx, int64_t opy, int64_t groups) {
    CtArgs a;
    if (fill(a, nullptr, nullptr, nullptr, nullptr, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, opx, opy, groups) != MI_OK) return 0;
    if (!shuffle_ok(a, opx, opy)) return 0;
    const CtScratch s = scratch_of(a);
    return s.w2 + s.bias2 + s.y + s.gemm;
}

int mi_convtranspose2d_f16(void *out, const void *x, const void *w, const void *bias,
                           int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                           int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy,
                           int64_t opx, int64_t opy, int64_t groups, void *ws, size_t ws_bytes, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !x || !w) return MI_DECLINE_OPERANDS;
    CtArgs a;
    int rc = fill(a, out, x, w, bias, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, opx, opy, groups);
    if (rc != MI_OK) return rc;
    if (N == 0) return MI_OK;
    hipStream_t st = (hipStream_t)stream;
    if (!shuffle_ok(a, opx, opy)) {
        const long total = (long)a.N * a.Cout * a.OH * a.OW;
        if (ceil_div(total, 256) > INT32_MAX) return MI_DECLINE_EXTENT;
        hipLaunchKernelGGL(ct_gather_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, a);
        return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
    }
    const CtScratch s = scratch_of(a);
    if (!ws || ws_bytes < s.w2 + s.bias2 + s.y + s.gemm || !aligned_to(ws, 256)) return MI_DECLINE_WORKSPACE;
    const int M = a.Cout * a.KH * a.KW, HW = a.Hi * a.Wi, taps = a.KH * a.KW;
    char *base = reinterpret_cast<char *>(ws);
    half_t *w2 = reinterpret_cast<half_t *>(base);
    half_t *bias2 = reinterpret_cast<half_t *>(base + s.w2);
    half_t *y = reinterpret_cast<half_t *>(base + s.w2 + s.bias2);
    const int tiles_m = (int)ceil_div((int64_t)M, 32), tile_blocks = tiles_m * (int)ceil_div((int64_t)a.Cin, 32);
    hipLaunchKernelGGL(ct_prepare_kernel, dim3((unsigned)(tile_blocks + (int)ceil_div((int64_t)M, 256))), dim3(256), 0, st,
                       w2, bias2, a.w, a.bias, a.Cin, M, taps, tiles_m, tile_blocks);
    if (hipGetLastError() != hipSuccess) return MI_ERROR_LAUNCH;
    // y[n][M][HW] = w2[M][Cin] . x[n][Cin][HW]: the pixel axis is the contiguous one of both, the expanded bias is per row
    rc = mi_internal_gemm(y, w2, a.x, a.bias ? bias2 : nullptr, M, HW, HW, a.Cin, HW, a.Cin, HW, 1, MI_BIAS_ROW, MI_EPI_NONE, 0,
                          a.N, (long)M * HW, 0, (long)a.Cin * HW, base + s.w2 + s.bias2 + s.y, s.gemm, st);
    if (rc != MI_OK) return rc;
    if (a.OW % 8 == 0 && aligned_to(out, 16)) {
        const long total = (long)a.Cout * a.OH * (a.OW / 8);
        hipLaunchKernelGGL(ct_shuffle_kernel<8>, dim3((unsigned)ceil_div(total, 256), (unsigned)a.N), dim3(256), 0, st,
                           a.out, y, a.Wi, a.Hi, a.KW, a.KH, a.Cout);
    } else {
        const long total = (long)a.Cout * a.OH * a.OW;
        hipLaunchKernelGGL(ct_shuffle_kernel<1>, dim3((unsigned)ceil_div(total, 256), (unsigned)a.N), dim3(256), 0, st,
                           a.out, y, a.Wi, a.Hi, a.KW, a.KH, a.Cout);
    }
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

}  // extern "C"
