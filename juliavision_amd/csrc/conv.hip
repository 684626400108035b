// Convolution as GEMM for gfx950, in the reference's layout:
//   x (W,H,Cin,N) = [N][Cin][H][W],  w (KW,KH,Cin,Cout) = [Cout][Cin][KH][KW],
//   out (OW,OH,Cout,N) = [N][Cout][OH][OW].
// Per image:  out[Cout][PQ] = w[Cout][CRS] . col[CRS][PQ]   (PQ = OH*OW pixels)
// so the weight is the K-contiguous operand as it lies, the pixel axis is the
// contiguous axis of both col and out, and the bias is per output ROW.
//   1x1 / stride 1 / no padding : col is x itself, no copy (conv.jl:63-66,117-131)
//   otherwise                   : im2col into scratch, then the same GEMM
//                                 (conv_coopmat.jl:246-392)
//   groups != 1                 : the direct kernel (conv.jl:26-51,298-302)
#include "common.hpp"

namespace {

struct ConvArgs {
    const half_t *x, *w, *bias;
    void *out;
    int Wi, Hi, Cin, N, KW, KH, Cout, OW, OH;
    int sx, sy, px, py, dx, dy, groups, relu;
};

// wp[co][CRSP] = w[co][CRS] zero-padded: the blocks of an im2col launch past its own work do this (image 0 only), so
// that padding the weights to the matrix's depth is not a launch of its own.
__device__ __forceinline__ void padweight_block(half_t *wp, const half_t *w, int Cout, int CRS, int CRSP, int block) {
    const int idx = block * blockDim.x + threadIdx.x;
    if (idx >= Cout * CRSP) return;
    const int c = idx % CRSP, co = idx / CRSP;
    wp[idx] = c < CRS ? w[(long)co * CRS + c] : (half_t)0.0f;
}

// col[c][m], m fastest: c = (ci, kh, kw) with kw fastest, m = (oh, ow) with ow
// fastest (the order of im2col_kernel!, conv_coopmat.jl:259-286).  Rows c >= CRS
// and columns m >= PQ are zero, as are taps that fall in the padding.  A thread
// produces eight consecutive pixels of one row c (one 16-byte store), so the
// index decomposition is paid once per eight elements; 32-bit arithmetic throughout.
__global__ void im2col_kernel(half_t *col, ConvArgs a, int PQP, int CRSP, half_t *wp, int col_blocks) {
    if ((int)blockIdx.x >= col_blocks) {
        if (blockIdx.y == 0) padweight_block(wp, a.w, a.Cout, a.Cin * a.KH * a.KW, CRSP, blockIdx.x - col_blocks);
        return;
    }
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int groups = PQP >> 3;
    if (idx >= groups * CRSP) return;
    const int n = blockIdx.y;
    const int m0 = (idx % groups) * 8, c = idx / groups;
    const int PQ = a.OW * a.OH, CRS = a.Cin * a.KH * a.KW;
    half8v val;
#pragma unroll
    for (int j = 0; j < 8; j++) val[j] = (half_t)0.0f;
    if (c < CRS) {
        const int kw = c % a.KW, t = c / a.KW, kh = t % a.KH, ci = t / a.KH;
        const half_t *xp = a.x + ((long)n * a.Cin + ci) * a.Hi * a.Wi;
        int ow = m0 % a.OW, oh = m0 / a.OW;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if (m0 + j < PQ) {
                const int ix = ow * a.sx - a.px + kw * a.dx, iy = oh * a.sy - a.py + kh * a.dy;
                if (ix >= 0 && ix < a.Wi && iy >= 0 && iy < a.Hi) val[j] = xp[iy * a.Wi + ix];
            }
            if (++ow == a.OW) { ow = 0; oh++; }
        }
    }
    *reinterpret_cast<half8v *>(col + (long)n * PQP * CRSP + (long)c * PQP + m0) = val;
}

// The same matrix token-major: col[n][m][c], c = (ci, kh, kw) fastest and zero from CRS to CRSP -- the row-major A
// operand of a GEMM whose output rows are pixels.  A thread gathers eight consecutive c of one pixel (one 16-byte store).
__global__ void im2col_rows_kernel(half_t *col, ConvArgs a, int CRSP, half_t *wp, int col_blocks) {
    if ((int)blockIdx.x >= col_blocks) {
        if (blockIdx.y == 0) padweight_block(wp, a.w, a.Cout, a.Cin * a.KH * a.KW, CRSP, blockIdx.x - col_blocks);
        return;
    }
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int groups = CRSP >> 3;
    const int PQ = a.OW * a.OH, CRS = a.Cin * a.KH * a.KW;
    if (idx >= groups * PQ) return;
    const int n = blockIdx.y;
    const int c0 = (idx % groups) * 8, m = idx / groups;
    const int ow = m % a.OW, oh = m / a.OW;
    const int ix0 = ow * a.sx - a.px, iy0 = oh * a.sy - a.py;
    int kw = c0 % a.KW, t = c0 / a.KW, kh = t % a.KH, ci = t / a.KH;
    const half_t *xp = a.x + (long)n * a.Cin * a.Hi * a.Wi;
    half8v val;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        val[j] = (half_t)0.0f;
        if (c0 + j < CRS) {
            const int ix = ix0 + kw * a.dx, iy = iy0 + kh * a.dy;
            if (ix >= 0 && ix < a.Wi && iy >= 0 && iy < a.Hi) val[j] = xp[((long)ci * a.Hi + iy) * a.Wi + ix];
        }
        if (++kw == a.KW) { kw = 0; if (++kh == a.KH) { kh = 0; ci++; } }
    }
    *reinterpret_cast<half8v *>(col + ((long)n * PQ + m) * CRSP + c0) = val;
}

// xp[n][ci][Hp][Wp]: x with py rows of zeros above and below and px (and the round-up to a multiple
// of 8) columns left and right; one 16-byte store per thread.  What the implicit-GEMM path reads.
// The same launch re-lays the weights as w2[co][kh][kw][ci] (blocks past the padding work, image 0
// only): the K order in which the implicit GEMM walks the taps.
__global__ void conv_pad_kernel(half_t *xp, half_t *w2, ConvArgs a, int Hp, int Wp, int pad_blocks, long shifted) {
    if ((int)blockIdx.x >= pad_blocks) {
        if (blockIdx.y != 0) return;
        // a thread gathers eight channels of one (co, tap) and stores them with one 16-byte write; with the tap
        // as the fastest thread index a wave reads a dense stretch of the source
        const int idx = (blockIdx.x - pad_blocks) * blockDim.x + threadIdx.x;
        const int taps = a.KH * a.KW, c8s = a.Cin >> 3;
        if (idx >= a.Cout * c8s * taps) return;
        const int tap = idx % taps, t = idx / taps, c8 = t % c8s, co = t / c8s;
        const half_t *src = a.w + ((long)co * a.Cin + c8 * 8) * taps + tap;
        half8v v;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = src[j * taps];
        *reinterpret_cast<half8v *>(w2 + ((long)co * taps + tap) * a.Cin + c8 * 8) = v;
        return;
    }
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int cpr = Wp >> 3;
    if (idx >= cpr * Hp * a.Cin) return;
    const int n = blockIdx.y;
    const int c8 = (idx % cpr) * 8, t = idx / cpr, yp = t % Hp, ci = t / Hp;
    const int iy = yp - a.py;
    // elements c8 .. c8+8 of the padded row: the first eight go to the copy proper, the last eight to the
    // copy that sits one element to the left (its chunk at the same position)
    half_t e[9];
#pragma unroll
    for (int j = 0; j < 9; j++) e[j] = (half_t)0.0f;
    if (iy >= 0 && iy < a.Hi) {
        const half_t *row = a.x + (((long)n * a.Cin + ci) * a.Hi + iy) * a.Wi;
#pragma unroll
        for (int j = 0; j < 9; j++) {
            const int ix = c8 + j - a.px;
            if (ix >= 0 && ix < a.Wi) e[j] = row[ix];
        }
    }
    half8v v0, v1;
#pragma unroll
    for (int j = 0; j < 8; j++) { v0[j] = e[j]; v1[j] = e[j + 1]; }
    const long at = (((long)n * a.Cin + ci) * Hp + yp) * Wp + c8;
    *reinterpret_cast<half8v *>(xp + at) = v0;
    *reinterpret_cast<half8v *>(xp + shifted + at) = v1;
}

// One thread per output; fp32 accumulator seeded with the bias; the loop order
// of the reference's conv2d (conv.jl:26-51).
__global__ void conv_direct_kernel(ConvArgs a) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)a.N * a.Cout * a.OH * a.OW;
    if (idx >= total) return;
    const int ox = (int)(idx % a.OW);
    long t = idx / a.OW;
    const int oy = (int)(t % a.OH); t /= a.OH;
    const int co = (int)(t % a.Cout);
    const int n = (int)(t / a.Cout);
    const int cing = a.Cin / a.groups, coutg = a.Cout / a.groups;
    const int g = co / coutg;
    float acc = a.bias ? (float)a.bias[co] : 0.0f;
    for (int ci = 0; ci < cing; ci++) {
        const int xc = g * cing + ci;
        for (int ky = 0; ky < a.KH; ky++) {
            const int iy = oy * a.sy - a.py + ky * a.dy;
            if (iy < 0 || iy >= a.Hi) continue;
            for (int kx = 0; kx < a.KW; kx++) {
                const int ix = ox * a.sx - a.px + kx * a.dx;
                if (ix < 0 || ix >= a.Wi) continue;
                acc = fmaf((float)a.x[(((long)n * a.Cin + xc) * a.Hi + iy) * a.Wi + ix],
                           (float)a.w[(((long)co * cing + ci) * a.KH + ky) * a.KW + kx], acc);
            }
        }
    }
    half_t r = (half_t)acc;
    if (a.relu && (float)r < 0.0f) r = (half_t)0.0f;
    reinterpret_cast<half_t *>(a.out)[idx] = r;
}

bool onebyone(const ConvArgs &a) {   // conv.jl:63-66
    return a.groups == 1 && a.KW == 1 && a.KH == 1 && a.sx == 1 && a.sy == 1 && a.px == 0 && a.py == 0 && a.dx == 1 && a.dy == 1;
}

int fill(ConvArgs &a, void *out, const void *x, const void *w, const void *bias,
         int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
         int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy, int64_t groups, int act) {
    if (Wi < 1 || Hi < 1 || Cin < 1 || N < 0 || KW < 1 || KH < 1 || Cout < 1) return MI_DECLINE_EXTENT;
    if (sx < 1 || sy < 1 || dx < 1 || dy < 1 || px < 0 || py < 0 || groups < 1) return MI_DECLINE_EXTENT;
    if (Cin % groups || Cout % groups) return MI_DECLINE_EXTENT;
    if (act != MI_EPI_NONE && act != MI_EPI_RELU) return MI_DECLINE_UNSUPPORTED;
    int64_t OW = mi_convsize(Wi, KW, sx, px, dx), OH = mi_convsize(Hi, KH, sy, py, dy);
    if (OW < 1 || OH < 1) return MI_DECLINE_EXTENT;
    if (Wi * Hi * Cin > INT32_MAX || OW * OH * Cout > INT32_MAX || Cin * KW * KH > INT32_MAX / 8 || N > 65535) return MI_DECLINE_EXTENT;
    a.x = (const half_t *)x; a.w = (const half_t *)w; a.bias = (const half_t *)bias; a.out = out;
    a.Wi = (int)Wi; a.Hi = (int)Hi; a.Cin = (int)Cin; a.N = (int)N; a.KW = (int)KW; a.KH = (int)KH; a.Cout = (int)Cout;
    a.OW = (int)OW; a.OH = (int)OH;
    a.sx = (int)sx; a.sy = (int)sy; a.px = (int)px; a.py = (int)py; a.dx = (int)dx; a.dy = (int)dy;
    a.groups = (int)groups; a.relu = act == MI_EPI_RELU;
    return MI_OK;
}

// Implicit GEMM needs eight consecutive output pixels to be eight consecutive input columns (stride 1
// along x, OW a multiple of 8) and 64-deep K tiles that are 64 channels of one tap (Cin % 64 == 0).
bool implicit_ok(const ConvArgs &a) {
    return a.sx == 1 && a.OW % 8 == 0 && a.Cin % 64 == 0 && (long)a.Cin * a.KH * a.KW >= 128;
}

int conv_path(const ConvArgs &a) {
    if (a.groups != 1) return MI_CONV_DIRECT;
    if (onebyone(a)) return MI_CONV_GEMM_1X1;
    if (implicit_ok(a)) return MI_CONV_IMPLICIT_GEMM;
    return MI_CONV_IM2COL_GEMM;
}

void padded_extents(const ConvArgs &a, int &Hp, int &Wp) {
    Hp = a.Hi + 2 * a.py;
    Wp = (int)round_up((size_t)(a.Wi + 2 * a.px), 8);
}

// The matrix is padded with zero rows to a multiple of 8 taps, and -- from 256 taps on, where that adds a quarter at
// most -- to a multiple of 64, the depth the software-pipelined GEMM steps by (a ViT's 14 x 14 x 3 patch: 588 -> 640).
void im2col_extents(const ConvArgs &a, int64_t &PQP, int64_t &CRSP) {
    const size_t CRS = (size_t)a.Cin * a.KH * a.KW;
    PQP = round_up((size_t)a.OW * a.OH, 8);
    CRSP = round_up(CRS, CRS >= 256 ? 64 : 8);
}

}  // namespace

extern "C" {

int64_t mi_convsize(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d) { return (n + 2 * p - d * (k - 1) - 1) / s + 1; }

int mi_conv2d_f16_plan(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                       int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy, int64_t groups) {
    ConvArgs a;
    if (fill(a, nullptr, nullptr, nullptr, nullptr, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, groups, MI_EPI_NONE) != MI_OK)
        return MI_CONV_DECLINE;
    return conv_path(a);
}

size_t mi_conv2d_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                               int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy) {
    ConvArgs a;
    if (fill(a, nullptr, nullptr, nullptr, nullptr, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, 1, MI_EPI_NONE) != MI_OK) return 0;
    if (conv_path(a) == MI_CONV_IMPLICIT_GEMM) {
        int Hp, Wp;
        padded_extents(a, Hp, Wp);
        return 2 * round_up((size_t)N * Cin * Hp * Wp * 2, 256) + round_up((size_t)Cout * Cin * KH * KW * 2, 256) +
               mi_internal_gemm_workspace(Cout, Cin * KH * KW, (int64_t)a.OW * a.OH, N);
    }
    if (conv_path(a) != MI_CONV_IM2COL_GEMM) return 0;
    int64_t PQP, CRSP;
    im2col_extents(a, PQP, CRSP);
    size_t col = round_up((size_t)N * PQP * CRSP * 2, 256);
    size_t wp = CRSP != (int64_t)Cin * KH * KW ? round_up((size_t)Cout * CRSP * 2, 256) : 0;
    return col + wp + mi_internal_gemm_workspace(Cout, CRSP, (int64_t)a.OW * a.OH, N);
}

int mi_conv2d_f16(void *out, const void *x, const void *w, const void *bias,
                  int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                  int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy, int64_t groups, int act,
                  void *ws, size_t ws_bytes, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !x || !w) return MI_DECLINE_OPERANDS;
    ConvArgs a;
    int rc = fill(a, out, x, w, bias, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, groups, act);
    if (rc != MI_OK) return rc;
    if (N == 0) return MI_OK;
    hipStream_t st = (hipStream_t)stream;
    const int path = conv_path(a);
    const int PQ = a.OW * a.OH;
    const int epi = a.relu ? MI_EPI_RELU : MI_EPI_NONE;
    if (path == MI_CONV_DIRECT) {
        long total = (long)a.N * a.Cout * PQ;
        hipLaunchKernelGGL(conv_direct_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, a);
        return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
    }
    if (path == MI_CONV_GEMM_1X1) {
        // out[n][Cout][PQ] = w[Cout][Cin] . x[n][Cin][PQ]; the [K][N] operand needs
        // PQ % 8 == 0 for 16-byte loads, otherwise the scalar GEMM takes it.
        return mi_internal_gemm(out, w, x, bias, a.Cout, PQ, PQ, a.Cin, PQ, a.Cin, PQ, 1, MI_BIAS_ROW, epi, 0,
                                a.N, (long)a.Cout * PQ, 0, (long)a.Cin * PQ, nullptr, 0, st);
    }
    if (path == MI_CONV_IMPLICIT_GEMM) {
        int Hp, Wp;
        padded_extents(a, Hp, Wp);
        const int CRS = a.Cin * a.KH * a.KW;
        const size_t xp1 = round_up((size_t)a.N * a.Cin * Hp * Wp * 2, 256), xp_bytes = 2 * xp1;     // the copy and its shifted twin
        const size_t w2_bytes = round_up((size_t)a.Cout * CRS * 2, 256);
        const size_t gemm_bytes = mi_internal_gemm_workspace(a.Cout, CRS, PQ, a.N);
        if (!ws || ws_bytes < xp_bytes + w2_bytes + gemm_bytes || !aligned_to(ws, 256)) return MI_DECLINE_WORKSPACE;
        if ((long)a.Cin * Hp * Wp > INT32_MAX || (long)a.Cout * CRS > INT32_MAX) return MI_DECLINE_EXTENT;
        half_t *xp = reinterpret_cast<half_t *>(ws);
        half_t *w2 = reinterpret_cast<half_t *>(reinterpret_cast<char *>(ws) + xp_bytes);
        const int pad_blocks = (int)ceil_div((int64_t)(Wp / 8) * Hp * a.Cin, 256), w_blocks = (int)ceil_div((int64_t)a.Cout * CRS / 8, 256);
        hipLaunchKernelGGL(conv_pad_kernel, dim3((unsigned)(pad_blocks + w_blocks), (unsigned)a.N), dim3(256), 0, st, xp, w2, a, Hp, Wp, pad_blocks, (long)(xp1 / 2));
        if (hipGetLastError() != hipSuccess) return MI_ERROR_LAUNCH;
        ConvGather g;
        g.xp = xp; g.img = (long)a.Cin * Hp * Wp; g.odd = (long)(xp1 / 2) - 1; g.HpWp = Hp * Wp; g.Wp = Wp; g.OW = a.OW; g.sy = a.sy;
        g.dyWp = a.dy * Wp; g.dx = a.dx; g.KW = a.KW; g.cpt = a.Cin / 64; g.split = 0;
        // B is never dereferenced in this mode; xp stands in so that the operand checks see an aligned pointer
        return mi_internal_gemm(out, w2, xp, bias, a.Cout, PQ, PQ, CRS, PQ, CRS, PQ, 1, MI_BIAS_ROW, epi, 0,
                                a.N, (long)a.Cout * PQ, 0, 0, reinterpret_cast<char *>(ws) + xp_bytes + w2_bytes, gemm_bytes, st, &g);
    }
    int64_t PQP, CRSP;
    im2col_extents(a, PQP, CRSP);
    const int CRS = a.Cin * a.KH * a.KW;
    size_t col_bytes = round_up((size_t)N * PQP * CRSP * 2, 256);
    size_t wp_bytes = CRSP != CRS ? round_up((size_t)Cout * CRSP * 2, 256) : 0;
    const size_t gemm_bytes = mi_internal_gemm_workspace(Cout, CRSP, PQ, N);
    if (!ws || ws_bytes < col_bytes + wp_bytes + gemm_bytes || !aligned_to(ws, 256)) return MI_DECLINE_WORKSPACE;
    if (PQP * CRSP > INT32_MAX) return MI_DECLINE_EXTENT;
    half_t *col = reinterpret_cast<half_t *>(ws);
    const half_t *wuse = a.w;
    half_t *wp = wp_bytes ? reinterpret_cast<half_t *>(reinterpret_cast<char *>(ws) + col_bytes) : nullptr;
    const int col_blocks = (int)ceil_div(PQP / 8 * CRSP, 256), w_blocks = wp ? (int)ceil_div((int64_t)Cout * CRSP, 256) : 0;
    hipLaunchKernelGGL(im2col_kernel, dim3((unsigned)(col_blocks + w_blocks), (unsigned)a.N), dim3(256), 0, st, col, a, (int)PQP, (int)CRSP, wp, col_blocks);
    if (wp) wuse = wp;
    if (hipGetLastError() != hipSuccess) return MI_ERROR_LAUNCH;
    return mi_internal_gemm(out, wuse, col, bias, a.Cout, PQ, (int)PQP, (int)CRSP, PQ, CRSP, PQP, 1, MI_BIAS_ROW, epi, 0,
                            a.N, (long)a.Cout * PQ, 0, PQP * CRSP, reinterpret_cast<char *>(ws) + col_bytes + wp_bytes, gemm_bytes, st);
}

// The convolution with its output token-major: out[n][m][co], m = (oh, ow), a row of Cout values per pixel at pitch
// ld_out, images out_image_stride apart -- what a patch embedding's flatten + transpose makes of the channel-major
// result -- and optionally + residual[n][m][co] (same pitch, images res_image_stride apart, 0 = one for all: the
// position embedding).  out[m][co] = col[m][c] . w[co][c]^T: the im2col matrix written token-major is the row-major
// operand, the weights are the K-contiguous one as they lie (padded to the matrix's depth), the bias is per column
// and the residual joins in the GEMM's store with one more rounding, like an add after the convolution.
size_t mi_conv2d_tokens_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                                      int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy) {
    ConvArgs a;
    if (fill(a, nullptr, nullptr, nullptr, nullptr, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, 1, MI_EPI_NONE) != MI_OK) return 0;
    int64_t PQP, CRSP;
    im2col_extents(a, PQP, CRSP);
    const int64_t PQ = (int64_t)a.OW * a.OH;
    const size_t col = round_up((size_t)N * PQ * CRSP * 2, 256);
    const size_t wp = CRSP != (int64_t)Cin * KH * KW ? round_up((size_t)Cout * CRSP * 2, 256) : 0;
    return col + wp + mi_internal_gemm_workspace(PQ, CRSP, Cout, 1);
}

int mi_conv2d_tokens_f16(void *out, int64_t ld_out, int64_t out_image_stride,
                         const void *x, const void *w, const void *bias, const void *residual, int64_t res_image_stride,
                         int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                         int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy, int act,
                         void *ws, size_t ws_bytes, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !x || !w) return MI_DECLINE_OPERANDS;
    ConvArgs a;
    int rc = fill(a, out, x, w, bias, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, 1, act);
    if (rc != MI_OK) return rc;
    if (N == 0) return MI_OK;
    const int64_t PQ = (int64_t)a.OW * a.OH;
    if (ld_out < Cout || (N > 1 && out_image_stride < PQ * ld_out) || res_image_stride < 0) return MI_DECLINE_EXTENT;
    if (ld_out % 8 || out_image_stride % 8 || res_image_stride % 8 || !aligned_to(out, 16) || (residual && !aligned_to(residual, 16)))
        return MI_DECLINE_OPERANDS;
    hipStream_t st = (hipStream_t)stream;
    int64_t PQP, CRSP;
    im2col_extents(a, PQP, CRSP);
    const int CRS = a.Cin * a.KH * a.KW;
    const size_t col_bytes = round_up((size_t)N * PQ * CRSP * 2, 256);
    const size_t wp_bytes = CRSP != CRS ? round_up((size_t)Cout * CRSP * 2, 256) : 0;
    const size_t gemm_bytes = mi_internal_gemm_workspace(PQ, CRSP, Cout, 1);
    if (!ws || ws_bytes < col_bytes + wp_bytes + gemm_bytes || !aligned_to(ws, 256)) return MI_DECLINE_WORKSPACE;
    if (PQ * CRSP > INT32_MAX) return MI_DECLINE_EXTENT;
    half_t *col = reinterpret_cast<half_t *>(ws);
    const half_t *wuse = a.w;
    half_t *wp = wp_bytes ? reinterpret_cast<half_t *>(reinterpret_cast<char *>(ws) + col_bytes) : nullptr;
    const int col_blocks = (int)ceil_div(PQ * (CRSP / 8), 256), w_blocks = wp ? (int)ceil_div((int64_t)Cout * CRSP, 256) : 0;
    hipLaunchKernelGGL(im2col_rows_kernel, dim3((unsigned)(col_blocks + w_blocks), (unsigned)a.N), dim3(256), 0, st, col, a, (int)CRSP, wp, col_blocks);
    if (wp) wuse = wp;
    if (hipGetLastError() != hipSuccess) return MI_ERROR_LAUNCH;
    const int epi = a.relu ? MI_EPI_RELU : MI_EPI_NONE;
    void *gws = reinterpret_cast<char *>(ws) + col_bytes + wp_bytes;
    // the residual is addressed like the output; images whose residuals lie at another distance go one launch each
    const bool together = !residual || N == 1 || res_image_stride == out_image_stride;
    for (int64_t n = 0; n < (together ? 1 : N); n++) {
        half_t *yo = reinterpret_cast<half_t *>(out) + n * out_image_stride;
        const half_t *ro = residual ? reinterpret_cast<const half_t *>(residual) + n * res_image_stride : nullptr;
        rc = mi_internal_gemm(yo, col + n * PQ * CRSP, wuse, bias, (int)PQ, a.Cout, a.Cout, (int)CRSP, ld_out, CRSP, CRSP, 0, MI_BIAS_COL, epi, 0,
                              together ? N : 1, out_image_stride, PQ * CRSP, 0, gws, gemm_bytes, st, nullptr, nullptr, ro);
        if (rc != MI_OK) return rc;
    }
    return MI_OK;
}

// Channels-last convolution as an implicit GEMM with nothing staged: out[(n,oh,ow)][Cout] = patch[(n,oh,ow)][(kh,kw,ci)] .
// w[Cout][(kh,kw,ci)]^T.  The patch matrix is gathered from x by the GEMM's A-operand loads (64 channels of one tap
// are 128 contiguous bytes of a pixel; taps outside the image load zeros), the weights are the K-contiguous operand
// as they lie, the bias is per output column: no padded copy, no re-laid weights, no im2col.
size_t mi_conv2d_nhwc_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                                    int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy) {
    ConvArgs a;
    if (fill(a, nullptr, nullptr, nullptr, nullptr, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, 1, MI_EPI_NONE) != MI_OK) return 0;
    return mi_internal_gemm_workspace((int64_t)N * a.OH * a.OW, Cin * KH * KW, Cout, 1);
}

int mi_conv2d_nhwc_f16(void *out, const void *x, const void *w, const void *bias,
                       int64_t Wi, int64_t Hi, int64_t Cin, int64_t N, int64_t KW, int64_t KH, int64_t Cout,
                       int64_t sx, int64_t sy, int64_t px, int64_t py, int64_t dx, int64_t dy, int act,
                       void *ws, size_t ws_bytes, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !x || !w) return MI_DECLINE_OPERANDS;
    ConvArgs a;
    int rc = fill(a, out, x, w, bias, Wi, Hi, Cin, N, KW, KH, Cout, sx, sy, px, py, dx, dy, 1, act);
    if (rc != MI_OK) return rc;
    if (N == 0) return MI_OK;
    const int64_t M = (int64_t)N * a.OH * a.OW, K = Cin * KH * KW;
    // the gathered operand is read in runs of 64 channels; other channel counts go through the reference layout
    if (Cin % 64 || K < 128 || M > INT32_MAX || K > INT32_MAX || Cout % 8) return MI_DECLINE_UNSUPPORTED;
    if (!aligned_to(x, 16) || !aligned_to(w, 16) || !aligned_to(out, 16)) return MI_DECLINE_OPERANDS;
    NhwcGather g;
    g.x = (const half_t *)x; g.H = a.Hi; g.W = a.Wi; g.C = a.Cin; g.OH = a.OH; g.OW = a.OW;
    g.sx = a.sx; g.sy = a.sy; g.px = a.px; g.py = a.py; g.dx = a.dx; g.dy = a.dy; g.KW = a.KW; g.cpt = a.Cin / 64; g.split = 0;
    const int epi = a.relu ? MI_EPI_RELU : MI_EPI_NONE;
    // A is never dereferenced through its pointer and leading dimension in this mode; x and K stand in for the operand checks
    return mi_internal_gemm(out, x, w, bias, (int)M, (int)Cout, (int)Cout, (int)K, Cout, K, K, 0, MI_BIAS_COL, epi, 0,
                            1, 0, 0, 0, ws, ws_bytes, (hipStream_t)stream, nullptr, &g);
}

}  // extern "C"
