// fp16 GEMM for gfx950: MFMA 32x32x16 f16 with fp32 accumulation, LDS
// double-buffered operand tiles, 128-bit global loads, fused bias / activation /
// residual store; a split-K bandwidth kernel for decode-sized T; a scalar
// kernel for operands the tiled kernels cannot address.
//
// Internal problem statement (row-major):  Y[M x N] = A[M x K] . B  (+ bias)
//   A is K-contiguous.  B is either N-contiguous [K][N] (B_KN) or K-contiguous
//   [N][K].  For a linear layer M = tokens, N = features, A = X, B = W.
#include "common.hpp"
#include "sk_exchange.hpp"
#include <type_traits>
#include <atomic>

// Arrival flags of the split-K peer reduction (gemm_w4_kernel, SK): SK_BANKS banks of SK_FLAGS words, and as many
// counters behind them (word i's counter is word i + SK_WORDS).  A launch uses the bank its epoch selects, so launches
// that overlap on one GPU (up to SK_BANKS of them) do not see each other's.  Every word is zero when the module loads
// and zero again when a launch ends: the last consumer of a flag clears it (and its counter), so a captured launch --
// whose epoch and bank are fixed at capture -- starts every replay from clean flags.
constexpr int SK_BANKS = 16, SK_FLAGS = 4096, SK_WORDS = SK_BANKS * SK_FLAGS;
static __device__ unsigned sk_flag_words[2 * SK_WORDS];

// Sticky device status word (mi_device_status): kernels OR a bit of enum mi_device_status_bits into word 0 when a
// bounded wait inside a launch gave up; nothing on the device ever clears it.
static __device__ unsigned device_status_words[4];

// Static device scratch of the allocation-free entry point (see mi_gemm_f16_noalloc).
static __device__ __align__(256) unsigned char scratch[MI_NOALLOC_SCRATCH_BYTES];

namespace {

struct GemmArgs {
    void *Y;
    const half_t *A, *B, *bias, *residual;
    int M, N, K;
    int NB;                 // columns addressable in B (>= N; a multiple of 8 for the [K][N] layout)
    long ldY, ldA, ldB;
    long sY, sA, sB, sBias; // batch strides (elements)
    int bias_mode, epi, out_f32;
    int tiles_m, tiles_n, group_m;
    int vec_store;          // Y (and residual) rows allow 16-byte accesses
    ConvGather cv;          // cv.xp != nullptr: B is the im2col matrix of a convolution, gathered on the fly
    NhwcGather ag;          // ag.x != nullptr: A is the patch matrix of a channels-last convolution, gathered on the fly
    // Decode-sized kernels only: the rows of A are layer-normalised over K on their way into LDS
    // (ln_on; gamma, beta may be null), exactly as layernorm_vec_kernel would have written them.
    const half_t *ln_gamma, *ln_beta;
    float ln_eps;
    int ln_on;
    // Output side: when lnout is set, the rows of Y are also layer-normalised over N into lnout (dense rows of N
    // halves), as mi_layernorm_f16 on Y would write them (the next block's first norm riding in this GEMM's store).
    half_t *lnout;
    const half_t *lnout_gamma, *lnout_beta;
    float lnout_eps;
    // Tiled kernels and the split-K plane sums: > 0 clamps the fp16 result to [-clamp, clamp] after the residual add,
    // as a separate aten::clamp on Y would (the overflow guard of exported fp16 encoder layers).
    float clamp;
    // Measurement only (mi_set_clock_probe): workgroup 0 of a four-wave launch stores {shader clock, 100 MHz clock}
    // here when it starts and again after its last store.  Null in ordinary use.
    unsigned long long *clk;
    // Measurement only (mi_set_phase_probe): every matrix wave of the first phase_wgs workgroups of a four-wave launch
    // stores the shader clocks it spent {before its K loop, in it, issuing its store, waiting for the store to drain}.
    unsigned long long *phase;
    int phase_wgs;
    // Split-K with the partial tiles exchanged between the workgroups of a tile instead of written as planes
    // (gemm_w4_kernel, SK instance): sk_S = 2 workgroups per tile, tiles dealt sk_tpx per XCD; partials in sk_part,
    // per-wave arrival flags in sk_flags (they carry sk_epoch; the last reader of a flag clears it).
    int sk_S, sk_tpx;
    float *sk_part;
    unsigned *sk_flags;
    unsigned sk_epoch;
    // Layer norm folded away (mi_lnfold_gemm_f16): A holds the raw rows, B carries gamma, and the store turns an
    // accumulator into r (acc - mu colsum[n]) + biasp[n], with the row's (mu, r) combined from lnf_stats.
    const float *lnf_stats;           // [lnf_nseg][M][2]: (sum, squares about its own mean) of each 32-column segment of a row
    const float *lnf_colsum, *lnf_biasp;      // fp32[N], plane stride lnf_svec
    long lnf_svec;
    int lnf_nseg;
    float lnf_eps;
    // Row statistics of the result for a later folded norm: stats_out[n / 32][m] = (sum, squares about the mean) of the
    // final fp16 values Y[m][32 (n / 32) .. + 32); stats_nseg segments per row.
    float *stats_out;
    int stats_nseg;
    int sk_spin;                      // polls before a wave gives up on its partners
    unsigned sk_pub_xor, sk_xcc_xor;  // zero in ordinary use: mi_test_exchange_faults makes the waits fail from the host side
    unsigned *status;                 // the device's sticky status word
};

// ------------------------------------------------------------------------------------------
// Staging of a K-contiguous operand tile ROWS x BK: each thread moves 16-byte
// chunks global -> registers -> LDS rows of BK+8 halves (the 16-byte pad makes
// the 32 rows an MFMA operand read touches fall in distinct bank groups).
template <int ROWS, int BK, int NT>
struct KcStage {
    static constexpr int CPR = BK / 8;
    static constexpr int CHUNKS = ROWS * CPR;
    static constexpr int PER = (CHUNKS + NT - 1) / NT;
    static constexpr int LD = BK + 8;
    u32x4 r[PER];

    __device__ __forceinline__ void load(const half_t *base, long ld, int row0, int nrows, int k0, int K, int tid) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            int c = tid + i * NT;
            int row = c / CPR, kc = c % CPR;
            int gr = min(row0 + row, nrows - 1);
            int gk = k0 + kc * 8;
            u32x4 z = {0u, 0u, 0u, 0u};
            if (CHUNKS % NT == 0 || c < CHUNKS) r[i] = gk < K ? ldg16(base + (long)gr * ld + gk) : z;
        }
    }
    __device__ __forceinline__ void store(half_t *lds, int tid) const {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            int c = tid + i * NT;
            int row = c / CPR, kc = c % CPR;
            if (CHUNKS % NT == 0 || c < CHUNKS) *reinterpret_cast<u32x4 *>(lds + row * LD + kc * 8) = r[i];
        }
    }
};

// Staging of an N-contiguous operand tile [BK][COLS] into the same K-contiguous
// LDS rows: a thread loads an 8(k) x 8(n) block with eight 16-byte row loads,
// transposes it in registers (v_perm_b32) and writes eight 16-byte LDS rows.
template <int COLS, int BK, int NT>
struct KnStage {
    static constexpr int KB = BK / 8;
    static constexpr int BLOCKS = KB * (COLS / 8);
    static constexpr int PER = (BLOCKS + NT - 1) / NT;
    static constexpr int LD = BK + 8;
    u32x4 r[PER][8];

    __device__ __forceinline__ void load(const half_t *base, long ld, int col0, int ncols, int k0, int K, int tid) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            int blk = tid + i * NT;
            int kb = blk % KB, nb = blk / KB;
            int gn = min(col0 + nb * 8, ncols - 8);
            if (BLOCKS % NT == 0 || blk < BLOCKS) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    int gk = k0 + kb * 8 + j;
                    u32x4 z = {0u, 0u, 0u, 0u};
                    r[i][j] = gk < K ? ldg16(base + (long)gk * ld + gn) : z;
                }
            }
        }
    }
    __device__ __forceinline__ void store(half_t *lds, int tid) const {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            int blk = tid + i * NT;
            int kb = blk % KB, nb = blk / KB;
            if (BLOCKS % NT == 0 || blk < BLOCKS) {
#pragma unroll
                for (int w = 0; w < 4; w++) {   // dword w of each row holds columns 2w, 2w+1
                    u32x4 lo, hi;
                    lo.x = pack_lo(r[i][0][w], r[i][1][w]); hi.x = pack_hi(r[i][0][w], r[i][1][w]);
                    lo.y = pack_lo(r[i][2][w], r[i][3][w]); hi.y = pack_hi(r[i][2][w], r[i][3][w]);
                    lo.z = pack_lo(r[i][4][w], r[i][5][w]); hi.z = pack_hi(r[i][4][w], r[i][5][w]);
                    lo.w = pack_lo(r[i][6][w], r[i][7][w]); hi.w = pack_hi(r[i][6][w], r[i][7][w]);
                    *reinterpret_cast<u32x4 *>(lds + (nb * 8 + 2 * w) * LD + kb * 8) = lo;
                    *reinterpret_cast<u32x4 *>(lds + (nb * 8 + 2 * w + 1) * LD + kb * 8) = hi;
                }
            }
        }
    }
};

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Workgroup id -> output tile.  The hardware deals consecutive workgroups
// round-robin over the 8 XCDs, each with its own L2; this hands every XCD one
// contiguous run of the tile order, and the tile order walks GROUP_M row tiles
// per column tile so a run reuses a small set of A and B panels.
__device__ __forceinline__ void tile_of(int pid, int nwg, int tiles_m, int tiles_n, int group_m, int &tm, int &tn) {
    int xcd = pid & 7, idx = pid >> 3;
    int full = nwg >> 3, rem = nwg & 7;
    int logical = xcd * full + min(xcd, rem) + idx;
    int width = group_m * tiles_n;
    int g = logical / width, in = logical - g * width;
    int first = g * group_m;
    int gsz = min(tiles_m - first, group_m);
    tm = first + in % gsz;
    tn = in / gsz;
}

// What the store of a folded norm needs, fetched while the first operand tiles are on their way and parked in `slot`
// (LDS past everything else the kernel keeps there: BM float2 (r, r mu), then BN column sums, then BN biases).
//
// A row's mean and reciprocal standard deviation over its K elements come from the per-segment statistics a producer
// left (stats[seg][row] = (sum, squares about the segment's own mean)).  LPR lanes share a row, each with every LPR-th
// segment, many loads in flight at a time (a lane that walked all segments one dependent load after the other held
// the whole workgroup at its first barrier for 10 us).  One pass: the squares between the segments are taken about the
// first segment's mean, which lies within a segment mean's spread of the row mean, so the final subtraction cancels
// nothing that matters -- sum(x^2) - n mean^2 about zero would.  r = 1 / sqrt(var + eps), rmu = r * mean.
// The caller synchronises the workgroup before anybody reads the slot.
template <int BM, int BN, int NT, typename Args>
__device__ __forceinline__ void lnf_stage(const Args &p, float2v *slot, int m0, int n0, long bz, int tid) {
    if (!p.lnf_stats) return;
    constexpr int LPR = NT >= 4 * BM ? 4 : NT >= 2 * BM ? 2 : 1;
    static_assert(NT >= BM && (BM * LPR) % 64 == 0, "whole waves work on the rows");
    if (tid < BM * LPR) {
        const int row = tid / LPR, q = tid % LPR;
        const float2v *seg = reinterpret_cast<const float2v *>(p.lnf_stats) + min(m0 + row, p.M - 1);
        const float ref = seg[0][0] / (float)min(32, p.K);
        float total = 0.0f, within = 0.0f, between = 0.0f;
        // U loads in flight per lane: all of a row's segments in one trip to memory for K <= 1536 (2048 with four lanes a
        // row) -- a trip costs 1 to 2 us here (the statistics were written by another kernel, on other XCDs), and the
        // first operand tiles, requested before this, take about as long, so one trip is hidden and every further one
        // is not (two and three batches of eight measured +3.3 and +4.3 us per launch)
        constexpr int U = LPR == 4 ? 16 : 24;
        for (int s0 = q; s0 < p.lnf_nseg; s0 += U * LPR) {
            float2v v[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int sg = s0 + u * LPR;
                const float2v z = {0.0f, 0.0f};
                v[u] = sg < p.lnf_nseg ? seg[(long)sg * p.M] : z;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int sg = s0 + u * LPR;
                if (sg < p.lnf_nseg) {
                    const int left = p.K - 32 * sg;
                    const float cnt = left >= 32 ? 32.0f : (float)left, inv = left >= 32 ? 1.0f / 32.0f : 1.0f / (float)left;
                    const float d = fmaf(v[u][0], inv, -ref);
                    total += v[u][0];
                    within += v[u][1];
                    between = fmaf(cnt * d, d, between);
                }
            }
        }
        if constexpr (LPR >= 2) { total += lane_xor<1>(total); within += lane_xor<1>(within); between += lane_xor<1>(between); }
        if constexpr (LPR >= 4) { total += lane_xor<2>(total); within += lane_xor<2>(within); between += lane_xor<2>(between); }
        if (q == 0) {
            const float mu = total / (float)p.K, dm = mu - ref;
            const float m2 = within + fmaxf(between - (float)p.K * dm * dm, 0.0f);
            const float r = 1.0f / sqrtf(m2 / (float)p.K + p.lnf_eps);
            const float2v o = {r, r * mu};
            slot[row] = o;
        }
    }
    // the tile's columns of colsum and biasp
    for (int t = tid; t < BN / 2; t += NT) {
        const int which = t / (BN / 4), c = (t % (BN / 4)) * 4, n = n0 + c;
        const float *src = (which == 0 ? p.lnf_colsum : p.lnf_biasp) + bz * p.lnf_svec;
        float4v v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (n + 3 < p.N) v = *reinterpret_cast<const float4v *>(src + n);
        else for (int e = 0; e < 4; e++) if (n + e < p.N) v[e] = src[n + e];
        *reinterpret_cast<float4v *>(reinterpret_cast<float *>(slot + BM) + which * BN + c) = v;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

// ------------------------------------------------------------------------------------------
// Accumulator tile -> memory, shared by the tiled kernels.
// acc[i][j][r]: n = n0 + wn*WTN + 32 i + 8 (r/4) + 4 (lane/32) + r%4,  m = m0 + wm*WTM + 32 j + lane%32.
// Each wave stages one 32 x WTN sub-tile at a time in its own LDS region (bias
// joined in fp32, one rounding), then reads it back row-wise so that the
// activation, the residual add and the global stores run on 16-byte vectors
// that are contiguous along the output row.  The caller has synchronised the
// workgroup after its last read of the operand tiles.
// The column bias of a wave's sub-tile, in the accumulator's order: cb[i][g] covers
// n = n0 + wn*WTN + 32 i + 8 g + 4 (lane/32) .. +3.  Fetched by the kernels ahead of their last
// k-step so that the epilogue does not start with a trip to memory.
template <int TN, int WTN>
__device__ __forceinline__ void load_col_bias(const GemmArgs &p, half4v (&cb)[TN][4], int n0, int wn, int lane, long bz) {
    const half4v z = {(half_t)0.0f, (half_t)0.0f, (half_t)0.0f, (half_t)0.0f};
    const bool on = p.bias_mode == MI_BIAS_COL;
    const half_t *bias = on ? p.bias + bz * p.sBias : nullptr;
    const bool vec = (reinterpret_cast<uintptr_t>(bias) & 7) == 0;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int n = n0 + wn * WTN + 32 * i + 8 * g + 4 * (lane >> 5);
            cb[i][g] = z;
            if (on) {
                if (n + 3 < p.N && vec) cb[i][g] = *reinterpret_cast<const half4v *>(bias + n);
                else for (int e = 0; e < 4; e++) if (n + e < p.N) cb[i][g][e] = bias[n + e];
            }
        }
}

// What the store of a folded layer norm carries (by value, so that it stays in registers): (r, r mu) of the lane's rows
// m0 + wm WTM + 32 j + lane % 32, and the LDS copy of the tile's colsum (bn floats) followed by its biasp.
template <int TM>
struct LnFold {
    bool on = false;
    float r[TM] = {}, rmu[TM] = {};
    const float *col = nullptr;
    int bn = 0;
};
template <int EPI, int TM, int TN, int WTM, int WTN, int NWAVES, int LDS_BYTES>
__device__ __forceinline__ void store_tile_epi(const GemmArgs &p, float16v (&acc)[TN][TM], const half4v (&cb)[TN][4], char *smem, int m0, int n0, int wm, int wn,
                                               int wave, int lane, long bz, const LnFold<TM> ln = LnFold<TM>{}) {
    const int frow = lane & 31;
    const half_t *bias = p.bias ? p.bias + bz * p.sBias : nullptr;
    constexpr int SLD_H = WTN + 8;                 // halves per staged row (fp16 output)
    constexpr int SLD_F = WTN + 4;                 // floats per staged row (fp32 output)
    constexpr int STAGE_BYTES = 32 * SLD_F * 4;
    static_assert(STAGE_BYTES * NWAVES <= LDS_BYTES, "epilogue staging exceeds the operand LDS");
    char *stage = smem + wave * STAGE_BYTES;
    const int hl = lane >> 5;
    // Row biases for all of the wave's rows before the first store (store_tile_simple says why).
    float brow_j[TM];
#pragma unroll
    for (int j = 0; j < TM; j++) {
        const int m = m0 + wm * WTM + 32 * j + frow;
        brow_j[j] = (p.bias_mode == MI_BIAS_ROW && m < p.M) ? (float)bias[m] : 0.0f;
    }
    static_for<TM>([&](auto J) {
        constexpr int j = decltype(J)::value;
        const int mrow = m0 + wm * WTM + 32 * j;
        const float brow = brow_j[j];
#pragma unroll
        for (int i = 0; i < TN; i++) {
            // folded layer norm: this lane's columns of colsum and biasp from their LDS copy, a 32-column group at a time
            float4v lc4[4], lb4[4];
            if (ln.on) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int nl = 32 * i + 8 * g + 4 * hl;
                    lc4[g] = *reinterpret_cast<const float4v *>(ln.col + wn * WTN + nl);
                    lb4[g] = *reinterpret_cast<const float4v *>(ln.col + ln.bn + wn * WTN + nl);
                }
            }
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int nl = 32 * i + 8 * g + 4 * hl;
                const int n = n0 + wn * WTN + nl;
                float v[4];
                if (ln.on) {      // uniform: r (acc - mu colsum) + biasp
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = fmaf(acc[i][j][4 * g + e], ln.r[j], fmaf(-ln.rmu[j], lc4[g][e], lb4[g][e]));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * g + e] + brow + (float)cb[i][g][e];
                }
                if (p.out_f32) {
                    float4v o = {v[0], v[1], v[2], v[3]};
                    *reinterpret_cast<float4v *>(reinterpret_cast<float *>(stage) + frow * SLD_F + nl) = o;
                } else {
                    half4v o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                    *reinterpret_cast<half4v *>(reinterpret_cast<half_t *>(stage) + frow * SLD_H + nl) = o;
                }
            }
        }
        // A wave reads back only what it staged itself, and its LDS operations complete in order:
        // no workgroup barrier, only a stop for the compiler.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (p.out_f32) {
            constexpr int CPR = WTN / 4;
            for (int c = lane; c < 32 * CPR; c += 64) {
                const int row = c / CPR, ch = c % CPR;
                const int m = mrow + row, n = n0 + wn * WTN + ch * 4;
                if (m < p.M && n < p.N) {
                    float4v x = *reinterpret_cast<const float4v *>(reinterpret_cast<const float *>(stage) + row * SLD_F + ch * 4);
                    float *yp = reinterpret_cast<float *>(p.Y) + bz * p.sY + (long)m * p.ldY + n;
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] = apply_epi_c<EPI>(x[e]);
                    if (p.vec_store && n + 3 < p.N) *reinterpret_cast<float4v *>(yp) = x;
                    else for (int e = 0; e < 4; e++) if (n + e < p.N) yp[e] = x[e];
                }
            }
        } else {
            constexpr int CPR = WTN / 8;
            static_assert((32 * CPR) % 64 == 0 && CPR % 4 == 0, "whole waves walk the staged tile; four lanes hold a 32-column segment");
            for (int c = lane; c < 32 * CPR; c += 64) {
                const int row = c / CPR, ch = c % CPR;
                const int m = mrow + row, n = n0 + wn * WTN + ch * 8;
                half8v x = {};
                if (m < p.M && n < p.N) {
                    x = *reinterpret_cast<const half8v *>(reinterpret_cast<const half_t *>(stage) + row * SLD_H + ch * 8);
                    const long off = bz * p.sY + (long)m * p.ldY + n;
                    half_t *yp = reinterpret_cast<half_t *>(p.Y) + off;
                    if constexpr (EPI != MI_EPI_NONE) {
#pragma unroll
                        for (int e = 0; e < 8; e++) x[e] = (half_t)apply_epi_c<EPI>((float)x[e]);
                    }
                    if (p.vec_store && n + 7 < p.N) {
                        if (p.residual) {
                            half8v rv = as_half8(ldg16(p.residual + off));
#pragma unroll
                            for (int e = 0; e < 8; e++) x[e] = (half_t)((float)x[e] + (float)rv[e]);
                        }
                        if (p.clamp > 0.0f) {
#pragma unroll
                            for (int e = 0; e < 8; e++) x[e] = (half_t)fminf(fmaxf((float)x[e], -p.clamp), p.clamp);
                        }
                        *reinterpret_cast<half8v *>(yp) = x;
                    } else {
                        for (int e = 0; e < 8; e++) {
                            if (n + e < p.N) {
                                half_t o = x[e];
                                if (p.residual) o = (half_t)((float)o + (float)p.residual[off + e]);
                                if (p.clamp > 0.0f) o = (half_t)fminf(fmaxf((float)o, -p.clamp), p.clamp);
                                yp[e] = o;
                            }
                        }
                    }
                }
                if (p.stats_out) {      // uniform; the launcher admits it with 16-byte stores and N % 8 == 0 only
                    // the four lanes of a quad hold the 32 columns of one segment of one row (chunks that lie past N
                    // or below M count nothing): sum, then squares about the segment's own mean, both over the quad
                    const bool have = m < p.M && n < p.N;
                    float cnt = have ? 8.0f : 0.0f, sum = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; e++) sum += have ? (float)x[e] : 0.0f;
                    sum += lane_xor<1>(sum); sum += lane_xor<2>(sum);
                    cnt += lane_xor<1>(cnt); cnt += lane_xor<2>(cnt);
                    const float mean = sum / fmaxf(cnt, 1.0f);
                    float sq = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; e++) { const float d = (float)x[e] - mean; sq = have ? fmaf(d, d, sq) : sq; }
                    sq += lane_xor<1>(sq); sq += lane_xor<2>(sq);
                    if (have && (ch & 3) == 0) {
                        const float2v o = {sum, sq};
                        *reinterpret_cast<float2v *>(p.stats_out + ((long)(n / 32) * p.M + m) * 2) = o;
                    }
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    });
}

// Block j (32 rows) of a wave's accumulators -> its staging area `dst` (32 rows of WTN + 8 halves), rounded to fp16 once
// with the column bias -- or the folded layer norm's r (acc - mu colsum) + biasp -- joined in fp32.
template <int j, int TM, int TN, int WTN>
__device__ __forceinline__ void stage_block(float16v (&acc)[TN][TM], const half4v (&cb)[TN][4], const LnFold<TM> &ln, int wn, char *dst, int lane) {
    constexpr int SLD_H = WTN + 8;
    const int frow = lane & 31, hl = lane >> 5;
    half_t *st = reinterpret_cast<half_t *>(dst) + frow * SLD_H + 4 * hl;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int nl = 32 * i + 8 * g;
            float v[4];
            if (ln.on) {      // uniform; the tile's colsum and biasp from their LDS copy
                const float4v lc = *reinterpret_cast<const float4v *>(ln.col + wn * WTN + nl + 4 * hl);
                const float4v lb = *reinterpret_cast<const float4v *>(ln.col + ln.bn + wn * WTN + nl + 4 * hl);
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = fmaf(acc[i][j][4 * g + e], ln.r[j], fmaf(-ln.rmu[j], lc[e], lb[e]));
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * g + e] + (float)cb[i][g][e];
            }
            const half4v o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
            *reinterpret_cast<half4v *>(st + nl) = o;
        }
}

// The common store: fp16 output in whole 16-byte chunks, column bias (or a folded layer norm), optional activation,
// residual, clamp and row statistics; no row bias, no fp32 output, no ragged N.
//
// Loads and stores of a wave share one counter and complete in order, so a wait for a load -- wherever the compiler
// places it -- is also a wait for every store issued before that load to be acknowledged: a trip of two microseconds
// under the burst of all workgroups' stores.  The general store above pays it once per 32-row block of a wave's tile
// and once per residual chunk (8 000 clocks of a 44 000-clock launch at 1500 x 1280 -> 5120).  Here nothing is fetched
// behind a store that anybody then waits for: the caller's column bias is pinned in registers ahead of the first store,
// and the residual chunks of block j + 1 are requested before block j's stores go out.
// Same arithmetic as the general store (bias joined in fp32, one rounding, activation on the rounded value, residual,
// clamp), so the two give the same bits.  Two staging areas a wave: block j + 1 is staged while block j's chunks are on
// their way back from the LDS (a wave's LDS operations complete in order: no wait between staging a block and reading it).
template <int EPI, int TM, int TN, int WTM, int WTN, int NWAVES, int LDS_BYTES>
__device__ __forceinline__ void store_tile_simple(const GemmArgs &p, float16v (&acc)[TN][TM], const half4v (&cb)[TN][4], char *smem, int m0, int n0, int wm, int wn,
                                                  int wave, int lane, long bz, const LnFold<TM> ln) {
    constexpr int SLD_H = WTN + 8, BUF_BYTES = 32 * SLD_H * 2;      // halves per staged row; one staging area
    constexpr int CPR = WTN / 8, RPI = 64 / CPR, NIT = 32 / RPI;     // 16-byte chunks per row; rows a wave covers at a time; chunks per lane and block
    static_assert(2 * BUF_BYTES * NWAVES <= LDS_BYTES && 64 % CPR == 0 && CPR % 4 == 0, "two staging areas a wave; four lanes hold a 32-column segment");
    char *const buf = smem + wave * 2 * BUF_BYTES;
    const int frow = lane & 31, hl = lane >> 5;
    const int ch = lane % CPR, r0 = lane / CPR;                      // this lane's chunks of a block: rows r0 + RPI t, columns 8 ch ..
    const int mw = m0 + wm * WTM, n = n0 + wn * WTN + ch * 8;
    const bool col_ok = n < p.N;                                     // N % 8 == 0: a chunk that starts below N ends below it
    const long off0 = bz * p.sY + (long)(mw + r0) * p.ldY + n;
    half_t *const ybase = reinterpret_cast<half_t *>(p.Y) + off0;
    const half_t *const rbase = p.residual ? p.residual + off0 : nullptr;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) asm volatile("" ::"v"(cb[i][g]));
    auto stage = [&](auto J) {
        constexpr int j = decltype(J)::value;
        stage_block<j, TM, TN, WTN>(acc, cb, ln, wn, buf + (j & 1) * BUF_BYTES, lane);
    };
    half8v res[2][NIT];
    auto fetch_residual = [&](auto J) {
        constexpr int j = decltype(J)::value;
#pragma unroll
        for (int t = 0; t < NIT; t++) {
            res[j & 1][t] = half8v{};
            if (col_ok && mw + 32 * j + r0 + t * RPI < p.M) res[j & 1][t] = as_half8(ldg16(rbase + (long)(32 * j + t * RPI) * p.ldY));
        }
    };
    if (rbase) fetch_residual(std::integral_constant<int, 0>{});
    stage(std::integral_constant<int, 0>{});
    static_for<TM>([&](auto J) {
        constexpr int j = decltype(J)::value;
        const half_t *rd = reinterpret_cast<const half_t *>(buf + (j & 1) * BUF_BYTES) + r0 * SLD_H + ch * 8;
        half8v x[NIT];
#pragma unroll
        for (int t = 0; t < NIT; t++) x[t] = *reinterpret_cast<const half8v *>(rd + t * RPI * SLD_H);
        if constexpr (j + 1 < TM) {
            stage(std::integral_constant<int, j + 1>{});
            if (rbase) fetch_residual(std::integral_constant<int, j + 1>{});
        }
#pragma unroll
        for (int t = 0; t < NIT; t++) {
            const int m = mw + 32 * j + r0 + t * RPI;
            const bool have = col_ok && m < p.M;
            if constexpr (EPI != MI_EPI_NONE) {
#pragma unroll
                for (int e = 0; e < 8; e++) x[t][e] = (half_t)apply_epi_c<EPI>((float)x[t][e]);
            }
            if (rbase) {
#pragma unroll
                for (int e = 0; e < 8; e++) x[t][e] = (half_t)((float)x[t][e] + (float)res[j & 1][t][e]);
            }
            if (p.clamp > 0.0f) {
#pragma unroll
                for (int e = 0; e < 8; e++) x[t][e] = (half_t)fminf(fmaxf((float)x[t][e], -p.clamp), p.clamp);
            }
            if (have) *reinterpret_cast<half8v *>(ybase + (long)(32 * j + t * RPI) * p.ldY) = x[t];
            if (p.stats_out) {      // uniform
                // the four lanes of a quad hold the 32 columns of one segment of one row (chunks that lie past N or
                // below M count nothing): sum, then squares about the segment's own mean, both over the quad
                float cnt = have ? 8.0f : 0.0f, sum = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) sum += have ? (float)x[t][e] : 0.0f;
                sum += lane_xor<1>(sum); sum += lane_xor<2>(sum);
                cnt += lane_xor<1>(cnt); cnt += lane_xor<2>(cnt);
                const float mean = sum / fmaxf(cnt, 1.0f);
                float sq = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) { const float d = (float)x[t][e] - mean; sq = have ? fmaf(d, d, sq) : sq; }
                sq += lane_xor<1>(sq); sq += lane_xor<2>(sq);
                if (have && (ch & 3) == 0) {
                    const float2v o = {sum, sq};
                    *reinterpret_cast<float2v *>(p.stats_out + ((long)(n / 32) * p.M + m) * 2) = o;
                }
            }
        }
    });
}

// The four-wave kernel's store, shared between a matrix wave and the helper wave on its SIMD.  One wave issues a vector
// instruction every eight clocks, a SIMD takes one every four: the erf-GELU of a 128 x 256 tile (a reciprocal, an
// exponential and thirteen other vector instructions on each of 128 values a lane) cost a lone matrix wave 14 600
// clocks, 8 100 with a helper, and the plain store gains too (1500 x 1280 -> 5120 + bias: 21.8 us against 22.8).  The
// matrix wave stages its 32-row blocks as in store_tile_simple and takes the first half of each block's chunks, the
// helper the second half; a workgroup barrier per block says "block j is staged" (a wave passes barrier j + 1 only
// when it has block j's chunks in registers, so staging block j + 2 over block j's area after that barrier is safe).
// Launches without residual, clamp or statistics only: the others keep store_tile_simple on the matrix waves alone.
__host__ __device__ __forceinline__ bool coop_store_applies(const GemmArgs &p) {
    return !p.out_f32 && p.vec_store && p.N % 8 == 0 && p.bias_mode != MI_BIAS_ROW && !p.residual &&
           !(p.clamp > 0.0f) && !p.stats_out;
}
template <int EPI, int TM, int WTN, bool HELPER, typename StageF, typename BarrierF>
__device__ __forceinline__ void store_coop_epi(const GemmArgs &p, char *buf, int mw, int nw, int lane, long bz, StageF stage, BarrierF barrier) {
    constexpr int SLD_H = WTN + 8, BUF_BYTES = 32 * SLD_H * 2;
    constexpr int CPR = WTN / 8, RPI = 64 / CPR, NIT = 32 / RPI, T0 = HELPER ? NIT / 2 : 0, T1 = HELPER ? NIT : NIT / 2;
    static_assert(NIT % 2 == 0, "the chunks of a block split in two");
    const int ch = lane % CPR, r0 = lane / CPR;
    const int n = nw + ch * 8;
    const bool col_ok = n < p.N;
    half_t *const ybase = reinterpret_cast<half_t *>(p.Y) + bz * p.sY + (long)(mw + r0) * p.ldY + n;
    if constexpr (!HELPER) stage(std::integral_constant<int, 0>{});
    static_for<TM>([&](auto J) {
        constexpr int j = decltype(J)::value;
        barrier();                                             // block j is staged
        const half_t *rd = reinterpret_cast<const half_t *>(buf + (j & 1) * BUF_BYTES) + r0 * SLD_H + ch * 8;
        half8v x[T1 - T0];
#pragma unroll
        for (int t = T0; t < T1; t++) x[t - T0] = *reinterpret_cast<const half8v *>(rd + t * RPI * SLD_H);
        if constexpr (!HELPER && j + 1 < TM) stage(std::integral_constant<int, j + 1>{});
#pragma unroll
        for (int t = T0; t < T1; t++) {
#pragma unroll
            for (int e = 0; e < 8; e++) x[t - T0][e] = (half_t)apply_epi_c<EPI>((float)x[t - T0][e]);
            if (col_ok && mw + 32 * j + r0 + t * RPI < p.M) *reinterpret_cast<half8v *>(ybase + (long)(32 * j + t * RPI) * p.ldY) = x[t - T0];
        }
    });
}
template <int TM, int WTN, bool HELPER, typename StageF, typename BarrierF>
__device__ __forceinline__ void store_coop(const GemmArgs &p, char *buf, int mw, int nw, int lane, long bz, StageF stage, BarrierF barrier) {
    switch (p.epi) {
    case MI_EPI_GELU_ERF: store_coop_epi<MI_EPI_GELU_ERF, TM, WTN, HELPER>(p, buf, mw, nw, lane, bz, stage, barrier); break;
    case MI_EPI_GELU_TANH: store_coop_epi<MI_EPI_GELU_TANH, TM, WTN, HELPER>(p, buf, mw, nw, lane, bz, stage, barrier); break;
    case MI_EPI_RELU: store_coop_epi<MI_EPI_RELU, TM, WTN, HELPER>(p, buf, mw, nw, lane, bz, stage, barrier); break;
    default: store_coop_epi<MI_EPI_NONE, TM, WTN, HELPER>(p, buf, mw, nw, lane, bz, stage, barrier); break;
    }
}

// The activation is a compile-time choice inside the store loops: one uniform branch per tile
// instead of one per element.
template <int TM, int TN, int WTM, int WTN, int NWAVES, int LDS_BYTES>
__device__ __forceinline__ void store_tile(const GemmArgs &p, float16v (&acc)[TN][TM], const half4v (&cb)[TN][4], char *smem, int m0, int n0, int wm, int wn,
                                           int wave, int lane, long bz, const LnFold<TM> ln = LnFold<TM>{}) {
    const bool simple = !p.out_f32 && p.vec_store && p.N % 8 == 0 && p.bias_mode != MI_BIAS_ROW;
    if (simple) {
        switch (p.epi) {
        case MI_EPI_GELU_ERF: store_tile_simple<MI_EPI_GELU_ERF, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
        case MI_EPI_GELU_TANH: store_tile_simple<MI_EPI_GELU_TANH, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
        case MI_EPI_RELU: store_tile_simple<MI_EPI_RELU, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
        default: store_tile_simple<MI_EPI_NONE, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
        }
        return;
    }
    switch (p.epi) {
    case MI_EPI_GELU_ERF: store_tile_epi<MI_EPI_GELU_ERF, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
    case MI_EPI_GELU_TANH: store_tile_epi<MI_EPI_GELU_TANH, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
    case MI_EPI_RELU: store_tile_epi<MI_EPI_RELU, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
    default: store_tile_epi<MI_EPI_NONE, TM, TN, WTM, WTN, NWAVES, LDS_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln); break;
    }
}

// ------------------------------------------------------------------------------------------
// The tiled MFMA kernel.  BM x BN output tile per workgroup, WAVES_M x WAVES_N
// waves, each owning a (BM/WAVES_M) x (BN/WAVES_N) sub-tile as 32x32 MFMA
// tiles.  The MFMA is issued "transposed" (rows = n, columns = m) so that a
// lane's four consecutive accumulator registers are four consecutive n of one
// output row: an 8-byte fp16 store.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool B_KN>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_mfma_kernel(GemmArgs p) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int LD = BK + 8;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    extern __shared__ __align__(16) char smem[];
    half_t *As = reinterpret_cast<half_t *>(smem);   // [2][BM][LD]
    half_t *Bs = As + 2 * BM * LD;                   // [2][BN][LD]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    int tm_, tn_;
    tile_of(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, p.group_m, tm_, tn_);
    const int m0 = tm_ * BM, n0 = tn_ * BN;
    const long bz = blockIdx.y;
    const half_t *A = p.A + bz * p.sA;
    const half_t *B = p.B + bz * p.sB;

    KcStage<BM, BK, NT> sa;
    KcStage<BN, BK, NT> sbk;
    KnStage<BN, BK, NT> sbn;

    float16v acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int nk = (p.K + BK - 1) / BK;
    sa.load(A, p.ldA, m0, p.M, 0, p.K, tid);
    if (B_KN) sbn.load(B, p.ldB, n0, p.NB, 0, p.K, tid); else sbk.load(B, p.ldB, n0, p.N, 0, p.K, tid);
    sa.store(As, tid);
    if (B_KN) sbn.store(Bs, tid); else sbk.store(Bs, tid);
    __syncthreads();

    const int frow = lane & 31, fk = (lane >> 5) * 8;
    for (int kt = 0; kt < nk; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < nk;
        if (more) {
            sa.load(A, p.ldA, m0, p.M, (kt + 1) * BK, p.K, tid);
            if (B_KN) sbn.load(B, p.ldB, n0, p.NB, (kt + 1) * BK, p.K, tid); else sbk.load(B, p.ldB, n0, p.N, (kt + 1) * BK, p.K, tid);
        }
        const half_t *as = As + cur * BM * LD + (wm * WTM + frow) * LD + fk;
        const half_t *bs = Bs + cur * BN * LD + (wn * WTN + frow) * LD + fk;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            half8v fa[TM], fb[TN];
#pragma unroll
            for (int j = 0; j < TM; j++) fa[j] = *reinterpret_cast<const half8v *>(as + j * 32 * LD + ks * 16);
#pragma unroll
            for (int i = 0; i < TN; i++) fb[i] = *reinterpret_cast<const half8v *>(bs + i * 32 * LD + ks * 16);
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[i], fa[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            sa.store(As + (cur ^ 1) * BM * LD, tid);
            if (B_KN) sbn.store(Bs + (cur ^ 1) * BN * LD, tid); else sbk.store(Bs + (cur ^ 1) * BN * LD, tid);
        }
        __syncthreads();
    }

    half4v cb[TN][4];
    load_col_bias<TN, WTN>(p, cb, n0, wn, lane, bz);
    store_tile<TM, TN, WTM, WTN, WAVES_M * WAVES_N, 2 * (BM + BN) * LD * 2>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz);
}

// ------------------------------------------------------------------------------------------
// The software-pipelined kernel for K % 64 == 0 (every linear of the encoder
// configurations).  Same tiles and LDS layout as gemm_mfma_kernel, but the K loop
// is written out as a four-phase pipeline per 64-deep tile:
//   phase 0: read fragments of k-step 1 | MFMAs of k-step 0   (+ issue the global loads of tile kt+2)
//   phase 1: read fragments of k-step 2 | MFMAs of k-step 1 | write the A part of tile kt+1 to the other LDS buffer
//   phase 2: read fragments of k-step 3 | MFMAs of k-step 2 | write the B part of tile kt+1
//   barrier
//   phase 3: read fragments of k-step 0 of tile kt+1 | MFMAs of k-step 3
// Global loads run two tiles ahead through two register sets, so a load has a
// whole tile of MFMAs to land before its LDS write; the only barrier of a tile sits
// where its successor's first fragment read can be hidden behind the last k-step.
// Two waves per SIMD (8 waves on a 128 x 256 tile) cover each other's waits.
// BMODE: 0 = B is [N][K], 1 = B is [K][N], 2 = B is [K][N] gathered from a padded image (implicit-GEMM convolution).
// AMODE 1: A is gathered from a channels-last image (NhwcGather); B is then an ordinary [N][K] or [K][N] operand.
// AMODE 2: the rows of A are layer-normalised over K on their way in (K <= 512): before the K loop every wave
// normalises rows of the tile's A panel -- one wave per row, a lane holding eight consecutive k, statistics,
// arithmetic and rounding exactly those of layernorm_vec_kernel -- into an LDS panel [BM][K + 8] that stays resident;
// the K loop then streams B alone and reads its A fragments from the panel.
template <int BM, int BN, int WAVES_M, int WAVES_N, int BMODE, int AMODE = 0>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, 2) void gemm_pipe_kernel(GemmArgs p) {
    constexpr bool B_KN = BMODE != 0, CONV = BMODE == 2, LNA = AMODE == 2;
    static_assert(AMODE == 0 || BMODE != 2, "one gathered operand at a time");
    constexpr int BK = 64, LD = BK + 8, NT = WAVES_M * WAVES_N * 64;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, TM = WTM / 32, TN = WTN / 32;
    constexpr int PA = BM * 8 / NT, PB = BN * 8 / NT;     // 16-byte chunks per thread per tile
    // The [K][N] operand keeps its layout in LDS: BK rows of BN halves, padded by
    // 32 halves so that the four rows a transposing read touches fall in distinct
    // bank groups.  Its MFMA fragments come from ds_read_b64_tr_b16 (see fread).
    constexpr int BLD = BN + 32, CPRB = BN / 8;
    static_assert(PA >= 1 && PB >= 1, "tile too small for this workgroup");
    constexpr int BSZ = B_KN ? BK * BLD : BN * LD;      // halves per B buffer
    extern __shared__ __align__(16) char smem[];
    half_t *As = reinterpret_cast<half_t *>(smem);   // [2][BM][LD]; AMODE 2: the normalised panel [BM][K + 8]
    const int KP = p.K + 8;                          // panel row (halves): 16 bytes off a multiple of 128, like LD
    half_t *Bs = As + (LNA ? BM * KP : 2 * BM * LD); // [2][BN][LD] or [2][BK][BLD]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    int tm_, tn_;
    tile_of(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, p.group_m, tm_, tn_);
    const int m0 = tm_ * BM, n0 = tn_ * BN;
    const long bz = blockIdx.y;
    const half_t *A = p.A + bz * p.sA;
    const half_t *B = p.B + bz * p.sB;

    // Per-thread global sources; rows and columns past the edge re-read the last
    // valid one (their results are never stored).
    const half_t *ap[PA], *bp[PB];
#pragma unroll
    for (int i = 0; i < PA; i++) { const int c = tid + i * NT; ap[i] = A + (long)min(m0 + (c >> 3), p.M - 1) * p.ldA + (c & 7) * 8; }
#pragma unroll
    for (int i = 0; i < PB; i++) {
        const int c = tid + i * NT;
        if (!B_KN) bp[i] = B + (long)min(n0 + (c >> 3), p.N - 1) * p.ldB + (c & 7) * 8;
        else       bp[i] = B + (long)(c / CPRB) * p.ldB + min(n0 + (c % CPRB) * 8, p.NB - 8);
    }
    // Implicit GEMM: every chunk of this thread lies in the same eight columns (NT is a multiple of
    // CPRB), i.e. at one pixel offset, in channels NT / CPRB apart; which tap and which 64 channels a tile
    // covers is the same for the whole workgroup.
    const half_t *cpix = nullptr;
    int ctile0 = 0;
    if constexpr (CONV) {
        static_assert(NT % CPRB == 0 && PB * (NT / CPRB) == BK, "a thread's chunks share their columns, NT / CPRB rows apart");
        const int ncol = min(n0 + (tid % CPRB) * 8, p.NB - 8);
        const int oh = ncol / p.cv.OW, ow = ncol % p.cv.OW;
        cpix = p.cv.xp + (p.cv.split ? 0 : bz * p.cv.img) + (long)oh * p.cv.sy * p.cv.Wp + ow + (long)(tid / CPRB) * p.cv.HpWp;
        ctile0 = p.cv.split ? (int)bz * (p.K / BK) : 0;
    }
    // Channels-last gather: a thread's rows are fixed output pixels; (iy0, ix0) is where tap (0, 0) of each lands.
    int aiy0[PA], aix0[PA];
    int atile0 = 0;
    if constexpr (AMODE == 1) {
#pragma unroll
        for (int i = 0; i < PA; i++) {
            const int c = tid + i * NT;
            const int m = min(m0 + (c >> 3), p.M - 1);
            const int pq = p.ag.OH * p.ag.OW;
            const int n = m / pq, rem = m - n * pq, oh = rem / p.ag.OW, ow = rem - oh * p.ag.OW;
            aiy0[i] = oh * p.ag.sy - p.ag.py;
            aix0[i] = ow * p.ag.sx - p.ag.px;
            ap[i] = p.ag.x + (long)n * p.ag.H * p.ag.W * p.ag.C + (c & 7) * 8;
        }
        atile0 = p.ag.split ? (int)bz * (p.K / BK) : 0;
    }
    u32x4 ga[2][PA], gb[2][PB];
    auto gload = [&](int set, int kt) {
        const long ko = (long)kt * BK;
        if constexpr (AMODE == 1) {
            const int t = atile0 + kt, tap = t / p.ag.cpt, ci0 = (t - tap * p.ag.cpt) * BK;       // the same for every lane
            const int kh = tap / p.ag.KW, kw = tap - kh * p.ag.KW;
            const int ddy = kh * p.ag.dy, ddx = kw * p.ag.dx;
#pragma unroll
            for (int i = 0; i < PA; i++) {
                const int iy = aiy0[i] + ddy, ix = aix0[i] + ddx;
                const bool in = (unsigned)iy < (unsigned)p.ag.H && (unsigned)ix < (unsigned)p.ag.W;
                const u32x4 z = {0u, 0u, 0u, 0u};
                ga[set][i] = in ? ldg16(ap[i] + ((long)iy * p.ag.W + ix) * p.ag.C + ci0) : z;
            }
        } else if constexpr (!LNA) {
#pragma unroll
            for (int i = 0; i < PA; i++) ga[set][i] = ldg16(ap[i] + ko);
        }
#pragma unroll
        for (int i = 0; i < PB; i++) {
            if constexpr (CONV) {
                const int t = ctile0 + kt, tap = t / p.cv.cpt, ci0 = (t - tap * p.cv.cpt) * BK;
                const int kh = tap / p.cv.KW, kw = tap - kh * p.cv.KW;
                const int toff = ci0 * p.cv.HpWp + kh * p.cv.dyWp + kw * p.cv.dx;       // same for every lane
                // The eight halves start kw*dx elements into an aligned row, i.e. at a 2-byte boundary, and
                // vector loads want 4-byte alignment: odd starts are read from the second copy of the padded
                // input, which is the first shifted by one element (the choice is the same for every lane).
                const uint32_t *src = reinterpret_cast<const uint32_t *>(cpix + toff + ((toff & 1) ? p.cv.odd : 0L) + (long)i * (NT / CPRB) * p.cv.HpWp);
                uint32_t w4[4];
                __builtin_memcpy(w4, src, 16);
#pragma unroll
                for (int q = 0; q < 4; q++) gb[set][i][q] = w4[q];
            } else {
                gb[set][i] = ldg16(bp[i] + (B_KN ? ko * p.ldB : ko));
            }
        }
    };
    auto lwrite_a = [&](int set, int buf) {
        if constexpr (LNA) return;                     // the panel is already there
#pragma unroll
        for (int i = 0; i < PA; i++) { const int c = tid + i * NT; *reinterpret_cast<u32x4 *>(As + buf * BM * LD + (c >> 3) * LD + (c & 7) * 8) = ga[set][i]; }
    };
    auto lwrite_b = [&](int set, int buf) {
#pragma unroll
        for (int i = 0; i < PB; i++) {
            const int c = tid + i * NT;
            half_t *dst = !B_KN ? Bs + buf * BSZ + (c >> 3) * LD + (c & 7) * 8 : Bs + buf * BSZ + (c / CPRB) * BLD + (c % CPRB) * 8;
            *reinterpret_cast<u32x4 *>(dst) = gb[set][i];
        }
    };

    float16v acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int frow = lane & 31, fk = (lane >> 5) * 8;
    const int aoff = (wm * WTM + frow) * (LNA ? KP : LD) + fk, boff = (wn * WTN + frow) * LD + fk;
    // [K][N] fragments: within each block of 16 lanes, lane i of ds_read_b64_tr_b16
    // receives, for j = 0..3, element i%4 of the 8 bytes addressed by lane 4j + i/4.
    // Pointing lane s at row (k0 + s/4), columns (n0 + 4 (s%4) .. +3) therefore hands
    // lane i the four consecutive k of column n0 + i: the MFMA operand layout.
    const int tboff = (fk + ((lane & 15) >> 2)) * BLD + wn * WTN + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    half8v fa[2][TM], fb[2][TN];
    auto fread = [&](int fs, int buf, int ks, int kt) {
        const half_t *as = LNA ? As + aoff + kt * BK + ks * 16 : As + buf * BM * LD + aoff + ks * 16;
        const int jstep = 32 * (LNA ? KP : LD);
#pragma unroll
        for (int j = 0; j < TM; j++) fa[fs][j] = *reinterpret_cast<const half8v *>(as + j * jstep);
        if (!B_KN) {
            const half_t *bs = Bs + buf * BSZ + boff + ks * 16;
#pragma unroll
            for (int i = 0; i < TN; i++) fb[fs][i] = *reinterpret_cast<const half8v *>(bs + i * 32 * LD);
        } else {
            const half_t *bs = Bs + buf * BSZ + tboff + ks * 16 * BLD;
#pragma unroll
            for (int i = 0; i < TN; i++) {
                short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(bs + i * 32));
                short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(bs + i * 32 + 4 * BLD));
                short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                fb[fs][i] = __builtin_bit_cast(half8v, both);
            }
        }
    };
    auto mma = [&](int fs) {
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[fs][i], fa[fs][j], acc[i][j], 0, 0, 0);
    };

    const int nk = p.K / BK;   // the launcher guarantees K % 64 == 0 and nk >= 2
    gload(0, 0);
    gload(1, 1);
    // folded layer norm: (r, r mu) of the tile's rows, worked out while the first tiles are on their way and parked
    // in LDS behind the operand buffers until the store (the barrier after the first LDS write covers it)
    float2v *ln_slot = reinterpret_cast<float2v *>(smem + 2 * (BM * LD + BSZ) * 2);
    if constexpr (!LNA) lnf_stage<BM, BN, NT>(p, ln_slot, m0, n0, bz, tid);
    if constexpr (LNA) {
        // One wave per row, all rows of a wave in flight at once (one trip to memory).  Rows past M repeat the last one.
        constexpr int NW = NT / 64, RB = BM / NW;
        static_assert(RB >= 1 && RB <= 16 && BM % NW == 0, "a wave's rows fit its registers");
        const int e0 = lane * 8;
        const bool mine = e0 < p.K;
        const u32x4 z = {0u, 0u, 0u, 0u};
        const half8v gv = as_half8((p.ln_gamma && mine) ? ldg16(p.ln_gamma + e0) : z);
        const half8v bv = as_half8((p.ln_beta && mine) ? ldg16(p.ln_beta + e0) : z);
        for (int r0 = wave * (BM / NW); r0 < (wave + 1) * (BM / NW); r0 += RB) {
            u32x4 raw[RB];
#pragma unroll
            for (int q = 0; q < RB; q++) raw[q] = mine ? ldg16(A + (long)min(m0 + r0 + q, p.M - 1) * p.ldA + e0) : z;
#pragma unroll
            for (int q = 0; q < RB; q++) {
                const half8v t = as_half8(raw[q]);
                float x[8], sum = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; j++) { x[j] = mine ? (float)t[j] : 0.0f; if (mine) sum += x[j]; }
                sum = wave_sum(sum);
                const float mu = sum / (float)p.K;
                float s2 = 0.0f;
                if (mine) {
#pragma unroll
                    for (int j = 0; j < 8; j++) { const float d = x[j] - mu; s2 = fmaf(d, d, s2); }
                }
                s2 = wave_sum(s2);
                const float rs = 1.0f / sqrtf(s2 / (float)p.K + p.ln_eps);
                if (mine) {
                    half8v o8;
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        o8[j] = ln_norm1(x[j], mu, rs, p.ln_gamma != nullptr, p.ln_gamma ? (float)gv[j] : 0.0f, p.ln_beta != nullptr, p.ln_beta ? (float)bv[j] : 0.0f);
                    *reinterpret_cast<half8v *>(As + (r0 + q) * KP + e0) = o8;
                }
            }
        }
    }
    lwrite_a(0, 0);
    lwrite_b(0, 0);
    __syncthreads();
    fread(0, 0, 0, 0);

    // MODE 0: steady state; 1: second-to-last tile (nothing left to fetch); 2: last tile.
    // Tile kt is computed from LDS buffer `cur`; register set `gw` holds tile kt+1, set `gl` receives tile kt+2.
    auto body = [&](auto MODE_, int kt, int cur, int gw, int gl) {
        constexpr int MODE = decltype(MODE_)::value;
        constexpr int NM = TM * TN;               // MFMAs per k-step
        constexpr int NR = TM + (B_KN ? 2 * TN : TN);   // fragment reads per k-step
        // Each k-step is pinned to: its fragment reads first, then its MFMAs with the step's
        // memory instructions dealt out between them, so that neither the LDS pipe nor the
        // vector-memory path sees a burst.
        if constexpr (MODE == 0) gload(gl, kt + 2);
        fread(1, cur, 1, kt);
        mma(0);
        __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
#pragma unroll
        for (int g = 0; g < NM; g++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x020, (PA + PB + NM - 1) / NM, 0); }
        __builtin_amdgcn_sched_barrier(0);
        fread(0, cur, 2, kt);
        mma(1);
        if constexpr (MODE < 2) lwrite_a(gw, cur ^ 1);
        __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
#pragma unroll
        for (int g = 0; g < NM; g++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x200, (PA + NM - 1) / NM, 0); }
        __builtin_amdgcn_sched_barrier(0);
        fread(1, cur, 3, kt);
        mma(0);
        if constexpr (MODE < 2) lwrite_b(gw, cur ^ 1);
        __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
#pragma unroll
        for (int g = 0; g < NM; g++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x200, (PB + NM - 1) / NM, 0); }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        if constexpr (MODE < 2) fread(0, cur ^ 1, 0, kt + 1);
        mma(1);
        __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    using M0 = std::integral_constant<int, 0>;
    using M1 = std::integral_constant<int, 1>;
    using M2 = std::integral_constant<int, 2>;
    const int npairs = (nk - 2) >> 1;       // steady-state tiles come in (buffer 0, buffer 1) pairs
    int kt = 0;
    for (int pr = 0; pr < npairs; pr++, kt += 2) {
        body(M0{}, kt, 0, 1, 0);
        body(M0{}, kt + 1, 1, 0, 1);
    }
    half4v cb[TN][4];
    if (nk & 1) {
        body(M0{}, kt, 0, 1, 0);
        body(M1{}, kt + 1, 1, 0, 1);
        load_col_bias<TN, WTN>(p, cb, n0, wn, lane, bz);
        body(M2{}, kt + 2, 0, 1, 0);
    } else {
        body(M1{}, kt, 0, 1, 0);
        load_col_bias<TN, WTN>(p, cb, n0, wn, lane, bz);
        body(M2{}, kt + 1, 1, 0, 1);
    }
    __syncthreads();
    LnFold<TM> ln;
    if (!LNA && p.lnf_stats) {
        ln.on = true; ln.col = reinterpret_cast<const float *>(ln_slot + BM); ln.bn = BN;
#pragma unroll
        for (int j = 0; j < TM; j++) { const float2v v = ln_slot[wm * WTM + 32 * j + (lane & 31)]; ln.r[j] = v[0]; ln.rmu[j] = v[1]; }
    }
    store_tile<TM, TN, WTM, WTN, WAVES_M * WAVES_N, 2 * (BM * LD + BSZ) * 2>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln);
}

// ------------------------------------------------------------------------------------------
// Split-K without fp32 planes and without a second launch: the two workgroups of a tile (gemm_w4_kernel, SK) exchange
// their partial tiles inside the launch.
//
// Workgroup pid runs on XCD pid % 8 (workgroups are dealt to the XCDs round robin; mi_init checks that this device
// does so and the path stays off otherwise): pid = (slot * 2 + s) * 8 + xcd computes K-slice s of tile xcd * tpx + slot,
// so the partners of a tile share an XCD, i.e. one L2, and are dispatched together.  After its K loop every wave owns
// half of its 64 x 64 accumulators -- the 32-row block s -- writes the other half into its partner's slot of sk_part
// (plain stores: they stay in the shared L2), waits for them to be acknowledged, and raises its flag; it then waits
// (bounded) for the same wave of its partner, adds what it sent in slice order (the result does not depend on which
// workgroup sums), and stores its share through the usual epilogue.  Both workgroups publish before they wait, so the
// waits are not circular among resident workgroups; the launcher only checks that the grid fits an IDLE device in
// one round.  Under overlap (another stream's kernel holding CUs) a partner may not be resident yet: the wait is
// bounded, and a wave that runs into the bound -- or finds its partner on another XCD -- raises the device's sticky
// status word (mi_device_status), stores NaN over its share of Y and releases nothing (sk_exchange.hpp has the
// protocol; tests/sk_exchange_host_test.cpp runs it on CPU threads, with one and with three partners).
// (Four slices of a 128 x 256 tile were built and measured as well: three partners to wait for, 23 MB exchanged at
// 1500 x 5120 -> 1280, 40.8 us against 29.8 us for two slices of 128 x 128.)
struct SkDeviceMem {
    __device__ static unsigned load(const unsigned *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    __device__ static void store(unsigned *p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    __device__ static unsigned fetch_add(unsigned *p, unsigned v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    __device__ static void pause() { __builtin_amdgcn_s_sleep(1); }
};
using SkExchange = sk::Exchange<SkDeviceMem>;

// A wave whose exchange failed marks its share of the output instead of storing a plausible sum: NaN in the output
// type over rows [r0, r0 + 32) x columns [c0, c0 + ncols) of the tile.
// (Scalars by value: a reference to the kernel's argument block would force the block into private memory.)
__device__ __noinline__ void sk_poison_region(void *Y, long ldY, int M, int N, int out_f32, int r0, int c0, int ncols, int lane) {
    for (int e = lane; e < 32 * ncols; e += 64) {
        const int m = r0 + e / ncols, n = c0 + e % ncols;
        if (m < M && n < N) {
            const long off = (long)m * ldY + n;
            if (out_f32) reinterpret_cast<unsigned *>(Y)[off] = 0x7fc00000u;
            else reinterpret_cast<unsigned short *>(Y)[off] = (unsigned short)0x7e00u;
        }
    }
}

// The end of a split-K launch whose two K-slices exchange their partial tiles: every wave sends the 32-row block it
// does not keep to its partner, raises its flag, waits (bounded) for the same wave of the partner, sums what arrived
// in slice order and stores its block.
// sk_part[tile][owner][source][wave of NWAVES][column half][4][64 lanes][4]; flags [tile][slice][8].
template <int TM, int TN, int WTM, int WTN, int NWAVES, int LDS_BYTES>
__device__ __forceinline__ void sk_finish(const GemmArgs &p, float16v (&acc)[TN][TM], const half4v (&cb)[TN][4], char *smem, int sk_tile, int sk_s,
                                          int m0, int n0, int wm, int wn, int wave, int lane, long bz) {
    static_assert(TM == 2 && TN == 2, "a wave's 64 x 64 accumulators: two 32-row blocks of two 32 x 32 sub-tiles");
    // four registers per lane and access, 1 KB per wave instruction
    auto part_of = [&](int owner, int src) { return p.sk_part + ((((long)sk_tile * 2 + owner) * 2 + src) * NWAVES + wave) * 2048L + lane * 4; };
    float16v own[2];
    static_for<2>([&](auto J) {
        constexpr int j = decltype(J)::value;
        if (j == sk_s) {                                       // uniform: the block this wave keeps
            own[0] = acc[0][j]; own[1] = acc[1][j];
        } else {
            float *dst = part_of(j, sk_s);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    const float4v v = {acc[i][j][4 * r4], acc[i][j][4 * r4 + 1], acc[i][j][4 * r4 + 2], acc[i][j][4 * r4 + 3]};
                    *reinterpret_cast<float4v *>(dst + i * 1024 + r4 * 256) = v;
                }
        }
    });
    // the partials must have reached L2 before the flag can be seen
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned my_xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u;      // HW_REG_XCC_ID, bits 3:0
    unsigned *myflag = p.sk_flags + ((long)sk_tile * 2 + sk_s) * 8 + wave;
    unsigned *theirs = p.sk_flags + ((long)sk_tile * 2 + (1 - sk_s)) * 8 + wave;
    if (lane == 0) SkExchange::publish(myflag, p.sk_epoch ^ p.sk_pub_xor, my_xcc);
    // Co-residency of the partner is NOT guaranteed (another stream's kernel can hold an XCD's CUs): the bound is the
    // guard, and a wave that runs into it says so.
    const unsigned *const cfl[3] = {theirs, theirs, theirs};
    const sk::WaitResult wr = SkExchange::wait(cfl, 1, p.sk_epoch, my_xcc ^ p.sk_xcc_xor, p.sk_spin);
    asm volatile("" ::: "memory");
    if (wr != sk::ARRIVED) {
        // Loud failure: the sticky status word, NaN over this wave's share of Y, flags left as they are (the host
        // zeroes the banks when it reads the status).  The wave still leaves the kernel normally.
        if (lane == 0) __hip_atomic_fetch_or(p.status, wr == sk::TIMED_OUT ? (unsigned)MI_DEVSTAT_EXCHANGE_TIMEOUT : (unsigned)MI_DEVSTAT_EXCHANGE_XCD,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // (the exchange runs unbatched launches only: bz = 0)
        sk_poison_region(p.Y, p.ldY, p.M, p.N, p.out_f32, m0 + wm * WTM + 32 * sk_s, n0 + wn * WTN, WTN, lane);
        return;
    }
    // Ordinary loads: this CU has not touched these lines since the kernel began (its L1 was invalidated then), so
    // they come from the L2 the partner's acknowledged stores are in (the wait has checked that it is this XCD's).
    const float *from = part_of(sk_s, 1 - sk_s);
    float4v blk[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) blk[i][r4] = *reinterpret_cast<const float4v *>(from + i * 1024 + r4 * 256);
    float16v two[2][1];                                        // summed in slice order, whoever does the summing
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) two[i][0][r] = sk_s == 0 ? own[i][r] + blk[i][r >> 2][r & 3] : blk[i][r >> 2][r & 3] + own[i][r];
    // What the partner sent has arrived (the sums above used it): this wave clears the partner's flag, so the next
    // launch on this bank, which for a replayed graph carries this same epoch, starts from zero.
    if (lane == 0) SkExchange::release(theirs, theirs + SK_WORDS, 1);
    store_tile<1, 2, WTM, WTN, NWAVES, LDS_BYTES>(p, two, cb, smem, m0 + 32 * sk_s, n0, wm, wn, wave, lane, bz);
}

// ------------------------------------------------------------------------------------------
// Four matrix waves, one per SIMD, each with a BM x BN/4 strip of the tile, and a loader wave.
//
// The ping-pong kernel's 128 x 256 tile spends a third of its K loop in waits: per 64-deep tile its eight 64 x 64
// waves read 8 x 16 KB of fragments for 1024 clocks of MFMAs per SIMD, a SIMD takes 32 B/clock from the LDS, and the
// two phases of a tile came to 1590 clocks (measured with clock stamps; no different with every workgroup on one
// L2-resident tile, so it is not memory).  A wave that owns 128 x 64 reads 24 KB for twice the MFMAs.  With one matrix
// wave per SIMD there is no partner to alternate phases with; instead each wave overlaps its own work: three sets
// of fragment registers (4 A + 2 B fragments of a 16-deep step), the reads of step s + 2 dealt one or two at a time
// between the eight MFMAs of step s -- issued in one burst they held the wave at the LDS queue while its matrix pipe
// ran dry -- and an MFMA in flight does not hold up the wave's LDS instructions.  128 accumulator registers + 72 of
// fragments fit because at most two waves (a matrix wave and the loader) share a SIMD: 256 registers each.
// Measured: 1290 to 1390 clocks a tile, and 1500 x 1280 -> 5120 in 23.1 us against 25.5 to 26.1 us.
//
// One workgroup barrier per tile, B_kt, taken by the matrix waves in the middle of tile kt's third step -- after the
// last fragment read of the tile has returned, before the first read of tile kt + 1 -- and by the loader after it has
// waited for tile kt + 1 to land.  Past B_kt stage kt % 3 is free, and the loader requests tile kt + 3 into it.
template <int BM, int BN, int BK, bool B_KN>
struct DirectTile {
    static constexpr int CPR = BK / 8, ROWB = BK * 2, A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int SLOTS_A = A_BYTES / 1024, SLOTS_B = B_BYTES / 1024;      // 1 KB = one wave-wide request
    __device__ __forceinline__ static int rowswz(int r) { return BK == 64 ? (r & 7) ^ ((r >> 3) & 1) : (r >> 2) & 3; }
    // per-lane byte offset, from the tile's origin in memory, of what lands in 1 KB slot s of the A / B part of a stage
    __device__ __forceinline__ static uint32_t a_offset(const GemmArgs &p, int m0, int s, int lane) {
        const int q = s * 64 + lane, r = q / CPR, pos = q % CPR;
        return (uint32_t)(((long)(min(m0 + r, p.M - 1) - m0) * p.ldA + (pos ^ rowswz(r)) * 8) * 2);
    }
    __device__ __forceinline__ static uint32_t b_offset(const GemmArgs &p, int n0, int s, int lane) {
        const int q = s * 64 + lane;
        if (!B_KN) {
            const int r = q / CPR, pos = q % CPR;
            return (uint32_t)(((long)(min(n0 + r, p.N - 1) - n0) * p.ldB + (pos ^ rowswz(r)) * 8) * 2);
        } else {
            constexpr int CPRB = BN / 8;
            const int k = q / CPRB, pos = q % CPRB, j = pos ^ ((k & 3) << 2);
            return (uint32_t)(((long)k * p.ldB + (min(n0 + j * 8, p.NB - 8) - n0)) * 2);
        }
    }
    __device__ __forceinline__ static void request(const char *base, uint32_t off, uint32_t lds_dst) {
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_dst);
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(dst) : "memory");
    }
};

template <int BM, int BN, int WAVES_M, int WAVES_N, bool B_KN, bool SK = false>
__global__ __launch_bounds__(512) void gemm_w4_kernel(GemmArgs p) {
    constexpr int BK = 64, STAGES = 3, KS = 4;
    using T = DirectTile<BM, BN, BK, B_KN>;
    constexpr int ROWB = T::ROWB, A_BYTES = T::A_BYTES, STAGE_BYTES = T::STAGE_BYTES, PER_TILE = T::SLOTS_A + T::SLOTS_B;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, TM = WTM / 32, TN = WTN / 32;
    static_assert(WAVES_M * WAVES_N == 4 && TM * TN <= 8 && TM >= 2 && PER_TILE <= 63, "one matrix wave per SIMD; at most 128 accumulator registers a lane; vmcnt is a 6-bit counter");
    static_assert(!B_KN || BN >= 128, "the [K][N] permutation moves a chunk by up to 12 places inside its row");
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const unsigned long long t_entry = p.phase ? clock64() : 0ull;
    int tm_, tn_, sk_s = 0, sk_tile = 0;
    if constexpr (SK) {
        // K-slice s of tile xcd * tpx + slot is workgroup (slot * S + s) * 8 + xcd: a tile's slices share an XCD
        // (sk_finish says more).  An XCD's run of the tile order covers about as many row tiles as column tiles, so
        // its L2 pulls few panels of either operand: 1500 x 5120 -> 1280 fetched 156 MB with runs that walked whole
        // columns of 12 row tiles
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        sk_s = idx % p.sk_S;
        sk_tile = xcd * p.sk_tpx + idx / p.sk_S;
        if (sk_tile >= p.tiles_m * p.tiles_n) return;          // the whole workgroup: the last XCD's run may be short
        const int width = p.group_m * p.tiles_n, g = sk_tile / width, in = sk_tile - g * width;
        const int first = g * p.group_m, gsz = min(p.tiles_m - first, p.group_m);
        tm_ = first + in % gsz;
        tn_ = in / gsz;
    } else {
        tile_of(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, p.group_m, tm_, tn_);
    }
    // (the divisions above run on the vector unit: hand the results back to scalar registers, which the direct loads'
    // base addresses have to be in)
    const int m0 = __builtin_amdgcn_readfirstlane(tm_ * BM), n0 = __builtin_amdgcn_readfirstlane(tn_ * BN);
    sk_s = __builtin_amdgcn_readfirstlane(sk_s);
    const long bz = blockIdx.y;
    const int nk = SK ? p.K / BK / p.sk_S : p.K / BK;      // the launcher guarantees whole BK-deep tiles per slice
    const long a_step = BK * 2, b_step = B_KN ? (long)BK * p.ldB * 2 : BK * 2;
    const char *Ag = reinterpret_cast<const char *>(p.A + bz * p.sA + (long)m0 * p.ldA) + (SK ? (long)sk_s * nk * a_step : 0L);
    const char *Bg = reinterpret_cast<const char *>(p.B + bz * p.sB + (B_KN ? (long)n0 : (long)n0 * p.ldB)) + (SK ? (long)sk_s * nk * b_step : 0L);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;
    auto barrier = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // A launch whose store the helpers can share (coop_store_applies) has eight waves, and the four that do not multiply
    // take half of it (store_coop_epi): wave 4 + w shares a SIMD with matrix wave w.
    const bool coop = !SK && blockDim.x == 512 && coop_store_applies(p);      // uniform
    constexpr int COOP_BUF = 2 * 32 * (WTN + 8) * 2;                         // a matrix wave's two staging areas
    auto help_store = [&]() {
        const int mwave = wave - 4;
        store_coop<TM, WTN, true>(p, smem + mwave * COOP_BUF, m0 + (mwave % WAVES_M) * WTM, n0 + (mwave / WAVES_M) * WTN, lane, bz,
                                  [](auto) {}, barrier);
    };
    if (wave == 4) {
        // Per-lane offsets of the tile's 1 KB slots.  A tile that lies inside the operands needs no clamping, and its
        // slots s and s + 2 differ by a constant (eight rows of a K-contiguous operand, 64 / (BN / 8) k-rows of the
        // [K][N] one; the chunk permutation has period two in s): two offsets computed in full, the others one add
        // each -- this wave alone stands between the launch and the first request, at a vector instruction every
        // eight clocks.
        uint32_t offa[T::SLOTS_A], offb[T::SLOTS_B];
        if (m0 + BM <= p.M && n0 + BN <= (B_KN ? p.NB : p.N)) {          // uniform
            const uint32_t step_a = (uint32_t)(8 * p.ldA * 2), step_b = (uint32_t)((B_KN ? 64 / (BN / 8) : 8) * p.ldB * 2);
            const uint32_t a0 = T::a_offset(p, m0, 0, lane), a1 = T::a_offset(p, m0, 1, lane);
            const uint32_t b0 = T::b_offset(p, n0, 0, lane), b1 = T::b_offset(p, n0, 1, lane);
#pragma unroll
            for (int s = 0; s < T::SLOTS_A; s++) offa[s] = ((s & 1) ? a1 : a0) + (uint32_t)(s & ~1) * step_a;
#pragma unroll
            for (int s = 0; s < T::SLOTS_B; s++) offb[s] = ((s & 1) ? b1 : b0) + (uint32_t)(s & ~1) * step_b;
        } else {
#pragma unroll
            for (int s = 0; s < T::SLOTS_A; s++) offa[s] = T::a_offset(p, m0, s, lane);
#pragma unroll
            for (int s = 0; s < T::SLOTS_B; s++) offb[s] = T::b_offset(p, n0, s, lane);
        }
        auto request = [&](int kt, int stage) {
            const char *ab = Ag + (long)kt * a_step, *bb = Bg + (long)kt * b_step;
            const uint32_t sa = lds0 + stage * STAGE_BYTES, sb = sa + A_BYTES;
#pragma unroll
            for (int s = 0; s < T::SLOTS_A; s++) T::request(ab, offa[s], sa + s * 1024);
#pragma unroll
            for (int s = 0; s < T::SLOTS_B; s++) T::request(bb, offb[s], sb + s * 1024);
        };
        // requests complete in order: "tile t has landed" is "no more outstanding than were issued after it"
        request(0, 0);
        if (nk > 1) { request(1, 1); asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER_TILE) : "memory"); }
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        barrier();                                                  // tile 0 has landed
        if (nk > 2) request(2, 2);
        for (int kt = 0; kt < nk; kt++) {
            if (kt + 2 < nk) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER_TILE) : "memory");      // tile kt + 1 has landed
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            barrier();                                              // B_kt
            if (kt + 3 < nk) request(kt + 3, kt % 3);
        }
        if (coop) help_store();
        return;
    }
    float2v *ln_slot = reinterpret_cast<float2v *>(smem + STAGES * STAGE_BYTES);
    if (wave >= 5 && !(wave == 5 && p.lnf_stats)) {
        // nothing to do beside the K loop: keep the barriers' count, then help with the store
        barrier();
        for (int kt = 0; kt < nk; kt++) barrier();
        if (coop) help_store();
        return;
    }
    if (wave == 5) {
        // The statistics wave of a folded layer norm.  The matrix waves need (r, r mu) of
        // the tile's rows and the tile's columns of colsum and biasp at the store, not before: combining a row's
        // K / 32 segment statistics in the prologue held every wave at the first barrier (5 000 clocks at 128 rows,
        // 10 000 at 192: a trip to memory per batch of loads, then forty dependent steps a row).  This wave does it
        // beside the K loop instead: tile kt covers segments 2 kt and 2 kt + 1 (K % 64 == 0), so between two barriers
        // it takes in the two segments of each of its BM / 64 rows that it requested four tiles earlier, and the
        // result is in the LDS slot when it arrives at the last barrier, which the matrix waves pass before they
        // store.  Same arithmetic, in the same order per row, as lnf_stage with one lane a row.
        constexpr int NR = BM / 64, AHEAD = 4;
        static_assert(BM % 64 == 0 && NR * 2 * AHEAD <= 63, "whole rows per lane; vmcnt is a 6-bit counter");
        for (int t = lane; t < BN / 2; t += 64) {
            const int which = t / (BN / 4), c = (t % (BN / 4)) * 4, n = n0 + c;
            const float *src = (which == 0 ? p.lnf_colsum : p.lnf_biasp) + bz * p.lnf_svec;
            float4v v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (n + 3 < p.N) v = *reinterpret_cast<const float4v *>(src + n);
            else for (int e = 0; e < 4; e++) if (n + e < p.N) v[e] = src[n + e];
            *reinterpret_cast<float4v *>(reinterpret_cast<float *>(ln_slot + BM) + which * BN + c) = v;
        }
        const float2v *seg[NR];
#pragma unroll
        for (int i = 0; i < NR; i++) seg[i] = reinterpret_cast<const float2v *>(p.lnf_stats) + min(m0 + lane + 64 * i, p.M - 1);
        float2v v[AHEAD][NR][2];
        float ref[NR], total[NR], within[NR], between[NR];
#pragma unroll
        for (int i = 0; i < NR; i++) { ref[i] = 0.0f; total[i] = 0.0f; within[i] = 0.0f; between[i] = 0.0f; }
        auto fetch = [&](auto SLOT, int kt) {
            constexpr int sl = decltype(SLOT)::value;
#pragma unroll
            for (int i = 0; i < NR; i++)
#pragma unroll
                for (int h = 0; h < 2; h++) v[sl][i][h] = seg[i][(long)(2 * kt + h) * p.M];
        };
        auto take = [&](auto SLOT, int kt) {
            constexpr int sl = decltype(SLOT)::value;
#pragma unroll
            for (int i = 0; i < NR; i++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    if (kt == 0 && h == 0) ref[i] = v[sl][i][0][0] * (1.0f / 32.0f);
                    const float d = fmaf(v[sl][i][h][0], 1.0f / 32.0f, -ref[i]);
                    total[i] += v[sl][i][h][0];
                    within[i] += v[sl][i][h][1];
                    between[i] = fmaf(32.0f * d, d, between[i]);
                }
        };
        // tiles 0 .. AHEAD - 1 are requested before the first barrier; tile kt + AHEAD right after tile kt is taken in
        static_for<AHEAD>([&](auto S) { if (decltype(S)::value < nk) fetch(S, decltype(S)::value); });
        barrier();
        for (int kt0 = 0; kt0 < nk; kt0 += AHEAD) {
            static_for<AHEAD>([&](auto S) {
                const int kt = kt0 + decltype(S)::value;
                if (kt < nk) {
                    // requests complete in order: what was requested after tile kt may still be on its way
                    if (kt + AHEAD - 1 < nk) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * NR * 2) : "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    take(S, kt);
                    if (kt + AHEAD < nk) fetch(S, kt + AHEAD);
                    if (kt + 1 == nk) {
#pragma unroll
                        for (int i = 0; i < NR; i++) {
                            const float mu = total[i] / (float)p.K, dm = mu - ref[i];
                            const float m2 = within[i] + fmaxf(between[i] - (float)p.K * dm * dm, 0.0f);
                            const float r = 1.0f / sqrtf(m2 / (float)p.K + p.lnf_eps);
                            const float2v o = {r, r * mu};
                            ln_slot[lane + 64 * i] = o;
                        }
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    }
                    barrier();                                      // B_kt
                }
            });
        }
        if (coop) help_store();
        return;
    }
    // (a launch without the statistics wave and with a folded norm: combine in the prologue, as the other kernels do)
    if (blockDim.x < 384) lnf_stage<BM, BN, 256>(p, ln_slot, m0, n0, bz, tid);

    // fragment read offsets inside a stage (bytes): rows of A, and this wave's columns of B in either layout
    const int frow = lane & 31, fhi = lane >> 5;
    const int swz = T::rowswz(lane & 15);
    int a_rd[KS], b_rd[KS], bt_rd[TN];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const int cc = ((2 * ks + fhi) ^ swz) << 4;
        a_rd[ks] = (wm * WTM + frow) * ROWB + cc;
        b_rd[ks] = A_BYTES + (wn * WTN + frow) * ROWB + cc;
    }
    {
        const int kk = (lane >> 2) & 3;
#pragma unroll
        for (int i = 0; i < TN; i++) {
            const int col = (wn * WTN + i * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4) ^ (kk << 5);
            bt_rd[i] = A_BYTES + ((fhi * 8 + kk) * BN + col) * 2;
        }
    }
    // fragment q of a 16-deep step: q < TM the A rows 32 q .., else the wave's B columns 32 (q - TM) ..
    constexpr int NFRAG = TM + TN;
    auto read_frag = [&](const char *st, int ks, int q, half8v (&a)[TM], half8v (&b)[TN]) {
        if (q < TM) {
            a[q] = *reinterpret_cast<const half8v *>(st + a_rd[ks] + q * 32 * ROWB);
        } else if (!B_KN) {
            b[q - TM] = *reinterpret_cast<const half8v *>(st + b_rd[ks] + (q - TM) * 32 * ROWB);
        } else {
            const char *bs = st + bt_rd[q - TM] + ks * 16 * BN * 2;
            short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(bs));
            short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(bs + 4 * BN * 2));
            short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            b[q - TM] = __builtin_bit_cast(half8v, both);
        }
    };
    auto read_step = [&](const char *st, int ks, half8v (&a)[TM], half8v (&b)[TN]) {
#pragma unroll
        for (int q = 0; q < NFRAG; q++) read_frag(st, ks, q, a, b);
    };
    float16v acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    // The MFMAs of rows [JLO, JHI) x all columns of one step, from fragment set (a, b), with the reads of step ks of
    // the stage at st into set (da, db) dealt between them: a wave that issues its six or eight LDS instructions in
    // one burst stands at them while the LDS queue drains, and its matrix pipe runs dry behind it.  The scheduling
    // groups pin the order the source has: one MFMA, then the LDS reads that follow it.
    auto step = [&](auto JLO, auto JHI, const half8v (&a)[TM], const half8v (&b)[TN], const char *st, int ks, half8v (&da)[TM], half8v (&db)[TN]) {
        constexpr int jlo = decltype(JLO)::value, jhi = decltype(JHI)::value, NM = (jhi - jlo) * TN;
        static_for<NM>([&](auto Mi) {
            constexpr int m = decltype(Mi)::value, j = jlo + m / TN, i = m % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[i], a[j], acc[i][j], 0, 0, 0);
            constexpr int q0 = (m * NFRAG) / NM, q1 = ((m + 1) * NFRAG) / NM;      // fragments [q0, q1) go behind MFMA m
            static_for<q1 - q0>([&](auto Qi) { read_frag(st, ks, q0 + decltype(Qi)::value, da, db); });
        });
        static_for<NM>([&](auto Mi) {
            constexpr int m = decltype(Mi)::value, q0 = (m * NFRAG) / NM, q1 = ((m + 1) * NFRAG) / NM;
            constexpr int a_frags = (q1 < TM ? q1 : TM) - (q0 < TM ? q0 : TM), b_frags = (q1 - q0) - a_frags;
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (q1 > q0) __builtin_amdgcn_sched_group_barrier(0x100, a_frags + b_frags * (B_KN ? 2 : 1), 0);
        });
    };
    auto mma = [&](auto JLO, auto JHI, const half8v (&a)[TM], const half8v (&b)[TN]) {
        constexpr int jlo = decltype(JLO)::value, jhi = decltype(JHI)::value;
#pragma unroll
        for (int j = jlo; j < jhi; j++)
#pragma unroll
            for (int i = 0; i < TN; i++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[i], a[j], acc[i][j], 0, 0, 0);
    };
    const bool probe = p.clk && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0;
    if (probe) { p.clk[0] = clock64(); p.clk[1] = wall_clock64(); }
    const bool phases = p.phase && (int)blockIdx.x < p.phase_wgs && blockIdx.y == 0;      // uniform
    unsigned long long ph_t[4] = {0, 0, 0, t_entry};
    auto phase_mark = [&](int i) { if (phases) ph_t[i] = clock64(); };
    // Three sets of fragment registers: step s of a tile whose rotation is R sits in set (R + s) % 3, and the reads run
    // two steps ahead of the MFMAs (one step ahead, a wave's reads came back just too late: 6 KB per wave and step at the
    // 32 B/clock a SIMD takes from the LDS is 190 of the 256 clocks its eight MFMAs last, before any queueing).  Four
    // steps a tile, so the rotation advances by one per tile and the loop body is three tiles long.
    half8v fa[3][TM], fb[3][TN];
    half4v cb[TN][4];
    load_col_bias<TN, WTN>(p, cb, n0, wn, lane, bz);              // sixteen registers held through the loop; no trip to memory after it
    barrier();                                                      // tile 0 has landed
    read_step(smem, 0, fa[0], fb[0]);
    read_step(smem, 1, fa[1], fb[1]);
    int stage = 0;
    auto tile = [&](auto R, int kt) {
        constexpr int r = decltype(R)::value, s0 = r % 3, s1 = (r + 1) % 3, s2 = (r + 2) % 3;
        const char *st = smem + stage * STAGE_BYTES;
        stage = stage == STAGES - 1 ? 0 : stage + 1;
        const char *nx = smem + stage * STAGE_BYTES;
        using std::integral_constant;
        constexpr integral_constant<int, 0> J0{};
        constexpr integral_constant<int, TM / 2> JH{};
        constexpr integral_constant<int, TM> JE{};
        // steps 0 and 1, with the reads of steps 2 and 3
        step(J0, JE, fa[s0], fb[s0], st, 2, fa[s2], fb[s2]);
        __builtin_amdgcn_sched_barrier(0);
        step(J0, JE, fa[s1], fb[s1], st, 3, fa[s0], fb[s0]);
        __builtin_amdgcn_sched_barrier(0);
        // step 2: every fragment read of tile kt has returned before this wave lets the loader have the stage; the
        // reads of the next tile's steps 0 and 1 follow the barrier (past the last tile they fetch nothing anybody uses)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        mma(J0, JH, fa[s2], fb[s2]);
        __builtin_amdgcn_sched_barrier(0);
        barrier();                                                  // B_kt
        step(JH, JE, fa[s2], fb[s2], nx, 0, fa[s1], fb[s1]);
        __builtin_amdgcn_sched_barrier(0);
        // step 3
        step(J0, JE, fa[s0], fb[s0], nx, 1, fa[s2], fb[s2]);
        __builtin_amdgcn_sched_barrier(0);
        (void)kt;
    };
    phase_mark(0);
    for (int kt = 0;;) {
        tile(std::integral_constant<int, 0>{}, kt);
        if (++kt == nk) break;
        tile(std::integral_constant<int, 1>{}, kt);
        if (++kt == nk) break;
        tile(std::integral_constant<int, 2>{}, kt);
        if (++kt == nk) break;
    }
    phase_mark(1);
    auto phase_store = [&]() {
        if (!phases) return;
        const unsigned long long issued = clock64();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long done = clock64();
        if (lane == 0) {
            unsigned long long *t = p.phase + ((long)blockIdx.x * 4 + wave) * 4;
            t[0] = ph_t[0] - ph_t[3]; t[1] = ph_t[1] - ph_t[0]; t[2] = issued - ph_t[1]; t[3] = done - issued;
        }
    };
    if constexpr (SK) {
        sk_finish<TM, TN, WTM, WTN, 4, STAGES * STAGE_BYTES>(p, acc, cb, smem, sk_tile, sk_s, m0, n0, wm, wn, wave, lane, bz);
        phase_store();
        if (probe) { p.clk[2] = clock64(); p.clk[3] = wall_clock64(); }
        return;
    }
    LnFold<TM> ln;
    if (p.lnf_stats) {
        ln.on = true; ln.col = reinterpret_cast<const float *>(ln_slot + BM); ln.bn = BN;
#pragma unroll
        for (int j = 0; j < TM; j++) { const float2v v = ln_slot[wm * WTM + 32 * j + (lane & 31)]; ln.r[j] = v[0]; ln.rmu[j] = v[1]; }
    }
    if (coop) {
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) asm volatile("" ::"v"(cb[i][g]));      // in registers ahead of the first store (store_tile_simple)
        char *buf = smem + wave * COOP_BUF;
        store_coop<TM, WTN, false>(p, buf, m0 + wm * WTM, n0 + wn * WTN, lane, bz,
                                   [&](auto J) { constexpr int j = decltype(J)::value; stage_block<j, TM, TN, WTN>(acc, cb, ln, wn, buf + (j & 1) * (COOP_BUF / 2), lane); },
                                   barrier);
    } else {
        store_tile<TM, TN, WTM, WTN, 4, STAGES * STAGE_BYTES>(p, acc, cb, smem, m0, n0, wm, wn, wave, lane, bz, ln);
    }
    phase_store();
    if (probe) { p.clk[2] = clock64(); p.clk[3] = wall_clock64(); }
}

// ------------------------------------------------------------------------------------------
// Scalar kernel: one thread per output, fp32 accumulation seeded with the bias,
// any strides.  The arithmetic of the reference's mm2 (matmul.jl:17-27).
__global__ void gemm_scalar_kernel(GemmArgs p, int b_kn) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long total = (long)p.M * p.N;
    if (idx >= total) return;
    int n = (int)(idx % p.N), m = (int)(idx / p.N);
    long bz = blockIdx.y;
    const half_t *A = p.A + bz * p.sA + (long)m * p.ldA;
    const half_t *B = p.B + bz * p.sB;
    const half_t *bias = p.bias ? p.bias + bz * p.sBias : nullptr;
    float acc = p.bias_mode == MI_BIAS_COL ? (float)bias[n] : p.bias_mode == MI_BIAS_ROW ? (float)bias[m] : 0.0f;
    if (b_kn) for (int k = 0; k < p.K; k++) acc = fmaf((float)A[k], (float)B[(long)k * p.ldB + n], acc);
    else      for (int k = 0; k < p.K; k++) acc = fmaf((float)A[k], (float)B[(long)n * p.ldB + k], acc);
    long off = bz * p.sY + (long)m * p.ldY + n;
    if (p.out_f32) reinterpret_cast<float *>(p.Y)[off] = apply_epi(acc, p.epi);
    else {
        half_t o = (half_t)apply_epi((float)(half_t)acc, p.epi);
        if (p.residual) o = (half_t)((float)o + (float)p.residual[off]);
        reinterpret_cast<half_t *>(p.Y)[off] = o;
    }
}

// ------------------------------------------------------------------------------------------
// Decode-sized M (<= 8): bandwidth- and latency-bound.  Every weight byte is read once with
// 16-byte loads, a thread's loads are all issued before the first is used, and the activations
// (a few KB) are staged in LDS.  Products go through v_dot2_f32_f16: fp16 pairs, fp32 sum.
//
// [K][F] weights: a thread owns 8 consecutive columns, 16 threads span 128 columns, the 16 thread
// rows of a workgroup take interleaved k-pairs.  K is split over workgroups so that the whole chip
// pulls on HBM; each split writes an fp32 partial plane and skinny_epilogue_kernel sums the planes
// (the reference's split-K planes + mm_epilogue_kernel!, matmul.jl:192-217).
// Layer-norm statistics of up to MT rows of A, one wave per row, in the summation order of
// layernorm_vec_kernel (a lane takes the 16-byte chunks lane, lane + 64, ...; butterfly over the wave):
// the fused result is bit-identical to running that kernel first.  stats[m] = (mean, rstd).
template <int MT, int NCH = 8>                              // rows up to NCH * 512 halves stay in registers between the passes
__device__ __forceinline__ void ln_row_stats(const GemmArgs &p, float (*stats)[2], int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    for (int m = wave; m < MT && m < p.M; m += 4) {
        const half_t *row = p.A + (long)m * p.ldA;
        float s = 0.0f, s2 = 0.0f;
        if (p.K <= NCH * 512) {
            u32x4 raw[NCH];
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int e0 = (lane + 64 * i) * 8;
                const u32x4 z = {0u, 0u, 0u, 0u};
                raw[i] = e0 < p.K ? ldg16(row + e0) : z;
            }
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                if ((lane + 64 * i) * 8 < p.K) {
                    const half8v t = as_half8(raw[i]);
#pragma unroll
                    for (int j = 0; j < 8; j++) s += (float)t[j];
                }
            }
            s = wave_sum(s);
            const float mu = s / (float)p.K;
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                if ((lane + 64 * i) * 8 < p.K) {
                    const half8v t = as_half8(raw[i]);
#pragma unroll
                    for (int j = 0; j < 8; j++) { const float d = (float)t[j] - mu; s2 = fmaf(d, d, s2); }
                }
            }
            s2 = wave_sum(s2);
            if (lane == 0) { stats[m][0] = mu; stats[m][1] = 1.0f / sqrtf(s2 / (float)p.K + p.ln_eps); }
        } else {
            for (int e0 = lane * 8; e0 < p.K; e0 += 512) {
                const half8v t = as_half8(ldg16(row + e0));
#pragma unroll
                for (int j = 0; j < 8; j++) s += (float)t[j];
            }
            s = wave_sum(s);
            const float mu = s / (float)p.K;
            for (int e0 = lane * 8; e0 < p.K; e0 += 512) {
                const half8v t = as_half8(ldg16(row + e0));
#pragma unroll
                for (int j = 0; j < 8; j++) { const float d = (float)t[j] - mu; s2 = fmaf(d, d, s2); }
            }
            s2 = wave_sum(s2);
            if (lane == 0) { stats[m][0] = mu; stats[m][1] = 1.0f / sqrtf(s2 / (float)p.K + p.ln_eps); }
        }
    }
}

// Eight activations of row statistics (mu, r) at column k0 of A, normalised and rounded as layernorm_vec_kernel does.
__device__ __forceinline__ u32x4 ln_apply8(const GemmArgs &p, u32x4 raw, float mu, float r, int k0) {
    const half8v x = as_half8(raw);
    half8v gv, bv, o;
    if (p.ln_gamma) gv = as_half8(ldg16(p.ln_gamma + k0));
    if (p.ln_beta) bv = as_half8(ldg16(p.ln_beta + k0));
#pragma unroll
    for (int j = 0; j < 8; j++)
        o[j] = ln_norm1((float)x[j], mu, r, p.ln_gamma != nullptr, p.ln_gamma ? (float)gv[j] : 0.0f, p.ln_beta != nullptr, p.ln_beta ? (float)bv[j] : 0.0f);
    return __builtin_bit_cast(u32x4, o);
}

constexpr int SKN_COLS = 128;      // columns per workgroup
constexpr int SKN_KMAX = 256;      // deepest k-slice: 16 loads of 16 bytes per thread, all in flight at once
constexpr int SKN_LOADS = SKN_KMAX / 32;

template <int MT>
__global__ __launch_bounds__(256) void skinny_kn_kernel(GemmArgs p, float *part, int kper) {
    __shared__ __align__(16) half_t xs[MT][SKN_KMAX];
    __shared__ float red[4][MT][SKN_COLS];
    __shared__ float lnst[MT][2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cx = tid & 15, ky = tid >> 4;            // ky = 0..15: k-pairs 2 ky, 2 ky + 1 (+ 32 i)
    const int n = blockIdx.x * SKN_COLS + cx * 8;
    const int split = blockIdx.y;
    const int k0 = split * kper, klen = min(p.K - k0, kper);     // kper % 32 == 0, K % 8 == 0
    // weights first: they are what the memory system has to deliver
    u32x4 w[SKN_LOADS][2];
    const bool ncol = n < p.N;                          // NB % 8 == 0: a thread's 8 columns are in the row or all past N
    const half_t *bp = p.B + (long)k0 * p.ldB + n;
#pragma unroll
    for (int i = 0; i < SKN_LOADS; i++) {
        const int k = 32 * i + 2 * ky;
        const u32x4 z = {0u, 0u, 0u, 0u};
        if (32 * i < kper) {
            w[i][0] = (ncol && k < klen) ? ldg16(bp + (long)k * p.ldB) : z;
            w[i][1] = (ncol && k + 1 < klen) ? ldg16(bp + (long)(k + 1) * p.ldB) : z;
        }
    }
    if (p.ln_on) {                                      // uniform
        ln_row_stats<MT>(p, lnst, tid);
        __syncthreads();
    }
    for (int c = tid; c < MT * (kper >> 3); c += 256) {
        const int m = c / (kper >> 3), ch = c % (kper >> 3);
        u32x4 v = {0u, 0u, 0u, 0u};
        if (m < p.M && ch * 8 < klen) {
            v = ldg16(p.A + (long)m * p.ldA + k0 + ch * 8);
            if (p.ln_on) v = ln_apply8(p, v, lnst[m][0], lnst[m][1], k0 + ch * 8);
        }
        *reinterpret_cast<u32x4 *>(&xs[m][ch * 8]) = v;
    }
    __syncthreads();
    float acc[MT][8];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[m][e] = 0.0f;
#pragma unroll
    for (int i = 0; i < SKN_LOADS; i++) {
        if (32 * i < kper) {
            const int k = 32 * i + 2 * ky;
            // (w[k][n+e], w[k+1][n+e]) pairs
            uint32_t pr[8];
#pragma unroll
            for (int q = 0; q < 4; q++) { pr[2 * q] = pack_lo(w[i][0][q], w[i][1][q]); pr[2 * q + 1] = pack_hi(w[i][0][q], w[i][1][q]); }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const half2v x = *reinterpret_cast<const half2v *>(&xs[m][k]);
#pragma unroll
                for (int e = 0; e < 8; e++) acc[m][e] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, pr[e]), x, acc[m][e], false);
            }
        }
    }
    // a wave holds 4 thread rows of the same 16 column groups: fold them, then the 4 waves through LDS
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float v = acc[m][e];
            float x0 = v, y0 = v;
            swap_rows16(x0, y0); v = x0 + y0;            // v[lane] + v[lane ^ 16]
            x0 = v; y0 = v;
            swap_rows32(x0, y0); v = x0 + y0;            // ... + the same of lane ^ 32
            if (lane < 16) red[wave][m][cx * 8 + e] = v;
        }
    __syncthreads();
    for (int c = tid; c < MT * SKN_COLS; c += 256) {
        const int m = c / SKN_COLS, col = c % SKN_COLS;
        const int nn = blockIdx.x * SKN_COLS + col;
        if (m < p.M && nn < p.N) part[((long)split * p.M + m) * p.N + nn] = (red[0][m][col] + red[1][m][col]) + (red[2][m][col] + red[3][m][col]);
    }
}

// out[m][n] = epi(round(sum_s part[s][m][n] + bias)) (+ residual).  A thread's plane loads are
// issued eight at a time, so the sum costs a few memory round trips, not one per plane.
__global__ void skinny_epilogue_kernel(GemmArgs p, const float *part, int nsplit) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long total = (long)p.M * p.N;
    if (idx >= total) return;
    int n = (int)(idx % p.N), m = (int)(idx / p.N);
    float v = p.bias_mode == MI_BIAS_COL ? (float)p.bias[n] : p.bias_mode == MI_BIAS_ROW ? (float)p.bias[m] : 0.0f;
    int s = 0;
    for (; s + 8 <= nsplit; s += 8) {
        float t[8];
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = part[(long)(s + j) * total + idx];
        v += ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
    }
    for (; s < nsplit; s++) v += part[(long)s * total + idx];
    long off = (long)m * p.ldY + n;
    if (p.out_f32) reinterpret_cast<float *>(p.Y)[off] = apply_epi(v, p.epi);
    else {
        half_t o = (half_t)apply_epi((float)(half_t)v, p.epi);
        if (p.residual) o = (half_t)((float)o + (float)p.residual[off]);
        reinterpret_cast<half_t *>(p.Y)[off] = o;
    }
}

// [F][K] weights (K-contiguous): one wave per output column, lanes stride K in 16-byte chunks,
// wave reduction, and the epilogue in the same launch: no workspace, no second kernel.  The
// activations are staged in LDS once per workgroup (dynamic: MT rows of K halves).
//
// A decode-sized call moves a few MB, so its duration is a chain of trips to memory, not bandwidth.  Everything whose
// address does not depend on loaded data is therefore requested at the top, before anything is waited for: the wave's
// weight row (FK_PF chunks of 16 bytes per lane: K <= 6144 whole), its bias and residual elements, the thread's
// share of the activations and of gamma / beta.  The statistics of the layer-norm prologue, the staging and the dot
// products then run on data that arrives together: one trip instead of three or four in a row.
// FK_PF = 3 (K <= 1536) or 12: the registers of the up-front requests decide how many waves a SIMD holds, and a
// wide output (1280 -> 5120 is five waves per SIMD, a vocabulary projection many more) needs them all resident.
template <int MT, int FK_PF>
__global__ __launch_bounds__(256) void skinny_fk_kernel(GemmArgs p) {
    // activation chunks per thread requested up front: the whole MT x K panel up to four per thread
    constexpr int FK_XCAP = MT == 8 ? 1 : 4;              // eight rows of accumulators and operands leave room for one
    constexpr int FK_XPF = (MT * FK_PF * 64 + 255) / 256 < FK_XCAP ? (MT * FK_PF * 64 + 255) / 256 : FK_XCAP;
    extern __shared__ __align__(16) char smem[];
    half_t *xs = reinterpret_cast<half_t *>(smem);       // [MT][K]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __shared__ float lnst[MT][2];
    const int kch = p.K >> 3;
    const u32x4 z = {0u, 0u, 0u, 0u};
    const int n = blockIdx.x * 4 + wave;
    const bool live = n < p.N;                            // uniform over the wave
    const half_t *bp = p.B + (long)(live ? n : 0) * p.ldB;
    u32x4 w[FK_PF];
#pragma unroll
    for (int i = 0; i < FK_PF; i++) w[i] = live && lane * 8 + 512 * i < p.K ? ldg16(bp + lane * 8 + 512 * i) : z;
    float bv = 0.0f, rv = 0.0f;
    if (live && lane < p.M) {
        if (p.bias_mode == MI_BIAS_COL) bv = (float)p.bias[n];
        else if (p.bias_mode == MI_BIAS_ROW) bv = (float)p.bias[lane];
        if (p.residual && !p.out_f32) rv = (float)p.residual[(long)lane * p.ldY + n];
    }
    u32x4 xr[FK_XPF], gr[FK_XPF], br[FK_XPF];
#pragma unroll
    for (int i = 0; i < FK_XPF; i++) {
        const int c = tid + 256 * i, m = c / kch, ch = c % kch;
        xr[i] = gr[i] = br[i] = z;
        if (c < MT * kch && m < p.M) {
            xr[i] = ldg16(p.A + (long)m * p.ldA + ch * 8);
            if (p.ln_on && p.ln_gamma) gr[i] = ldg16(p.ln_gamma + ch * 8);
            if (p.ln_on && p.ln_beta) br[i] = ldg16(p.ln_beta + ch * 8);
        }
    }
    if (p.ln_on) {                                      // uniform
        ln_row_stats<MT, (FK_PF < 8 ? FK_PF : 8)>(p, lnst, tid);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < FK_XPF; i++) {
        const int c = tid + 256 * i, m = c / kch, ch = c % kch;
        if (c < MT * kch) {
            u32x4 v = xr[i];
            if (p.ln_on && m < p.M) {
                const half8v x = as_half8(v), gv = as_half8(gr[i]), bb = as_half8(br[i]);
                half8v o;
#pragma unroll
                for (int j = 0; j < 8; j++)
                    o[j] = ln_norm1((float)x[j], lnst[m][0], lnst[m][1], p.ln_gamma != nullptr, (float)gv[j], p.ln_beta != nullptr, (float)bb[j]);
                v = __builtin_bit_cast(u32x4, o);
            }
            *reinterpret_cast<u32x4 *>(xs + (long)m * p.K + ch * 8) = v;
        }
    }
    for (int c = tid + 256 * FK_XPF; c < MT * kch; c += 256) {
        const int m = c / kch, ch = c % kch;
        u32x4 v = z;
        if (m < p.M) {
            v = ldg16(p.A + (long)m * p.ldA + ch * 8);
            if (p.ln_on) v = ln_apply8(p, v, lnst[m][0], lnst[m][1], ch * 8);
        }
        *reinterpret_cast<u32x4 *>(xs + (long)m * p.K + ch * 8) = v;
    }
    __syncthreads();
    if (!live) return;
    // A wave walks columns n, n + 4 gridDim.x, ...: one for the widths of a decoder layer (the launcher gives every
    // column its wave), several for a vocabulary-sized output, where the staged activations and their norm are then
    // paid once per workgroup instead of once per four columns and the next column's row is requested under the
    // current one's dot products.
    const int stride = (int)gridDim.x * 4;
    for (int nc = n; nc < p.N; nc += stride) {
        const int nn = nc + stride;
        const bool more = nn < p.N;                       // uniform over the wave
        const half_t *bn = p.B + (long)(more ? nn : nc) * p.ldB;
        u32x4 wn[FK_PF];
        float bvn = 0.0f, rvn = 0.0f;
        if (more) {
#pragma unroll
            for (int i = 0; i < FK_PF; i++) wn[i] = lane * 8 + 512 * i < p.K ? ldg16(bn + lane * 8 + 512 * i) : z;
            if (lane < p.M) {
                if (p.bias_mode == MI_BIAS_COL) bvn = (float)p.bias[nn];
                else if (p.bias_mode == MI_BIAS_ROW) bvn = (float)p.bias[lane];
                if (p.residual && !p.out_f32) rvn = (float)p.residual[(long)lane * p.ldY + nn];
            }
        }
        float acc[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] = 0.0f;
        auto dot = [&](const u32x4 &wv, int k) {
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const u32x4 x = *reinterpret_cast<const u32x4 *>(xs + (long)m * p.K + k);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t wq = wv[q], xq = x[q];     // bit_cast wants an addressable scalar, not a vector element
                    acc[m] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, wq), __builtin_bit_cast(half2v, xq), acc[m], false);
                }
            }
        };
#pragma unroll
        for (int i = 0; i < FK_PF; i++)
            if (lane * 8 + 512 * i < p.K) dot(w[i], lane * 8 + 512 * i);
        const half_t *bc = p.B + (long)nc * p.ldB;
        for (int kb = lane * 8 + 512 * FK_PF; kb < p.K; kb += 4 * 512) {
            u32x4 t[4];
#pragma unroll
            for (int i = 0; i < 4; i++) t[i] = kb + 512 * i < p.K ? ldg16(bc + kb + 512 * i) : z;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (kb + 512 * i < p.K) dot(t[i], kb + 512 * i);
        }
        float mine = 0.0f;                                    // lane m keeps row m's sum
#pragma unroll
        for (int m = 0; m < MT; m++) {
            float sres = acc[m];
            sres = wave_sum(sres);
            if (lane == m) mine = sres;
        }
        if (lane < p.M) {
            const float v = mine + bv;
            const long off = (long)lane * p.ldY + nc;
            if (p.out_f32) reinterpret_cast<float *>(p.Y)[off] = apply_epi(v, p.epi);
            else {
                half_t o = (half_t)apply_epi((float)(half_t)v, p.epi);
                if (p.residual) o = (half_t)((float)o + rv);
                reinterpret_cast<half_t *>(p.Y)[off] = o;
            }
        }
        if (more) {
#pragma unroll
            for (int i = 0; i < FK_PF; i++) w[i] = wn[i];
            bv = bvn; rv = rvn;
        }
    }
}

// The same product with the activations in registers instead of LDS, for the few rows of a decode step: a lane's
// weight chunks sit at k = 8 lane + 512 i, so it needs exactly those chunks of every activation row and asks for
// them itself (the rows come from the L2: every wave of the launch reads the same few KB).  No staging, no barrier:
// a wave is a chain of one trip to memory, the norm statistics (its own copy, same summation order as
// ln_row_stats, so the same bits), the dot products, one wave reduction and a store.  R output columns per wave,
// all their weight rows requested up front.  (MT + R + 2) * PF chunks of registers: built for one and two rows of
// K <= 1536 (78 to 119 registers, four to six waves per SIMD); four rows, or K = 5120, would leave a SIMD one or
// two waves and stay with the staged kernel.
template <int MT, int PF, int R>
__global__ __launch_bounds__(256) void skinny_fk_reg_kernel(GemmArgs p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const u32x4 z = {0u, 0u, 0u, 0u};
    const int n0 = (blockIdx.x * 4 + wave) * R;
    if (n0 >= p.N) return;                                // uniform over the wave; no barrier below
    u32x4 w[R][PF];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const half_t *bp = p.B + (long)min(n0 + r, p.N - 1) * p.ldB;
#pragma unroll
        for (int i = 0; i < PF; i++) w[r][i] = lane * 8 + 512 * i < p.K ? ldg16(bp + lane * 8 + 512 * i) : z;
    }
    u32x4 x[MT][PF], gr[PF], br[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) {
        const int k = lane * 8 + 512 * i;
        gr[i] = br[i] = z;
#pragma unroll
        for (int m = 0; m < MT; m++) x[m][i] = m < p.M && k < p.K ? ldg16(p.A + (long)m * p.ldA + k) : z;
        if (p.ln_on && k < p.K) {
            if (p.ln_gamma) gr[i] = ldg16(p.ln_gamma + k);
            if (p.ln_beta) br[i] = ldg16(p.ln_beta + k);
        }
    }
    float bv[R], rv[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        bv[r] = rv[r] = 0.0f;
        if (lane < p.M && n0 + r < p.N) {
            if (p.bias_mode == MI_BIAS_COL) bv[r] = (float)p.bias[n0 + r];
            else if (p.bias_mode == MI_BIAS_ROW) bv[r] = (float)p.bias[lane];
            if (p.residual && !p.out_f32) rv[r] = (float)p.residual[(long)lane * p.ldY + n0 + r];
        }
    }
    if (p.ln_on) {                                        // uniform
#pragma unroll
        for (int m = 0; m < MT; m++) {
            float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int i = 0; i < PF; i++) {
                if (lane * 8 + 512 * i < p.K) {
                    const half8v t = as_half8(x[m][i]);
#pragma unroll
                    for (int j = 0; j < 8; j++) s1 += (float)t[j];
                }
            }
            s1 = wave_sum(s1);
            const float mu = s1 / (float)p.K;
#pragma unroll
            for (int i = 0; i < PF; i++) {
                if (lane * 8 + 512 * i < p.K) {
                    const half8v t = as_half8(x[m][i]);
#pragma unroll
                    for (int j = 0; j < 8; j++) { const float d = (float)t[j] - mu; s2 = fmaf(d, d, s2); }
                }
            }
            s2 = wave_sum(s2);
            const float rs = 1.0f / sqrtf(s2 / (float)p.K + p.ln_eps);
#pragma unroll
            for (int i = 0; i < PF; i++) {
                const half8v t = as_half8(x[m][i]), gv = as_half8(gr[i]), bb = as_half8(br[i]);
                half8v o;
#pragma unroll
                for (int j = 0; j < 8; j++) o[j] = ln_norm1((float)t[j], mu, rs, p.ln_gamma != nullptr, (float)gv[j], p.ln_beta != nullptr, (float)bb[j]);
                x[m][i] = lane * 8 + 512 * i < p.K ? __builtin_bit_cast(u32x4, o) : z;
            }
        }
    }
    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MT; m++) acc[r][m] = 0.0f;
#pragma unroll
    for (int i = 0; i < PF; i++)
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t wq = w[r][i][q], xq = x[m][i][q];
                    acc[r][m] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, wq), __builtin_bit_cast(half2v, xq), acc[r][m], false);
                }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float mine = 0.0f;                                // lane m keeps row m's sum
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const float sres = wave_sum(acc[r][m]);
            if (lane == m) mine = sres;
        }
        if (lane < p.M && n0 + r < p.N) {
            const float v = mine + bv[r];
            const long off = (long)lane * p.ldY + n0 + r;
            if (p.out_f32) reinterpret_cast<float *>(p.Y)[off] = apply_epi(v, p.epi);
            else {
                half_t o = (half_t)apply_epi((float)(half_t)v, p.epi);
                if (p.residual) o = (half_t)((float)o + rv[r]);
                reinterpret_cast<half_t *>(p.Y)[off] = o;
            }
        }
    }
}

// Split-K epilogue: out = epi(round(sum_s part[s] + bias)) (+ residual), four columns per thread.
// The counterpart of mm_epilogue_kernel! (matmul.jl:192-217): the planes are fp32 M x N.
__global__ void splitk_epilogue_kernel(GemmArgs p, const float *part, int nsplit) {
    const long idx = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const long total = (long)p.M * p.N;
    if (idx >= total) return;
    const int n = (int)(idx % p.N), m = (int)(idx / p.N);
    float4v v = *reinterpret_cast<const float4v *>(part + idx);
    for (int s = 1; s < nsplit; s++) {
        float4v w = *reinterpret_cast<const float4v *>(part + (long)s * total + idx);
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] += w[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++)
        v[e] += p.bias_mode == MI_BIAS_COL ? (float)p.bias[n + e] : p.bias_mode == MI_BIAS_ROW ? (float)p.bias[m] : 0.0f;
    const long off = (long)m * p.ldY + n;
    if (p.out_f32) {
#pragma unroll
        for (int e = 0; e < 4; e++) reinterpret_cast<float *>(p.Y)[off + e] = apply_epi(v[e], p.epi);
    } else {
        half4v o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (half_t)apply_epi((float)(half_t)v[e], p.epi);
        if (p.residual) {
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = (half_t)((float)o[e] + (float)p.residual[off + e]);
        }
        if (p.clamp > 0.0f) {
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = (half_t)fminf(fmaxf((float)o[e], -p.clamp), p.clamp);
        }
        if (p.vec_store) *reinterpret_cast<half4v *>(reinterpret_cast<half_t *>(p.Y) + off) = o;
        else {
#pragma unroll
            for (int e = 0; e < 4; e++) reinterpret_cast<half_t *>(p.Y)[off + e] = o[e];
        }
    }
}

// The same sums, bias, activation and residual as splitk_epilogue_kernel, one wave per output row, followed by the
// layer norm of that row into p.lnout: lane and chunk order, summation order and rounding are those of
// layernorm_vec_kernel, so Y and lnout carry the bits the two separate launches would have written.
template <int NCH>
__global__ __launch_bounds__(256) void splitk_epilogue_ln_kernel(GemmArgs p, const float *part, int nsplit) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long m = (long)blockIdx.x * 4 + wave;
    if (m >= p.M) return;
    const long total = (long)p.M * p.N;
    const u32x4 z = {0u, 0u, 0u, 0u};
    u32x4 graw[NCH], braw[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        graw[i] = (p.lnout_gamma && e0 < p.N) ? ldg16(p.lnout_gamma + e0) : z;
        braw[i] = (p.lnout_beta && e0 < p.N) ? ldg16(p.lnout_beta + e0) : z;
    }
    float x[NCH][8];
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < p.N) {
            const float *pp = part + m * p.N + e0;
            float4v v0 = *reinterpret_cast<const float4v *>(pp), v1 = *reinterpret_cast<const float4v *>(pp + 4);
            for (int sp = 1; sp < nsplit; sp++) {
                const float4v w0 = *reinterpret_cast<const float4v *>(pp + (long)sp * total), w1 = *reinterpret_cast<const float4v *>(pp + (long)sp * total + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) { v0[e] += w0[e]; v1[e] += w1[e]; }
            }
            const long off = m * p.ldY + e0;
            half8v o;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                float v = e < 4 ? v0[e] : v1[e - 4];
                v += p.bias_mode == MI_BIAS_COL ? (float)p.bias[e0 + e] : p.bias_mode == MI_BIAS_ROW ? (float)p.bias[m] : 0.0f;
                o[e] = (half_t)apply_epi((float)(half_t)v, p.epi);
            }
            if (p.residual) {
                const half8v rv = as_half8(ldg16(p.residual + off));
#pragma unroll
                for (int e = 0; e < 8; e++) o[e] = (half_t)((float)o[e] + (float)rv[e]);
            }
            if (p.clamp > 0.0f) {
#pragma unroll
                for (int e = 0; e < 8; e++) o[e] = (half_t)fminf(fmaxf((float)o[e], -p.clamp), p.clamp);
            }
            *reinterpret_cast<half8v *>(reinterpret_cast<half_t *>(p.Y) + off) = o;
#pragma unroll
            for (int j = 0; j < 8; j++) { x[i][j] = (float)o[j]; s += x[i][j]; }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) x[i][j] = 0.0f;
        }
    }
    s = wave_sum(s);
    const float mu = s / (float)p.N;
    float s2 = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        if ((lane + 64 * i) * 8 < p.N) {
#pragma unroll
            for (int j = 0; j < 8; j++) { const float d = x[i][j] - mu; s2 = fmaf(d, d, s2); }
        }
    }
    s2 = wave_sum(s2);
    const float r = 1.0f / sqrtf(s2 / (float)p.N + p.lnout_eps);
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int e0 = (lane + 64 * i) * 8;
        if (e0 < p.N) {
            const half8v gv = as_half8(graw[i]), bv = as_half8(braw[i]);
            half8v o;
#pragma unroll
            for (int j = 0; j < 8; j++)
                o[j] = ln_norm1(x[i][j], mu, r, p.lnout_gamma != nullptr, p.lnout_gamma ? (float)gv[j] : 0.0f, p.lnout_beta != nullptr, p.lnout_beta ? (float)bv[j] : 0.0f);
            *reinterpret_cast<half8v *>(p.lnout + m * p.N + e0) = o;
        }
    }
}

// ------------------------------------------------------------------------------------------
bool g_ready = false;
int g_cus = 256;
// Inside mi_*_plan_caps the planners answer for the device the caller describes instead of the one they run on.
thread_local int tl_plan_cus = 0;          // > 0: compute units to plan for
thread_local bool tl_plan_mfma = true;     // false: the described device has no matrix unit
unsigned long long *g_clock_probe = nullptr;      // mi_set_clock_probe
unsigned long long *g_phase_probe = nullptr;      // mi_set_phase_probe
int g_phase_wgs = 0;

// Scratch of mi_gemm_f16_noalloc: every GPU the library runs on holds its own copy of this array, at its own
// address, until the process ends.  Host code never uses the name as a pointer; g_scratch_ptr[device] is the
// address hipGetSymbolAddress gave with that device current.
constexpr int MAX_DEVICES = 64;
void *g_scratch_ptr[MAX_DEVICES] = {};

unsigned *g_sk_flags_ptr[MAX_DEVICES] = {};
unsigned *g_status_ptr[MAX_DEVICES] = {};    // the device's copy of device_status_words
int g_sk_state[MAX_DEVICES] = {};            // 0: not probed, 1: usable, -1: this device does not deal workgroups round robin
std::atomic<unsigned> g_sk_epoch{0};
std::atomic<bool> g_sk_enabled{true};        // mi_set_in_launch_exchange
constexpr int SK_SPIN_DEFAULT = 1 << 18;     // polls of a few hundred ns each: a partner that has not shown up after ~0.1 s will not
int g_sk_spin = SK_SPIN_DEFAULT;             // mi_test_exchange_faults
unsigned g_sk_pub_xor = 0, g_sk_xcc_xor = 0;

// Workgroup -> XCD: every workgroup of a 1024-workgroup probe writes the id of the XCD it runs on (HW_REG_XCC_ID).
__global__ void xcc_probe_kernel(unsigned *out) {
    if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | 20);      // XCC_ID, bits 3:0
}

// The split-K peer reduction relies on workgroups pid, pid + 8, pid + 16, ... sharing an XCD (one L2).  Checked once
// per device on a probe launch: all workgroups with the same pid % 8 must report one XCD.  Uses the flag words as the
// probe's output (they are zeroed again) and synchronises the device: call from mi_init only.
int sk_probe_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return -1;
    if (g_sk_state[dev]) return g_sk_state[dev];
    void *ptr = nullptr, *sptr = nullptr;
    if (hipGetSymbolAddress(&sptr, HIP_SYMBOL(device_status_words)) != hipSuccess || !sptr) return g_sk_state[dev] = -1;
    g_status_ptr[dev] = reinterpret_cast<unsigned *>(sptr);
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(sk_flag_words)) != hipSuccess || !ptr) return g_sk_state[dev] = -1;
    g_sk_flags_ptr[dev] = reinterpret_cast<unsigned *>(ptr);
    constexpr int NP = 1024;
    static_assert(NP <= SK_BANKS * SK_FLAGS, "probe output fits the flag words");
    unsigned host[NP];
    hipLaunchKernelGGL(xcc_probe_kernel, dim3(NP), dim3(64), 0, 0, g_sk_flags_ptr[dev]);
    bool ok = hipGetLastError() == hipSuccess && hipMemcpy(host, g_sk_flags_ptr[dev], sizeof(host), hipMemcpyDeviceToHost) == hipSuccess;
    ok = ok && hipMemset(g_sk_flags_ptr[dev], 0, sizeof(host)) == hipSuccess && hipDeviceSynchronize() == hipSuccess;
    for (int i = 8; ok && i < NP; i++) ok = host[i] == host[i & 7];
    return g_sk_state[dev] = ok ? 1 : -1;
}
bool sk_usable() {
    int dev = -1;
    return g_sk_enabled.load() && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < MAX_DEVICES && g_sk_state[dev] == 1;
}

// The current device's copy of `scratch`; resolved once per device, with that device current.  Null on failure.
void *scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

template <typename KernelT>
int raise_lds(KernelT kern, int bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess ? 0 : 1;
}

// LDS of the four-wave kernel: three 64-deep stages of both operands (the store's staging reuses them), then a folded
// layer norm's (r, r mu) per row and colsum and biasp per column
template <int BM, int BN>
constexpr int w4_lds_bytes() { return 3 * (BM + BN) * 64 * 2 + BM * 8 + BN * 8; }

template <int BM, int BN, int BK>
constexpr int gemm_lds_bytes() {
    constexpr int kc = BN * (BK + 8), kn = BK * (BN + 32);       // B buffer in either layout
    return 2 * (BM * (BK + 8) + (kc > kn ? kc : kn)) * 2 + BM * 8 + BN * 8;      // + a folded layer norm's (r, r mu) per row, colsum and biasp per column
}

#define GEMM_BIG 128, 256, 64, 2, 2
#define GEMM_MID 128, 128, 64, 2, 2
#define GEMM_SMALL 64, 64, 64, 2, 2

// k-slice depth for the [K][F] skinny kernel: enough workgroups to put ~2 on every CU, slices a
// multiple of 32 within [64, SKN_KMAX].
int skinny_kper(int64_t K, int64_t F) {
    const int64_t colblocks = ceil_div(F, SKN_COLS);
    const int64_t want = ceil_div(2 * (int64_t)mi_num_cus(), colblocks);
    int64_t kper = (int64_t)round_up((size_t)ceil_div(K, want), 32);
    if (kper < 64) kper = 64;
    if (kper > SKN_KMAX) kper = SKN_KMAX;
    return (int)kper;
}
int skinny_splits(int64_t K, int64_t F) { return (int)ceil_div(K, skinny_kper(K, F)); }
constexpr size_t SKINNY_FK_LDS_MAX = 128 * 1024;    // activations of the [F][K] kernel: M rows of K halves

bool mfma_addressable(const GemmArgs &a, bool b_kn) {
    if (a.K % 8 || a.ldA % 8 || a.ldB % 8 || a.sA % 8 || a.sB % 8) return false;
    if (!aligned_to(a.A, 16) || !aligned_to(a.B, 16)) return false;
    if (b_kn && (a.NB % 8 || a.NB < 8 || a.NB < a.N)) return false;
    if (a.bias && a.bias_mode == MI_BIAS_COL && !aligned_to(a.bias, 8)) return false;
    return a.M >= 1 && a.N >= 1 && a.K >= 8;
}

template <int BM, int BN, int WM, int WN>
int launch_pipe(GemmArgs a, bool b_kn, int64_t nbatch, hipStream_t st) {
    // the kernel always walks at least two 64-deep tiles (its prologue fetches two ahead): one tile would read past K
    if (a.K < 128 || a.K % 64) return MI_DECLINE_EXTENT;
    a.tiles_m = (int)ceil_div(a.M, BM);
    a.tiles_n = (int)ceil_div(a.N, BN);
    a.group_m = a.tiles_m < 6 ? a.tiles_m : 6;
    a.vec_store = a.out_f32 ? (a.ldY % 4 == 0 && a.sY % 4 == 0 && aligned_to(a.Y, 16))
                            : (a.ldY % 8 == 0 && a.sY % 8 == 0 && aligned_to(a.Y, 16) && (!a.residual || aligned_to(a.residual, 16)));
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)nbatch);
    constexpr int lds = gemm_lds_bytes<BM, BN, 64>();
    if (a.ag.x) {
        if (a.cv.xp) return MI_DECLINE_UNSUPPORTED;
        if (b_kn) hipLaunchKernelGGL((gemm_pipe_kernel<BM, BN, WM, WN, 1, 1>), grid, dim3(WM * WN * 64), lds, st, a);
        else      hipLaunchKernelGGL((gemm_pipe_kernel<BM, BN, WM, WN, 0, 1>), grid, dim3(WM * WN * 64), lds, st, a);
    }
    else if (a.cv.xp)   hipLaunchKernelGGL((gemm_pipe_kernel<BM, BN, WM, WN, 2>), grid, dim3(WM * WN * 64), lds, st, a);
    else if (b_kn) hipLaunchKernelGGL((gemm_pipe_kernel<BM, BN, WM, WN, 1>), grid, dim3(WM * WN * 64), lds, st, a);
    else           hipLaunchKernelGGL((gemm_pipe_kernel<BM, BN, WM, WN, 0>), grid, dim3(WM * WN * 64), lds, st, a);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

// The pipelined kernel with the layer norm of A's rows as its prologue (AMODE 2): 64-row tiles, 128 <= K <= 512.
constexpr int LNA_KMAX = 512;
template <int BN, int WM, int WN>
constexpr int lna_lds_bytes(int K) {
    constexpr int kc = BN * (64 + 8), kn = 64 * (BN + 32);
    return (64 * (K + 8) + 2 * (kc > kn ? kc : kn)) * 2;
}
template <int BN, int WM, int WN>
int launch_pipe_ln(GemmArgs a, bool b_kn, hipStream_t st) {
    if (a.K < 128 || a.K % 64 || a.K > LNA_KMAX || a.cv.xp || a.ag.x) return MI_DECLINE_EXTENT;
    a.tiles_m = (int)ceil_div(a.M, 64);
    a.tiles_n = (int)ceil_div(a.N, BN);
    a.group_m = a.tiles_m < 6 ? a.tiles_m : 6;
    a.vec_store = a.out_f32 ? (a.ldY % 4 == 0 && a.sY % 4 == 0 && aligned_to(a.Y, 16))
                            : (a.ldY % 8 == 0 && a.sY % 8 == 0 && aligned_to(a.Y, 16) && (!a.residual || aligned_to(a.residual, 16)));
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n), 1);
    const int lds = lna_lds_bytes<BN, WM, WN>(a.K);
    if (b_kn) hipLaunchKernelGGL((gemm_pipe_kernel<64, BN, WM, WN, 1, 2>), grid, dim3(WM * WN * 64), lds, st, a);
    else      hipLaunchKernelGGL((gemm_pipe_kernel<64, BN, WM, WN, 0, 2>), grid, dim3(WM * WN * 64), lds, st, a);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

template <int BM, int BN, int WM, int WN>
int launch_w4(GemmArgs a, bool b_kn, int64_t nbatch, hipStream_t st) {
    if (a.K < 64 || a.K % 64 || a.cv.xp || a.ag.x) return MI_DECLINE_EXTENT;
    a.tiles_m = (int)ceil_div(a.M, BM);
    a.tiles_n = (int)ceil_div(a.N, BN);
    a.group_m = a.tiles_m < 6 ? a.tiles_m : 6;
    a.vec_store = a.out_f32 ? (a.ldY % 4 == 0 && a.sY % 4 == 0 && aligned_to(a.Y, 16))
                            : (a.ldY % 8 == 0 && a.sY % 8 == 0 && aligned_to(a.Y, 16) && (!a.residual || aligned_to(a.residual, 16)));
    // per-lane load offsets are 32-bit byte offsets from the tile origin
    if ((int64_t)BM * a.ldA * 2 >= (1ll << 31) || (int64_t)(b_kn ? 64 : BN) * a.ldB * 2 >= (1ll << 31)) return MI_DECLINE_EXTENT;
    a.clk = g_clock_probe;
    a.phase = g_phase_probe; a.phase_wgs = g_phase_wgs;
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)nbatch);
    constexpr int lds = w4_lds_bytes<BM, BN>();
    // four matrix waves and the loader, plus the statistics wave of a folded layer norm; eight waves when the four that
    // do not multiply can help with the store
    const dim3 block(coop_store_applies(a) ? 512 : a.lnf_stats ? 384 : 320);
    if (b_kn) hipLaunchKernelGGL((gemm_w4_kernel<BM, BN, WM, WN, true>), grid, block, lds, st, a);
    else      hipLaunchKernelGGL((gemm_w4_kernel<BM, BN, WM, WN, false>), grid, block, lds, st, a);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

bool sk_fits(int64_t M, int64_t N, int64_t K, int bm, int bn, int split);

// The four-wave kernel with two workgroups per 128 x 128 tile exchanging their partial tiles.
int launch_w4_peer(GemmArgs a, bool b_kn, int split, void *ws, hipStream_t st) {
    constexpr int BM = 128, BN = 128;
    if (a.cv.xp || a.ag.x || split != 2 || !sk_usable() || !sk_fits(a.M, a.N, a.K, BM, BN, split)) return MI_DECLINE_EXTENT;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MI_ERROR_DEVICE;
    a.tiles_m = (int)ceil_div(a.M, BM);
    a.tiles_n = (int)ceil_div(a.N, BN);
    a.group_m = 1;
    while (a.group_m * a.group_m < (int)ceil_div((int64_t)a.tiles_m * a.tiles_n, 8) && a.group_m < a.tiles_m) a.group_m++;
    a.vec_store = a.out_f32 ? (a.ldY % 4 == 0 && a.sY % 4 == 0 && aligned_to(a.Y, 16))
                            : (a.ldY % 8 == 0 && a.sY % 8 == 0 && aligned_to(a.Y, 16) && (!a.residual || aligned_to(a.residual, 16)));
    if ((int64_t)BM * a.ldA * 2 >= (1ll << 31) || (int64_t)(b_kn ? 64 : BN) * a.ldB * 2 >= (1ll << 31)) return MI_DECLINE_EXTENT;
    const int tiles = a.tiles_m * a.tiles_n;
    a.sk_S = split;
    a.sk_tpx = (int)ceil_div(tiles, 8);
    a.sk_part = reinterpret_cast<float *>(ws);
    const unsigned launch = ++g_sk_epoch;
    a.sk_epoch = sk::epoch_of(launch);
    a.sk_flags = g_sk_flags_ptr[dev] + (size_t)(launch % SK_BANKS) * SK_FLAGS;
    a.sk_spin = g_sk_spin; a.sk_pub_xor = g_sk_pub_xor; a.sk_xcc_xor = g_sk_xcc_xor;
    a.status = g_status_ptr[dev];
    a.clk = g_clock_probe;
    a.phase = g_phase_probe; a.phase_wgs = g_phase_wgs;
    dim3 grid((unsigned)(8 * a.sk_tpx * split), 1);
    constexpr int lds = w4_lds_bytes<BM, BN>();
    if (b_kn) hipLaunchKernelGGL((gemm_w4_kernel<BM, BN, 2, 2, true, true>), grid, dim3(320), lds, st, a);
    else      hipLaunchKernelGGL((gemm_w4_kernel<BM, BN, 2, 2, false, true>), grid, dim3(320), lds, st, a);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

// tile: index into TILE_MODELS.  The four-wave kernel takes ordinary operands only; a gathered operand (implicit-GEMM
// convolution) planned onto one of its tiles runs the pipelined kernel's same tile instead: same K order per
// output, same bits, and the plan (hence the workspace) stays a function of the extents alone.
int launch_tile(int tile, const GemmArgs &a, bool b_kn, int64_t nbatch, hipStream_t st) {
    const bool plain = !a.cv.xp && !a.ag.x;
    switch (tile) {
        case 0: return plain ? launch_w4<128, 256, 1, 4>(a, b_kn, nbatch, st) : launch_pipe<128, 256, 2, 4>(a, b_kn, nbatch, st);
        case 1: return plain ? launch_w4<192, 128, 2, 2>(a, b_kn, nbatch, st) : launch_pipe<192, 128, 2, 4>(a, b_kn, nbatch, st);
        case 2: return launch_pipe<128, 128, 2, 4>(a, b_kn, nbatch, st);
        case 3: return launch_pipe<64, 128, 2, 4>(a, b_kn, nbatch, st);
        default: return launch_pipe<64, 64, 2, 2>(a, b_kn, nbatch, st);
    }
}

template <int BM, int BN, int BK, int WM, int WN>
int launch_mfma(GemmArgs a, bool b_kn, int64_t nbatch, hipStream_t st) {
    a.tiles_m = (int)ceil_div(a.M, BM);
    a.tiles_n = (int)ceil_div(a.N, BN);
    a.group_m = a.tiles_m < 6 ? a.tiles_m : 6;
    a.vec_store = a.out_f32 ? (a.ldY % 4 == 0 && a.sY % 4 == 0 && aligned_to(a.Y, 16))
                            : (a.ldY % 8 == 0 && a.sY % 8 == 0 && aligned_to(a.Y, 16) && (!a.residual || aligned_to(a.residual, 16)));
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)nbatch);
    constexpr int lds = gemm_lds_bytes<BM, BN, BK>();
    if (b_kn) hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, BK, WM, WN, true>), grid, dim3(WM * WN * 64), lds, st, a);
    else      hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, BK, WM, WN, false>), grid, dim3(WM * WN * 64), lds, st, a);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

// Tile and K-split of a pipelined GEMM, chosen by estimated time.  The five tilings of gemm_pipe_kernel were timed
// on an MI355X over 400 shapes (M 64..8192, N 64..5120, K 128..5120), each unsplit and in 2, 4 and 8 K-slices; per
// tiling the time is launch + prologue/store + (K / 64) steps, and a step costs step_lo when few workgroups run, rises
// linearly to step_full when every CU holds one (clock and memory give way under load), and beyond that grows with
// the number of rounds of CUs-many workgroups (by `round`, below 1 where co-resident workgroups overlap).  A split adds
// the second launch (about 4 us) and the fp32 planes (0.25 us per MB).  Picking the cheapest estimate lands within
// 1 % of the best measured choice on average over those shapes and within 6 % on 95 % of them.
struct TileModel { int bm, bn; double step_lo, step_full, round, fixed; };
constexpr int NTILES = 5;
constexpr TileModel TILE_MODELS[NTILES] = {
    // (the two tiles of the four-wave kernel, re-timed with it: 1500 x 5120 in 25.3 / 70.5 us at K = 1280 / 5120,
    // 512 x 1280 in 16.3 / 47.2; 1500 x 3840 on 192 x 128 in 20.2 / 55.4, 512 x 1280 in 13.5 / 39.9)
    {128, 256, 0.520, 0.760, 1.06, 7.0},
    {192, 128, 0.420, 0.585, 1.00, 6.0},
    {128, 128, 0.428, 0.600, 1.00, 4.0},
    {64, 128, 0.318, 0.430, 0.90, 3.1},
    {64, 64, 0.235, 0.315, 0.73, 3.0},
};
struct TilePlan { int tile, split; bool peer; };      // peer: the K-slices exchange partial tiles in the kernel (no planes)

double tile_cost_us(int64_t M, int64_t N, int64_t K, int64_t nbatch, int tile, int split) {
    const TileModel &t = TILE_MODELS[tile];
    const double cus = (double)mi_num_cus();
    const int64_t wg = ceil_div(M, t.bm) * ceil_div(N, t.bn) * nbatch * split;
    const int64_t rounds = ceil_div(wg, (int64_t)mi_num_cus());
    const double load = wg < mi_num_cus() ? (double)wg / cus : 1.0;
    const double step = wg <= mi_num_cus() ? t.step_lo + (t.step_full - t.step_lo) * load : t.step_full * t.round * (double)rounds;
    double us = 2.0 + (t.fixed - 2.0) * (1.0 + 0.8 * (double)(rounds - 1)) + (t.fixed - 2.0) * 0.4 * load + (double)(K / (64 * split)) * step;
    if (split > 1) us += 4.0 + 0.25 * (double)split * (double)M * (double)N * 4.0 / 1e6;
    return us;
}

// Split-K with the partials exchanged inside the launch (four-wave kernel, 128 x 128 tiles in two K-slices, every
// workgroup resident at once): the tile's own estimate at that many workgroups, no planes and no second launch, plus
// the exchange.  A workgroup writes and reads half of its accumulators; what that costs is set by how fast the burst
// drains -- 7.7 MB from 120 or 240 workgroups take 2 to 3 us end to end.
constexpr int SK_TILE = 2;               // index into TILE_MODELS: 128 x 128
double sk_exchange_us(int64_t wg, int bm, int bn) {
    const double mb = (double)wg * bm * bn * 4.0 * 0.5 / 1e6;
    return 2.0 + 0.3 * mb;               // fitted: 29.8 us measured on 1500 x 5120 -> 1280, 22.1 on 512 x 5120 -> 1280
}
size_t sk_workspace_bytes(int64_t M, int64_t N, int bm, int bn, int split) { return (size_t)(ceil_div(M, bm) * ceil_div(N, bn)) * split * bm * bn * 4; }
bool sk_fits(int64_t M, int64_t N, int64_t K, int bm, int bn, int split) {
    const int64_t tiles = ceil_div(M, bm) * ceil_div(N, bn), tpx = ceil_div(tiles, 8);
    return split == 2 && bm == 128 && bn == 128 && K % 128 == 0 && K / 2 >= 128 && 8 * tpx * 2 <= mi_num_cus() && 8 * tpx * 2 * 8 <= SK_FLAGS;
}
// Before mi_init (planner queries without a device) the path is assumed: a workspace sized for it also holds the planes
// the same split falls back to.
bool sk_planned() {
    int dev = -1;
    if (!g_sk_enabled.load()) return false;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return true;
    return g_sk_state[dev] != -1;
}
double sk_cost_us(int64_t M, int64_t N, int64_t K, int tile, int split) {
    const TileModel &t = TILE_MODELS[tile];
    const int64_t wg = ceil_div(M, t.bm) * ceil_div(N, t.bn) * split;
    const double load = (double)wg / (double)mi_num_cus();
    const double step = t.step_lo + (t.step_full - t.step_lo) * load;
    return 2.0 + (t.fixed - 2.0) * (0.4 + 0.6 / (double)split) + (t.fixed - 2.0) * 0.4 * load + (double)(K / (64 * split)) * step +
           sk_exchange_us(wg, t.bm, t.bn);
}

// The plan depends on the extents alone, so a GEMM gives the same bits whichever entry point issues it.
TilePlan plan_tiles(int64_t M, int64_t N, int64_t K, int64_t nbatch, bool may_split) {
    TilePlan best = {4, 1, false};
    double best_us = 1e30;
    const int max_split = (may_split && nbatch == 1 && M > 8 && N % 4 == 0 && K % 64 == 0) ? 8 : 1;
    for (int split = 1; split <= max_split; split++) {
        if (K % (64 * split) != 0 || (split > 1 && K / split < 128)) continue;
        for (int tile = 0; tile < NTILES; tile++) {
            const double us = tile_cost_us(M, N, K, nbatch, tile, split);
            if (us < best_us) { best_us = us; best = {tile, split, false}; }
        }
        if (max_split > 1 && sk_planned()) {
            if (sk_fits(M, N, K, TILE_MODELS[SK_TILE].bm, TILE_MODELS[SK_TILE].bn, split)) {
                const double us = sk_cost_us(M, N, K, SK_TILE, split);
                if (us < best_us) { best_us = us; best = {SK_TILE, split, true}; }
            }
        }
    }
    return best;
}

// Workspace of a planned split: the planes, or the exchanged partials of the peer reduction (never less than the planes,
// so a launch that cannot take the peer path -- a gathered operand -- falls back to planes in the same workspace).
size_t plan_workspace_bytes(const TilePlan &tp, int64_t M, int64_t N) {
    if (tp.split <= 1) return 0;
    return round_up(tp.peer ? sk_workspace_bytes(M, N, TILE_MODELS[tp.tile].bm, TILE_MODELS[tp.tile].bn, tp.split) : (size_t)tp.split * M * N * sizeof(float), 256);
}

int gemm_path(const GemmArgs &a, bool b_kn, int64_t nbatch) {
    if (a.M < 1 || a.N < 1 || a.K < 1) return MI_GEMM_DECLINE;
    bool addr = mfma_addressable(a, b_kn);
    if (a.M <= 8 && nbatch == 1 && addr && (b_kn || (size_t)8 * a.K * sizeof(half_t) <= SKINNY_FK_LDS_MAX)) return MI_GEMM_SKINNY;
    if (addr && tl_plan_mfma) return MI_GEMM_MFMA;
    return MI_GEMM_SCALAR;
}

int run_skinny(GemmArgs a, bool b_kn, void *ws, size_t ws_bytes, hipStream_t st) {
    if (b_kn) {
        const int kper = skinny_kper(a.K, a.N), nsplit = (int)ceil_div(a.K, kper);
        size_t need = (size_t)nsplit * a.M * a.N * sizeof(float);
        if (!ws || ws_bytes < need || !aligned_to(ws, 256)) return MI_DECLINE_WORKSPACE;
        float *part = reinterpret_cast<float *>(ws);
        dim3 grid((unsigned)ceil_div(a.N, SKN_COLS), (unsigned)nsplit);
        if (a.M <= 1)      hipLaunchKernelGGL(skinny_kn_kernel<1>, grid, dim3(256), 0, st, a, part, kper);
        else if (a.M <= 2) hipLaunchKernelGGL(skinny_kn_kernel<2>, grid, dim3(256), 0, st, a, part, kper);
        else if (a.M <= 4) hipLaunchKernelGGL(skinny_kn_kernel<4>, grid, dim3(256), 0, st, a, part, kper);
        else if (a.M <= 8) hipLaunchKernelGGL(skinny_kn_kernel<8>, grid, dim3(256), 0, st, a, part, kper);
        else return MI_DECLINE_EXTENT;
        long total = (long)a.M * a.N;
        hipLaunchKernelGGL(skinny_epilogue_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, a, part, nsplit);
    } else {
        const int mt = a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : 8;
        const size_t lds = (size_t)mt * a.K * sizeof(half_t);
        if (a.M > 8 || lds > SKINNY_FK_LDS_MAX) return MI_DECLINE_EXTENT;
        // rows per wave: as many as still leave every CU a workgroup, at most eight (a workgroup stages
        // all M activation rows once, whatever the number of weight rows it then streams)
        // One weight row per wave.  More rows per wave would amortise the staging of the activations, but the
        // rows of a wave run one after the other, each a chain of dependent memory trips: measured slower at
        // every batch size (1280 -> 5120, batch 8: 9.1 us with one row, 13.7 us with four).
        // One or two rows without a norm in front: activations in registers, no staging (hot in a replayed graph at
        // batch 1: 2.88 / 3.13 / 3.34 us for 1280 -> 1280 / 3840 / 5120 against 3.01 / 3.33 / 3.57 us staged).  With
        // the layer-norm prologue every wave would normalise its own copy of the row -- 4.5 / 6.1 / 6.9 us against
        // 3.9 / 4.3 / 4.7 us -- so that stays staged, and so does a very wide output (51866 columns: 24.5 against 23.0 us).
        int R = 1;
        if (!a.ln_on && a.N <= 8192 && a.K <= 1536 && mt <= 2) {
            dim3 rg((unsigned)ceil_div(a.N, 4 * R));
            if (R == 2) {
                if (mt == 1)      hipLaunchKernelGGL((skinny_fk_reg_kernel<1, 3, 2>), rg, dim3(256), 0, st, a);
                else              hipLaunchKernelGGL((skinny_fk_reg_kernel<2, 3, 2>), rg, dim3(256), 0, st, a);
            } else {
                if (mt == 1)      hipLaunchKernelGGL((skinny_fk_reg_kernel<1, 3, 1>), rg, dim3(256), 0, st, a);
                else              hipLaunchKernelGGL((skinny_fk_reg_kernel<2, 3, 1>), rg, dim3(256), 0, st, a);
            }
            return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
        }
        // every column its own wave up to eight workgroups per CU; beyond that (a vocabulary projection) a wave walks
        // several columns behind one staging of the activations
        const int64_t wgs = ceil_div(a.N, 4), cap = (int64_t)mi_num_cus() * 8;
        dim3 grid((unsigned)(wgs < cap ? wgs : cap));
        if (a.K <= 1536) {
            if (mt == 1)      hipLaunchKernelGGL((skinny_fk_kernel<1, 3>), grid, dim3(256), lds, st, a);
            else if (mt == 2) hipLaunchKernelGGL((skinny_fk_kernel<2, 3>), grid, dim3(256), lds, st, a);
            else if (mt == 4) hipLaunchKernelGGL((skinny_fk_kernel<4, 3>), grid, dim3(256), lds, st, a);
            else              hipLaunchKernelGGL((skinny_fk_kernel<8, 3>), grid, dim3(256), lds, st, a);
        } else {
            if (mt == 1)      hipLaunchKernelGGL((skinny_fk_kernel<1, 12>), grid, dim3(256), lds, st, a);
            else if (mt == 2) hipLaunchKernelGGL((skinny_fk_kernel<2, 12>), grid, dim3(256), lds, st, a);
            else if (mt == 4) hipLaunchKernelGGL((skinny_fk_kernel<4, 12>), grid, dim3(256), lds, st, a);
            else              hipLaunchKernelGGL((skinny_fk_kernel<8, 12>), grid, dim3(256), lds, st, a);
        }
    }
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int fill_args(GemmArgs &a, void *Y, const void *X, const void *W, const void *bias, const void *residual,
              int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
              int w_layout, int bias_mode, int epi, int out_dtype, int64_t sY, int64_t sX, int64_t sW, int64_t sBias = 0) {
    if (!Y || !X || !W) return MI_DECLINE_OPERANDS;
    if (T < 0 || K < 0 || F < 0 || T > INT32_MAX || K > INT32_MAX || F > INT32_MAX) return MI_DECLINE_EXTENT;
    if (w_layout != MI_W_KF && w_layout != MI_W_FK) return MI_DECLINE_OPERANDS;
    if (out_dtype != MI_F16 && out_dtype != MI_F32) return MI_DECLINE_OPERANDS;
    if (epi < MI_EPI_NONE || epi > MI_EPI_RELU) return MI_DECLINE_UNSUPPORTED;
    if (bias_mode < MI_BIAS_NONE || bias_mode > MI_BIAS_ROW) return MI_DECLINE_BIAS;
    if (bias_mode != MI_BIAS_NONE && !bias) return MI_DECLINE_BIAS;
    if (residual && out_dtype != MI_F16) return MI_DECLINE_UNSUPPORTED;
    if (ldX < K || ldY < F || ldW < (w_layout == MI_W_KF ? F : K)) return MI_DECLINE_EXTENT;
    a.Y = Y; a.A = (const half_t *)X; a.B = (const half_t *)W;
    a.bias = bias_mode == MI_BIAS_NONE ? nullptr : (const half_t *)bias;
    a.residual = (const half_t *)residual;
    a.M = (int)T; a.N = (int)F; a.K = (int)K; a.NB = (int)F;
    a.ldY = ldY; a.ldA = ldX; a.ldB = ldW; a.sY = sY; a.sA = sX; a.sB = sW; a.sBias = sBias;
    a.bias_mode = bias_mode; a.epi = epi; a.out_f32 = out_dtype == MI_F32;
    a.tiles_m = a.tiles_n = a.group_m = 1; a.vec_store = 0;
    a.cv = ConvGather{};
    a.ag = NhwcGather{};
    a.ln_gamma = a.ln_beta = nullptr; a.ln_eps = 0.0f; a.ln_on = 0;
    a.lnout = nullptr; a.lnout_gamma = a.lnout_beta = nullptr; a.lnout_eps = 0.0f; a.clamp = 0.0f;
    a.clk = nullptr; a.phase = nullptr; a.phase_wgs = 0;
    a.sk_S = 0; a.sk_tpx = 0; a.sk_part = nullptr; a.sk_flags = nullptr; a.sk_epoch = 0;
    a.sk_spin = 0; a.sk_pub_xor = a.sk_xcc_xor = 0; a.status = nullptr;
    a.lnf_stats = a.lnf_colsum = a.lnf_biasp = nullptr; a.lnf_svec = 0; a.lnf_nseg = 0; a.lnf_eps = 0.0f; a.stats_out = nullptr; a.stats_nseg = 0;
    return MI_OK;
}

// Internal status: the split-K epilogue has also written a.lnout (the caller must not run the norm again).
constexpr int MI_LNOUT_DONE = -1;

bool lnout_rowwise_ok(const GemmArgs &a) {
    return !a.out_f32 && a.N % 8 == 0 && a.N <= 4096 && a.ldY % 8 == 0 && aligned_to(a.Y, 16) && aligned_to(a.lnout, 16) &&
           (!a.residual || aligned_to(a.residual, 16)) && (!a.lnout_gamma || aligned_to(a.lnout_gamma, 16)) &&
           (!a.lnout_beta || aligned_to(a.lnout_beta, 16));
}

int run_gemm(GemmArgs a, bool b_kn, int64_t nbatch, void *ws, size_t ws_bytes, hipStream_t st, int force_path) {
    if (!g_ready) return MI_ERROR_DEVICE;
    if (a.M == 0 || a.N == 0 || nbatch == 0) return MI_OK;
    int path = force_path ? force_path : gemm_path(a, b_kn, nbatch);
    if (path == MI_GEMM_DECLINE) return MI_DECLINE_EXTENT;
    if (path == MI_GEMM_SKINNY) return run_skinny(a, b_kn, ws, ws_bytes, st);
    if (path == MI_GEMM_MFMA) {
        if (!mfma_addressable(a, b_kn)) return MI_DECLINE_OPERANDS;
        // Split K over workgroups when the output alone cannot fill the chip: each K-slice is one plane
        // of a batched launch (plane strides: A advances along k, Y one fp32 M x N plane in ws), and a
        // second small kernel sums the planes and applies bias, activation and residual.
        const bool pipe = a.K % 64 == 0 && a.K >= 128;
        if ((a.cv.xp || a.ag.x) && !pipe) return MI_DECLINE_EXTENT;      // only the pipelined kernel gathers
        TilePlan tp = {4, 1, false};
        // A folded norm on the way in or row statistics on the way out live in the tiled kernels' own store: those calls
        // need the pipelined kernels, 16-byte rows, and K-slices only in the form that ends in that store (the in-launch
        // exchange), never planes.
        const bool in_store = a.lnf_stats || a.stats_out;
        if (in_store) {
            const bool rows16 = !a.out_f32 ? (a.N % 8 == 0 && a.ldY % 8 == 0 && a.sY % 8 == 0 && aligned_to(a.Y, 16) && (!a.residual || aligned_to(a.residual, 16)))
                                           : (a.N % 4 == 0 && a.ldY % 4 == 0 && a.sY % 4 == 0 && aligned_to(a.Y, 16));
            if (!pipe || a.cv.xp || a.ag.x || !rows16 || (a.stats_out && a.out_f32)) return MI_DECLINE_EXTENT;
        }
        if (pipe) {
            tp = plan_tiles(a.M, a.N, a.K, nbatch, !a.lnf_stats);
            if (tp.split > 1 && !(ws && aligned_to(ws, 256) && ws_bytes >= plan_workspace_bytes(tp, a.M, a.N)))
                tp = plan_tiles(a.M, a.N, a.K, nbatch, false);
            if (in_store && tp.split > 1 && !(tp.peer && sk_usable())) tp = plan_tiles(a.M, a.N, a.K, nbatch, false);
        }
        int split = tp.split;
        if (split > 1 && tp.peer && ws && aligned_to(ws, 256) && ws_bytes >= plan_workspace_bytes(tp, a.M, a.N)) {
            const int rc = launch_w4_peer(a, b_kn, split, ws, st);
            if (rc != MI_DECLINE_EXTENT) return rc;     // declined (a gathered operand, a device that failed the probe): planes
            if (in_store) { tp = plan_tiles(a.M, a.N, a.K, nbatch, false); split = 1; }
        }
        if (split > 1 && ws && aligned_to(ws, 256) && ws_bytes >= (size_t)split * a.M * a.N * sizeof(float)) {
            GemmArgs s1 = a;
            s1.Y = ws; s1.out_f32 = 1; s1.bias = nullptr; s1.bias_mode = MI_BIAS_NONE; s1.epi = MI_EPI_NONE; s1.residual = nullptr; s1.clamp = 0.0f;
            s1.ldY = a.N; s1.sY = (long)a.M * a.N;
            s1.K = a.K / split;
            s1.sA = s1.K; s1.sB = b_kn ? (long)s1.K * a.ldB : s1.K; s1.sBias = 0;
            s1.cv.split = 1;
            s1.ag.split = 1;
            int rc = launch_tile(tp.tile, s1, b_kn, split, st);
            if (rc != MI_OK) return rc;
            GemmArgs s2 = a;
            s2.vec_store = !a.out_f32 && a.ldY % 4 == 0 && aligned_to(a.Y, 8);
            const float *planes = reinterpret_cast<const float *>(ws);
            if (a.lnout && lnout_rowwise_ok(a)) {
                // the norm of the finished rows rides in the pass that sums the planes: one wave per row
                dim3 grid((unsigned)ceil_div(a.M, 4));
                if (a.N <= 512)       hipLaunchKernelGGL(splitk_epilogue_ln_kernel<1>, grid, dim3(256), 0, st, s2, planes, split);
                else if (a.N <= 1024) hipLaunchKernelGGL(splitk_epilogue_ln_kernel<2>, grid, dim3(256), 0, st, s2, planes, split);
                else if (a.N <= 2048) hipLaunchKernelGGL(splitk_epilogue_ln_kernel<4>, grid, dim3(256), 0, st, s2, planes, split);
                else                  hipLaunchKernelGGL(splitk_epilogue_ln_kernel<8>, grid, dim3(256), 0, st, s2, planes, split);
                return hipGetLastError() == hipSuccess ? MI_LNOUT_DONE : MI_ERROR_LAUNCH;
            }
            const long quads = ((long)a.M * a.N) / 4;
            hipLaunchKernelGGL(splitk_epilogue_kernel, dim3((unsigned)ceil_div(quads, 256)), dim3(256), 0, st, s2, planes, split);
            return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
        }
        if (pipe) return launch_tile(tp.tile, a, b_kn, nbatch, st);
        // K not a multiple of 64 (or a single tile deep): the unpipelined kernel, big tiles as soon as they cover half the CUs
        const int64_t big = ceil_div(a.M, 128) * ceil_div(a.N, 256) * nbatch;
        const int64_t mid = ceil_div(a.M, 128) * ceil_div(a.N, 128) * nbatch;
        if (big * 2 > mi_num_cus()) return launch_mfma<GEMM_BIG>(a, b_kn, nbatch, st);
        if (mid >= (mi_num_cus() * 3) / 8) return launch_mfma<GEMM_MID>(a, b_kn, nbatch, st);
        return launch_mfma<GEMM_SMALL>(a, b_kn, nbatch, st);
    }
    long total = (long)a.M * a.N;
    hipLaunchKernelGGL(gemm_scalar_kernel, dim3((unsigned)ceil_div(total, 256), (unsigned)nbatch), dim3(256), 0, st, a, b_kn ? 1 : 0);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

}  // namespace

bool mi_ready() { return g_ready; }
int mi_num_cus() { return tl_plan_cus > 0 ? tl_plan_cus : g_cus; }
bool mi_plan_mfma() { return tl_plan_mfma; }
void mi_plan_caps_begin(const int64_t *caps) {
    if (!caps) return;
    tl_plan_mfma = caps[0] != 0;
    tl_plan_cus = caps[5] > 0 ? (int)(caps[5] > 65536 ? 65536 : caps[5]) : 1;
}
void mi_plan_caps_end() { tl_plan_cus = 0; tl_plan_mfma = true; }
bool mi_xcd_round_robin() { return sk_usable(); }

// Split-K planes of a GEMM issued through mi_internal_gemm.
size_t mi_internal_gemm_workspace(int64_t T, int64_t K, int64_t F, int64_t nbatch) {
    if (T <= 8) return mi_gemm_f16_workspace(T, K, F, MI_W_KF, nbatch);      // decode-sized: the [K][F] kernel's planes
    if (nbatch > 1 || K % 64 || K < 128) return 0;
    return plan_workspace_bytes(plan_tiles(T, F, K, 1, true), T, F);
}

// Internal entry used by the convolution path (conv.hip): Y[M x N] = A . B with
// every GemmArgs field meaningful.
int mi_internal_gemm(void *Y, const void *A, const void *B, const void *bias, int M, int N, int NB, int K,
                     long ldY, long ldA, long ldB, int b_kn, int bias_mode, int epi, int out_f32,
                     long nbatch, long sY, long sA, long sB, void *ws, size_t ws_bytes, hipStream_t st,
                     const ConvGather *gather, const NhwcGather *agather, const void *residual) {
    GemmArgs a;
    a.cv = ConvGather{};
    a.ag = NhwcGather{};
    a.ln_gamma = a.ln_beta = nullptr; a.ln_eps = 0.0f; a.ln_on = 0;
    a.lnout = nullptr; a.lnout_gamma = a.lnout_beta = nullptr; a.lnout_eps = 0.0f; a.clamp = 0.0f;
    a.clk = nullptr; a.phase = nullptr; a.phase_wgs = 0;
    a.sk_S = 0; a.sk_tpx = 0; a.sk_part = nullptr; a.sk_flags = nullptr; a.sk_epoch = 0;
    a.sk_spin = 0; a.sk_pub_xor = a.sk_xcc_xor = 0; a.status = nullptr;
    a.lnf_stats = a.lnf_colsum = a.lnf_biasp = nullptr; a.lnf_svec = 0; a.lnf_nseg = 0; a.lnf_eps = 0.0f; a.stats_out = nullptr; a.stats_nseg = 0;
    a.Y = Y; a.A = (const half_t *)A; a.B = (const half_t *)B; a.bias = (const half_t *)bias; a.residual = out_f32 ? nullptr : (const half_t *)residual;
    a.M = M; a.N = N; a.NB = NB; a.K = K; a.ldY = ldY; a.ldA = ldA; a.ldB = ldB; a.sY = sY; a.sA = sA; a.sB = sB; a.sBias = 0;
    a.bias_mode = bias ? bias_mode : MI_BIAS_NONE; a.epi = epi; a.out_f32 = out_f32;
    a.tiles_m = a.tiles_n = a.group_m = 1; a.vec_store = 0;
    if (gather) a.cv = *gather;
    if (agather) a.ag = *agather;
    const bool addr = mfma_addressable(a, b_kn != 0);
    if ((gather || agather) && !addr) return MI_DECLINE_OPERANDS;
    int path = addr ? MI_GEMM_MFMA : MI_GEMM_SCALAR;
    return run_gemm(a, b_kn != 0, nbatch, ws, ws_bytes, st, path);
}

extern "C" {

int mi_version(void) { return MI355DNN_VERSION; }

int mi_init(void) {
    if (g_ready) return MI_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MI_ERROR_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return MI_ERROR_DEVICE;
    if (__builtin_strncmp(prop.gcnArchName, "gfx950", 6) != 0) return MI_ERROR_DEVICE;
    g_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    int bad = 0;
    bad |= raise_lds(gemm_mfma_kernel<GEMM_BIG, true>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_mfma_kernel<GEMM_BIG, false>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_mfma_kernel<GEMM_MID, true>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_mfma_kernel<GEMM_MID, false>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_mfma_kernel<GEMM_SMALL, true>, gemm_lds_bytes<64, 64, 64>());
    bad |= raise_lds(gemm_mfma_kernel<GEMM_SMALL, false>, gemm_lds_bytes<64, 64, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 256, 2, 4, true>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 256, 2, 4, false>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 128, 2, 4, true>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 128, 2, 4, false>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<64, 128, 2, 4, 1>, gemm_lds_bytes<64, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<64, 128, 2, 4, 0>, gemm_lds_bytes<64, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<192, 128, 2, 4, 1>, gemm_lds_bytes<192, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<192, 128, 2, 4, 0>, gemm_lds_bytes<192, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<192, 128, 2, 4, 2>, gemm_lds_bytes<192, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<192, 128, 2, 4, 0, 1>, gemm_lds_bytes<192, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<192, 128, 2, 4, 1, 1>, gemm_lds_bytes<192, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 256, 2, 4, 2>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 256, 2, 4, 0, 1>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 256, 2, 4, 1, 1>, gemm_lds_bytes<128, 256, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 128, 2, 4, 0, 1>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 128, 2, 4, 1, 1>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_pipe_kernel<128, 128, 2, 4, 2>, gemm_lds_bytes<128, 128, 64>());
    bad |= raise_lds(gemm_w4_kernel<128, 256, 1, 4, true>, w4_lds_bytes<128, 256>());
    bad |= raise_lds(gemm_w4_kernel<128, 256, 1, 4, false>, w4_lds_bytes<128, 256>());
    bad |= raise_lds(gemm_w4_kernel<192, 128, 2, 2, true>, w4_lds_bytes<192, 128>());
    bad |= raise_lds(gemm_w4_kernel<192, 128, 2, 2, false>, w4_lds_bytes<192, 128>());
    bad |= raise_lds(gemm_w4_kernel<128, 128, 2, 2, true, true>, w4_lds_bytes<128, 128>());
    bad |= raise_lds(gemm_w4_kernel<128, 128, 2, 2, false, true>, w4_lds_bytes<128, 128>());
    bad |= raise_lds(gemm_pipe_kernel<64, 128, 2, 4, 1, 2>, lna_lds_bytes<128, 2, 4>(LNA_KMAX));
    bad |= raise_lds(gemm_pipe_kernel<64, 128, 2, 4, 0, 2>, lna_lds_bytes<128, 2, 4>(LNA_KMAX));
    bad |= raise_lds(gemm_pipe_kernel<64, 64, 2, 2, 1, 2>, lna_lds_bytes<64, 2, 2>(LNA_KMAX));
    bad |= raise_lds(gemm_pipe_kernel<64, 64, 2, 2, 0, 2>, lna_lds_bytes<64, 2, 2>(LNA_KMAX));
    bad |= raise_lds(skinny_fk_kernel<1, 3>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<2, 3>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<4, 3>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<8, 3>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<1, 12>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<2, 12>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<4, 12>, (int)SKINNY_FK_LDS_MAX);
    bad |= raise_lds(skinny_fk_kernel<8, 12>, (int)SKINNY_FK_LDS_MAX);
    bad |= mi_sdpa_init();
    bad |= scratch_of_current_device() == nullptr;
    sk_probe_current_device();      // a device that fails the probe only loses that path
    if (bad) return MI_ERROR_DEVICE;
    g_ready = true;
    return MI_OK;
}

int mi_set_phase_probe(void *dev_u64, int64_t workgroups) {
    if (workgroups < 0 || workgroups > (1 << 20) || (dev_u64 && !aligned_to(dev_u64, 8))) return MI_DECLINE_OPERANDS;
    g_phase_probe = reinterpret_cast<unsigned long long *>(dev_u64);
    g_phase_wgs = dev_u64 ? (int)workgroups : 0;
    return MI_OK;
}

int mi_set_clock_probe(void *dev_u64x4) {
    if (dev_u64x4 && !aligned_to(dev_u64x4, 8)) return MI_DECLINE_OPERANDS;
    g_clock_probe = reinterpret_cast<unsigned long long *>(dev_u64x4);
    return MI_OK;
}

int mi_device_status(int reset) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES || !g_status_ptr[dev]) return -1;
    if (hipDeviceSynchronize() != hipSuccess) return -1;
    unsigned word = 0;
    if (hipMemcpy(&word, g_status_ptr[dev], sizeof(word), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    if (reset) {
        // a wave that gave up released nothing: zero every bank of flags and counters along with the word
        bool ok = hipMemset(g_status_ptr[dev], 0, sizeof(unsigned)) == hipSuccess;
        if (g_sk_flags_ptr[dev]) ok = ok && hipMemset(g_sk_flags_ptr[dev], 0, sizeof(unsigned) * 2 * SK_WORDS) == hipSuccess;
        if (!ok || hipDeviceSynchronize() != hipSuccess) return -1;
    }
    return (int)(word & 0x7fffffffu);
}

int mi_set_in_launch_exchange(int enabled) {
    g_sk_enabled.store(enabled != 0);
    return MI_OK;
}

int mi_test_exchange_faults(int spin_limit, unsigned publish_xor, unsigned xcc_xor) {
    g_sk_spin = spin_limit > 0 ? spin_limit : SK_SPIN_DEFAULT;
    g_sk_pub_xor = publish_xor & sk::EPOCH_MASK;
    g_sk_xcc_xor = xcc_xor & 15u;
    return MI_OK;
}

int mi_device_caps(int64_t out[6]) {
    if (!out) return MI_DECLINE_OPERANDS;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return MI_ERROR_DEVICE;
    out[0] = __builtin_strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    out[1] = 16;
    out[2] = prop.warpSize;
    out[3] = (int64_t)prop.maxSharedMemoryPerMultiProcessor;
    out[4] = prop.maxThreadsPerBlock;
    out[5] = prop.multiProcessorCount;
    return MI_OK;
}

size_t mi_gemm_f16_workspace(int64_t T, int64_t K, int64_t F, int w_layout, int64_t nbatch) {
    if (T < 1 || nbatch > 1) return 0;
    if (T > 8) {
        if (K % 64 || K < 128) return 0;
        return plan_workspace_bytes(plan_tiles(T, F, K, 1, true), T, F);
    }
    if (w_layout != MI_W_KF) return 0;      // the [F][K] skinny kernel finishes its outputs itself
    return round_up((size_t)skinny_splits(K, F) * T * F * sizeof(float), 256);
}

int mi_gemm_f16_plan(const void *Y, const void *X, const void *W,
                     int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                     int w_layout, int out_dtype, int64_t nbatch, int64_t sY, int64_t sX, int64_t sW) {
    GemmArgs a;
    int rc = fill_args(a, const_cast<void *>(Y), X, W, nullptr, nullptr, T, K, F, ldY, ldX, ldW, w_layout, MI_BIAS_NONE,
                       MI_EPI_NONE, out_dtype, sY, sX, sW);
    if (rc != MI_OK) return MI_GEMM_DECLINE;
    return gemm_path(a, w_layout == MI_W_KF, nbatch < 1 ? 1 : nbatch);
}

int mi_gemm_f16_plan_caps(const int64_t caps[6], const void *Y, const void *X, const void *W,
                          int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                          int w_layout, int out_dtype, int64_t nbatch, int64_t sY, int64_t sX, int64_t sW, int *ksplit_out) {
    mi_plan_caps_begin(caps);
    const int path = mi_gemm_f16_plan(Y, X, W, T, K, F, ldY, ldX, ldW, w_layout, out_dtype, nbatch, sY, sX, sW);
    if (ksplit_out) {
        *ksplit_out = 1;
        if (path == MI_GEMM_MFMA && K % 64 == 0 && K >= 128) *ksplit_out = plan_tiles(T, F, K, nbatch < 1 ? 1 : nbatch, true).split;
        if (path == MI_GEMM_SKINNY && w_layout == MI_W_KF) *ksplit_out = skinny_splits(K, F);
    }
    mi_plan_caps_end();
    return path;
}

int mi_gemm_f16_batched(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                        int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                        int w_layout, int bias_mode, int epi, int out_dtype,
                        int64_t nbatch, int64_t sY, int64_t sX, int64_t sW, int64_t sBias,
                        void *ws, size_t ws_bytes, void *stream) {
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi, out_dtype, sY, sX, sW, sBias);
    if (rc != MI_OK) return rc;
    if (nbatch < 0 || nbatch > 65535) return MI_DECLINE_EXTENT;
    if (K == 0) return MI_DECLINE_EXTENT;
    return run_gemm(a, w_layout == MI_W_KF, nbatch, ws, ws_bytes, (hipStream_t)stream, 0);
}

int mi_gemm_f16(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                int w_layout, int bias_mode, int epi, int out_dtype,
                void *ws, size_t ws_bytes, void *stream) {
    return mi_gemm_f16_batched(Y, X, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi, out_dtype,
                               1, 0, 0, 0, 0, ws, ws_bytes, stream);
}

int mi_gemm_ln_f16(void *Y, void *H, const void *X, const void *W, const void *bias, const void *residual,
                   const void *gamma, const void *beta, float eps,
                   int64_t T, int64_t K, int64_t F, int64_t ldX, int64_t ldW,
                   int w_layout, int bias_mode, int epi, void *ws, size_t ws_bytes, void *stream) {
    if (!H) return MI_DECLINE_OPERANDS;
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, F, ldX, ldW, w_layout, bias_mode, epi, MI_F16, 0, 0, 0);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    a.lnout = (half_t *)H; a.lnout_gamma = (const half_t *)gamma; a.lnout_beta = (const half_t *)beta; a.lnout_eps = eps;
    rc = run_gemm(a, w_layout == MI_W_KF, 1, ws, ws_bytes, (hipStream_t)stream, 0);
    if (rc == MI_LNOUT_DONE) return MI_OK;
    if (rc != MI_OK) return rc;
    return mi_layernorm_f16(H, nullptr, nullptr, Y, gamma, beta, F, T, eps, stream);      // rows of Y are dense: ldY = F
}

int mi_gemm_clamp_ln_f16(void *Y, void *H, const void *X, const void *W, const void *bias, const void *residual,
                         const void *gamma, const void *beta, float eps, float clamp,
                         int64_t T, int64_t K, int64_t F, int64_t ldX, int64_t ldW,
                         int w_layout, int bias_mode, int epi, void *ws, size_t ws_bytes, void *stream) {
    if (is_nan_arg(clamp) || clamp <= 0.0f) return MI_DECLINE_OPERANDS;
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, F, ldX, ldW, w_layout, bias_mode, epi, MI_F16, 0, 0, 0);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    if (T == 0 || F == 0) return MI_OK;
    const bool b_kn = w_layout == MI_W_KF;
    // the tiled kernels and the plane sums clamp in their stores; the decode-sized and scalar kernels do not: there the
    // clamp is a pass of its own over Y
    const bool in_store = gemm_path(a, b_kn, 1) == MI_GEMM_MFMA;
    if (in_store) a.clamp = clamp;
    if (H) { a.lnout = (half_t *)H; a.lnout_gamma = (const half_t *)gamma; a.lnout_beta = (const half_t *)beta; a.lnout_eps = eps; }
    if (!in_store) a.lnout = nullptr;
    rc = run_gemm(a, b_kn, 1, ws, ws_bytes, (hipStream_t)stream, 0);
    if (rc == MI_LNOUT_DONE) return MI_OK;
    if (rc != MI_OK) return rc;
    if (!in_store) {
        rc = mi_clamp_f16(Y, Y, -clamp, clamp, T * F, stream);
        if (rc != MI_OK) return rc;
    }
    return H ? mi_layernorm_f16(H, nullptr, nullptr, Y, gamma, beta, F, T, eps, stream) : MI_OK;
}

int mi_gemm_rowstats_f16(void *Y, float *stats, const void *X, const void *W, const void *bias, const void *residual, float clamp,
                         int64_t T, int64_t K, int64_t F, int64_t ldX, int64_t ldW,
                         int w_layout, int bias_mode, int epi, void *ws, size_t ws_bytes, void *stream) {
    if (!stats || !aligned_to(stats, 8) || is_nan_arg(clamp)) return MI_DECLINE_OPERANDS;
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, F, ldX, ldW, w_layout, bias_mode, epi, MI_F16, 0, 0, 0);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    if (T == 0 || F == 0) return MI_OK;
    if (gemm_path(a, w_layout == MI_W_KF, 1) != MI_GEMM_MFMA) return MI_DECLINE_EXTENT;
    a.stats_out = stats; a.stats_nseg = (int)ceil_div(F, 32);
    if (clamp > 0.0f) a.clamp = clamp;
    return run_gemm(a, w_layout == MI_W_KF, 1, ws, ws_bytes, (hipStream_t)stream, 0);
}

int mi_lnfold_gemm_f16(void *Y, float *stats_out, const void *X, const float *stats_in, float eps,
                       const void *Wp, const float *colsum, const float *biasp, const void *residual, float clamp,
                       int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                       int w_layout, int epi, int out_dtype,
                       int64_t nbatch, int64_t sY, int64_t sW, int64_t sVec, void *ws, size_t ws_bytes, void *stream) {
    if (!stats_in || !colsum || !biasp || !aligned_to(stats_in, 8) || !aligned_to(colsum, 16) || !aligned_to(biasp, 16) || sVec % 4) return MI_DECLINE_OPERANDS;
    if (is_nan_arg(eps) || is_nan_arg(clamp) || (stats_out && !aligned_to(stats_out, 8))) return MI_DECLINE_OPERANDS;
    if (nbatch < 1 || nbatch > 65535 || (stats_out && (nbatch != 1 || ldY != F || out_dtype != MI_F16))) return MI_DECLINE_EXTENT;
    GemmArgs a;
    int rc = fill_args(a, Y, X, Wp, nullptr, residual, T, K, F, ldY, ldX, ldW, w_layout, MI_BIAS_NONE, epi, out_dtype, sY, 0, sW);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    if (T == 0 || F == 0) return MI_OK;
    if (T <= 8 || !mfma_addressable(a, w_layout == MI_W_KF)) return MI_DECLINE_EXTENT;      // decode-sized rows: mi_ln_gemv_f16
    a.lnf_stats = stats_in; a.lnf_nseg = (int)ceil_div(K, 32); a.lnf_eps = eps;
    a.lnf_colsum = colsum; a.lnf_biasp = biasp; a.lnf_svec = sVec;
    if (stats_out) { a.stats_out = stats_out; a.stats_nseg = (int)ceil_div(F, 32); }
    if (clamp > 0.0f) a.clamp = clamp;
    return run_gemm(a, w_layout == MI_W_KF, nbatch, ws, ws_bytes, (hipStream_t)stream, MI_GEMM_MFMA);
}

// mi_gemm_f16 for callers that cannot allocate: the split-K / decode planes go to `scratch`, a file-scope
// device array, reached through the per-device address that hipGetSymbolAddress returns (the array's name is only a
// host-side stand-in).  The planes are written in full before they are summed, so nothing needs clearing between calls.
int mi_gemm_f16_noalloc(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                        int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                        int w_layout, int bias_mode, int epi, int out_dtype, void *stream) {
    if (!g_ready) return MI_ERROR_DEVICE;
    const size_t need = mi_gemm_f16_workspace(T, K, F, w_layout, 1);
    if (need > (size_t)MI_NOALLOC_SCRATCH_BYTES) return MI_DECLINE_SCRATCH_LIMIT;
    void *planes = nullptr;
    if (need) {
        planes = scratch_of_current_device();
        if (!planes) return MI_ERROR_DEVICE;
    }
    return mi_gemm_f16(Y, X, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi, out_dtype,
                       planes, need ? (size_t)MI_NOALLOC_SCRATCH_BYTES : 0, stream);
}

int mi_gemv_f16(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                int w_layout, int bias_mode, int epi, int out_dtype,
                void *ws, size_t ws_bytes, void *stream) {
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi, out_dtype, 0, 0, 0);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    if (T < 1 || T > 8) return MI_DECLINE_EXTENT;
    if (!mfma_addressable(a, w_layout == MI_W_KF)) return MI_DECLINE_OPERANDS;
    return run_skinny(a, w_layout == MI_W_KF, ws, ws_bytes, (hipStream_t)stream);
}

int mi_ln_gemm_f16(void *Y, const void *X, const void *gamma, const void *beta, float eps,
                   const void *W, const void *bias, const void *residual,
                   int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                   int w_layout, int bias_mode, int epi, int out_dtype,
                   void *ws, size_t ws_bytes, void *stream) {
    if (T >= 1 && T <= 8)
        return mi_ln_gemv_f16(Y, X, gamma, beta, eps, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi,
                              out_dtype, ws, ws_bytes, stream);
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi, out_dtype, 0, 0, 0);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    if (T == 0 || F == 0) return MI_OK;
    const bool b_kn = w_layout == MI_W_KF;
    if (!mfma_addressable(a, b_kn)) return MI_DECLINE_OPERANDS;
    if ((gamma && !aligned_to(gamma, 16)) || (beta && !aligned_to(beta, 16))) return MI_DECLINE_OPERANDS;
    if (K < 128 || K % 64 || K > LNA_KMAX) return MI_DECLINE_EXTENT;      // the caller runs the two ops
    // a shape whose plain GEMM would split K sums in another order: keep the promise of identical bits, decline
    if (plan_tiles(T, F, K, 1, true).split != 1) return MI_DECLINE_EXTENT;
    a.ln_on = 1; a.ln_gamma = (const half_t *)gamma; a.ln_beta = (const half_t *)beta; a.ln_eps = eps;
    // 64-row tiles only (the normalised panel of a workgroup stays in LDS); which width, by the same estimate as
    // every other tiled launch
    const bool wide = tile_cost_us(T, F, K, 1, 3, 1) <= tile_cost_us(T, F, K, 1, 4, 1);
    return wide ? launch_pipe_ln<128, 2, 4>(a, b_kn, (hipStream_t)stream) : launch_pipe_ln<64, 2, 2>(a, b_kn, (hipStream_t)stream);
}

int mi_ln_gemv_f16(void *Y, const void *X, const void *gamma, const void *beta, float eps,
                   const void *W, const void *bias, const void *residual,
                   int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                   int w_layout, int bias_mode, int epi, int out_dtype,
                   void *ws, size_t ws_bytes, void *stream) {
    GemmArgs a;
    int rc = fill_args(a, Y, X, W, bias, residual, T, K, F, ldY, ldX, ldW, w_layout, bias_mode, epi, out_dtype, 0, 0, 0);
    if (rc != MI_OK) return rc;
    if (!g_ready) return MI_ERROR_DEVICE;
    if (T < 1 || T > 8) return MI_DECLINE_EXTENT;
    if (!mfma_addressable(a, w_layout == MI_W_KF)) return MI_DECLINE_OPERANDS;
    if ((gamma && !aligned_to(gamma, 16)) || (beta && !aligned_to(beta, 16))) return MI_DECLINE_OPERANDS;
    if (w_layout == MI_W_FK && (size_t)8 * K * sizeof(half_t) > SKINNY_FK_LDS_MAX) return MI_DECLINE_EXTENT;
    a.ln_on = 1; a.ln_gamma = (const half_t *)gamma; a.ln_beta = (const half_t *)beta; a.ln_eps = eps;
    return run_skinny(a, w_layout == MI_W_KF, ws, ws_bytes, (hipStream_t)stream);
}

}  // extern "C"
