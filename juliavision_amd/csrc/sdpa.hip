// Scaled-dot-product attention for gfx950.
//
//  flash_fwd_kernel   fused attention on MFMA 32x32x16 f16: S^T = K.Q^T and
//                     O^T = V^T.P^T, so that the score tile leaves the first
//                     product in exactly the register layout the second product
//                     consumes -- scores and probabilities never touch LDS or
//                     HBM.  Online softmax in fp32, one query per lane pair.
//  sdpa_rows_kernel   one workgroup per (query row, key split): the
//                     bandwidth-bound form for decode-sized Lq, and the
//                     always-available path for additive masks, odd head
//                     sizes and strided operands; split partials are merged by
//                     sdpa_merge_kernel.
//
// Operands are (E, L, H, B) with element strides (the reference's layout,
// DNNKernels/src/kernels/extern/attention.jl:1-22); out is dense (E, Lq, H, B).
#include "common.hpp"
#include <atomic>
#include <cstdlib>
#include <type_traits>

namespace {

struct SdpaArgs {
    void *out;
    const half_t *q, *k, *v;
    long qs[4], ks[4], vs[4], os[4];   // (E, L, H, B) element strides
    const void *bias;
    long bs[4];                    // (Lk, Lq, H, B) element strides, 0 = broadcast
    const int *kv_len;
    float *part_o, *part_ml;       // split partials: [split][row][E], [split][row][2] (sdpa_decode_kernel: [row][split])
    unsigned *tickets;             // sdpa_decode_kernel with nsplit > 1: one arrival counter per (head, batch), zero between launches
    // sdpa_decode_kernel only: the newest key/value row (1 x E per head and batch); when set, key kv_len - 1 is
    // taken from here instead of the cache and written into the cache on the way (k, v are then written to)
    const half_t *k_new, *v_new;
    long ns[4];
    int E, Lq, Lk, H, B;
    int out_f32, bias_f32, nsplit;
    float scale;
};

constexpr float LOG2E = 1.4426950408889634f;

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// ------------------------------------------------------------------------------------------
// Fused kernel.  Workgroup = 4 waves = 128 queries (32 per wave); keys walked in
// blocks of BC = 64 through three LDS stages, both operands as they lie in memory:
//   Ks [BC][EP+8]    keys x head-dim   (A operand of S^T = K.Q^T, plain 16-byte reads)
//   Vs [BC][VLD]     keys x head-dim   (VLD = flash_vld(EP); A operand of O^T = V^T.P^T through
//                    ds_read_b64_tr_b16, which transposes 4 keys x 16 head-dim
//                    values per 16 lanes on the way out of LDS)
//
// MFMA 32x32 accumulator layout: lane l, register r holds row 8(r/4)+4(l/32)+r%4,
// column l%32.  With rows = keys and columns = queries, a lane owns one query
// and 16 keys per 32-key tile: row maxima and sums need one exchange with lane
// l^32.  Registers 8b..8b+7 of a tile are, in order, the keys
// {16b+4h+0..3, 16b+8+4h+0..3} (h = l/32): that is the k-order in which P^T is fed
// to the second product, and V^T is read from LDS in the same order.
//
// Softmax bookkeeping is arranged to cost as few vector instructions as possible,
// because at head size 64 the exponentials, not the MFMAs, are the long pole:
//   * Q is pre-multiplied by scale*log2(e) (in fp32, rounded to fp16 once), so the
//     first product is already in the base-2 exponent domain;
//   * the reference point M of the running softmax is subtracted by the MFMA itself:
//     the first product carries one extra k-step whose operands contribute
//     1.0 * (-M[query]) to every score -- or, in the ping-pong form, starts its chain from
//     -M[query] instead of zero -- so it delivers t = s - M and p = exp2(t)
//     needs no further arithmetic (M is kept fp16-representable so that what is
//     subtracted is exactly what the bookkeeping assumes);
//   * M is a *stale* reference, not the running maximum: it moves on the first
//     block and when a probability would leave fp16 range (some t reaches 16: the
//     fp32 row sum then grows by 2^16 in one block, which is what is tested), and then
//     to the block maximum.  The result is the same softmax -- every term of a row carries the
//     same factor 2^-M -- with the rescaling of flash.jl:25-38 applied lazily (the
//     reference's `lazyrescale`, flash.jl:1041-1096, skips it when no maximum grew;
//     this skips it until fp16 would overflow);
//   * row sums are plain fp32 adds of the probabilities: they overlap with the MFMAs of the
//     other wave on the SIMD, which v_dot2_f32_f16 was measured not to do.
//
// PP ("ping-pong"): eight waves per workgroup, 256 queries.  Waves w and w+4 share a SIMD and are kept
// half a key block apart by two workgroup barriers per block, so that while one of them is in its
// exponentials the other is in its matrix half (the block's second product and the next block's first):
// the matrix pipe and the vector ALU of a SIMD are then busy with different waves instead of both
// waves wanting the same unit at the same time.  All eight waves stage: a wave writes its sixteenth of block j + 2
// in its own matrix half of block j, into the stage whose last readers finished before the barrier it just passed,
// and two barriers lie between the later group's write and the first read of that stage.
//
// KH = 2 (grids that leave every CU at most one workgroup): eight waves on 128 queries.  Waves w and w+4 own the
// same 32 queries and share a SIMD; a stage holds 128 keys, of which waves 0-3 take the first 64 and waves 4-7 the
// second, so each wave walks half of the keys and a SIMD always has a second wave to run.  The two partial
// (O, M, l) of a query meet in LDS at the end (the merge identity of flash.jl:1385-1391), waves 0-3 store.
// It runs with PP as well: its two key-half groups then take turns like the two query groups above; all waves stage.
// Halves per V row in LDS: a multiple of 64 plus 32, so that consecutive key rows start 64 bytes apart modulo the
// 128 bytes of the banks (96 for head sizes 64 and 96, 160 for 128; 112 measured the same as 96 at 96).
constexpr int flash_vld(int EP) { return EP == 96 ? EP : EP + 32; }

//
// BIAS (four-wave form only): an additive mask (Lk, Lq, H, B), keys contiguous, fp16 or fp32, any of the other axes
// broadcast.  A lane owns one query and, per block, eight runs of four consecutive keys: its 32 mask values of block
// j + 1 are requested while block j is worked on (two register sets, like the scores) and join the scores, times
// log2(e), ahead of the exponentials -- the reference's bias term of attention.jl:55-59, which its own fused kernel
// declines (flash.jl:1327).
// BIAS = 3: an fp16 mask that depends on the key only (the query axis broadcast: a padding mask (B, 1, 1, Lk), a per-head key
// bias).  It costs no vector arithmetic at all: the extra k-step that subtracts the reference point also carries
// mask[key] * log2(e) -- the key-side operand holds the key's mask value in two slots, the query-side operand log2(e)
// split into an fp16 part just below it and the (positive) rest, so a -inf mask value gives -inf through both products
// and never meets a zero or a negative factor.  The (b, h) row of the mask sits in LDS behind the stages, copied there
// once, zero beyond the last key (FLASH_KEYMASK_MAX keys at most): a first product reads one value per lane and tile.
template <int EP, bool PP, int KH = 1, int BIAS = 0>      // BIAS: 0 none, 1 fp16, 2 fp32, 3 fp16 by key only
__global__ __launch_bounds__((PP || KH == 2) ? 512 : 256, (EP <= 96 && !PP && KH == 1 && (BIAS == 0 || EP == 64)) ? 2 : 1) void flash_fwd_kernel(SdpaArgs p) {
    static_assert(BIAS == 0 || (!PP && KH == 1) || (PP && KH == 2 && (BIAS == 1 || BIAS == 3) && EP == 64) || (PP && BIAS == 3 && EP == 64),
                  "the mask rides in the four-wave form, and as fp16 in the key-halves form; one that depends on the key only in every form");
    // PP with KH = 2: the two key-half groups of the eight-wave form (same 128 queries) take turns at the vector
    // and matrix units like the two query groups of the 256-query form do; every thread stages.
    constexpr int BC = 64, BR = (PP && KH == 1) ? 256 : 128, NT = (KH == 2 || PP) ? 512 : 256;     // NT: threads that stage K and V
    constexpr int BCS = BC * KH;                                                // keys per LDS stage
    constexpr int KLD = EP + 8, VLD = flash_vld(EP);
    constexpr int KS = EP / 16;       // k16 steps over the head dim
    constexpr int ET = EP / 32;       // 32-wide head-dim tiles of O
    constexpr int KCH = EP / 8;       // 16-byte chunks per key row
    constexpr int PER = BCS * KCH / NT;
    constexpr float TH = 8.0f;
    extern __shared__ __align__(16) char smem[];
    half_t (*Ks)[BCS * KLD] = reinterpret_cast<half_t (*)[BCS * KLD]>(smem);
    half_t (*Vs)[BCS * VLD] = reinterpret_cast<half_t (*)[BCS * VLD]>(smem + 3 * BCS * KLD * 2);
    half_t *Ms = reinterpret_cast<half_t *>(smem + 3 * BCS * (KLD + VLD) * 2);       // BIAS 3: the mask row, then zeros

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tid = threadIdx.x & (NT - 1);                  // index among the staging threads
    const int grp = wave >> 2;                               // PP, KH = 2: 0 = waves 0-3, 1 = waves 4-7
    const int qw = KH == 2 ? (wave & 3) : wave;              // which 32 queries of the block
    const int gk = KH == 2 ? grp * BC : 0;                   // this wave's first key within a stage
    constexpr bool loader = true;                            // every wave stages its share of a key block
    const int hl = lane >> 5, l32 = lane & 31;
    // Workgroups are dealt to the 8 XCDs round-robin in launch order; renumbering them so that each XCD
    // owns a contiguous run keeps all query blocks of a head on one XCD, whose L2 then holds that head's
    // K and V once instead of every XCD holding every head's.
    int qblk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    {
        const int nqb = gridDim.x, total = nqb * gridDim.y * gridDim.z;
        if ((total & 7) == 0) {
            int id = blockIdx.x + nqb * (blockIdx.y + gridDim.y * blockIdx.z);
            id = (id & 7) * (total >> 3) + (id >> 3);
            qblk = id % nqb;
            h = (id / nqb) % gridDim.y;
            b = id / (nqb * gridDim.y);
        }
    }
    // Key splits (small grids only): the x index carries (query block, split); a split walks a run of whole
    // key blocks and leaves (O, M, l) partials for sdpa_merge_kernel instead of the normalised output.
    const int split = PP ? 0 : qblk % p.nsplit;
    if (!PP) qblk /= p.nsplit;
    const int q0 = qblk * BR + qw * 32;
    const half_t *qb = p.q + h * p.qs[2] + b * p.qs[3];
    const half_t *kb = p.k + h * p.ks[2] + b * p.ks[3];
    const half_t *vb = p.v + h * p.vs[2] + b * p.vs[3];
    int Lk = p.Lk;
    if (p.kv_len) Lk = max(0, min(Lk, p.kv_len[b]));
    int LkLoad = p.Lk;                 // keys that exist in memory (rows past it are re-reads of the last one)
    if (!PP && p.nsplit > 1) {
        const int per = (((p.Lk + BC - 1) / BC + p.nsplit - 1) / p.nsplit) * BC;      // keys per split, whole blocks
        const int kbeg = split * per;
        kb += (long)kbeg * p.ks[1];
        vb += (long)kbeg * p.vs[1];
        Lk = max(0, min(Lk - kbeg, per));
        LkLoad = max(1, min(p.Lk - kbeg, per));
    }
    const float c = p.scale * LOG2E;
    // barrier between the half-block intervals of the ping-pong: LDS traffic of this wave done, nothing else waited for
    auto pp_barrier = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // Q^T fragments: column = query l32, k = head-dim 16 ks + 8 hl .. +7, times scale*log2(e)
    // (requested here, scaled after the first two key blocks have been requested as well: the workgroup's
    // start-up then costs one trip to memory, not three)
    half8v qf[KS];
    u32x4 qraw[KS];
    {
        const int qr = min(q0 + l32, p.Lq - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int e = 16 * ks + 8 * hl;
            u32x4 z = {0u, 0u, 0u, 0u};
            qraw[ks] = e < p.E ? ldg16(qb + (long)qr * p.qs[1] + e) : z;
        }
    }

    // Per-thread sources of its PER 16-byte chunks of a key block; a block whose
    // 64 keys all exist is fetched with one 64-bit add per chunk, the ragged last
    // one re-reads the last valid key for the rows past the end.
    u32x4 kr[PER], vr[PER];
    const half_t *kp0[PER], *vp0[PER];
    bool eok[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int cidx = tid + i * NT;
        const int row = cidx / KCH, ch = cidx % KCH;
        eok[i] = ch * 8 < p.E;
        kp0[i] = kb + (long)row * p.ks[1] + (eok[i] ? ch * 8 : 0);
        vp0[i] = vb + (long)row * p.vs[1] + (eok[i] ? ch * 8 : 0);
    }
    auto load_into = [&](u32x4 (&kx)[PER], u32x4 (&vx)[PER], int key0) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        if (key0 + BCS <= LkLoad && p.E == EP) {   // the common case: no predicate, no clamp
            const long ko = (long)key0 * p.ks[1], vo = (long)key0 * p.vs[1];
#pragma unroll
            for (int i = 0; i < PER; i++) {
                kx[i] = ldg16(kp0[i] + ko);
                vx[i] = ldg16(vp0[i] + vo);
            }
        } else {
#pragma unroll
            for (int i = 0; i < PER; i++) {
                const int cidx = tid + i * NT;
                const int row = cidx / KCH, ch = cidx % KCH;
                const int key = min(key0 + row, LkLoad - 1);
                kx[i] = eok[i] ? ldg16(kb + (long)key * p.ks[1] + ch * 8) : z;
                vx[i] = eok[i] ? ldg16(vb + (long)key * p.vs[1] + ch * 8) : z;
            }
        }
    };
    auto store_from = [&](const u32x4 (&kx)[PER], const u32x4 (&vx)[PER], int buf) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int cidx = tid + i * NT;
            const int row = cidx / KCH, ch = cidx % KCH;
            *reinterpret_cast<u32x4 *>(&Ks[buf][row * KLD + ch * 8]) = kx[i];
            *reinterpret_cast<u32x4 *>(&Vs[buf][row * VLD + ch * 8]) = vx[i];
        }
    };
    auto load_kv = [&](int key0) { load_into(kr, vr, key0); };
    auto store_kv = [&](int buf) { store_from(kr, vr, buf); };

    float16v o_acc[ET];
#pragma unroll
    for (int t = 0; t < ET; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[t][r] = 0.0f;
    // The reference point M rides along in the first product.  SEED (the 256-query ping-pong form, whose matrix half
    // is the longer one): every score of a lane belongs to its one query, so the chain starts from -M[query] in all
    // sixteen accumulator registers instead of from zero (config 4: 87 -> 79 us).  Otherwise: one more k-step with the
    // operand pair 1.0 and -M, two MFMAs more per block but sixteen registers fewer -- the forms that run two
    // workgroups per CU or are 96 wide sit at the register limit, and measured the same or slower with the seed
    // (config 3 19.0 -> 19.5 us, the 72-wide windows 13.4 -> 15.2 us).
    constexpr bool SEED = PP && KH == 1;
    float16v negm;
    half8v kext, qext;
#pragma unroll
    for (int r = 0; r < 16; r++) negm[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) { kext[j] = (half_t)0.0f; qext[j] = (half_t)0.0f; }
    if (hl == 0) kext[0] = (half_t)1.0f;
    if constexpr (BIAS == 3) {
        // log2(e) = 1.4423828125 (the fp16 value below it) + 0.00031220...: both factors positive
        if (hl == 0) { qext[1] = (half_t)1.4423828125f; qext[2] = (half_t)(1.44269504088896340736f - 1.4423828125f); }
    }
    float m_ref = 0.0f, l_run = 0.0f;    // m_ref is always exactly representable in fp16
    bool first = true;

    // Three LDS stages: while block j is in its softmax and second product, the first
    // product of block j+1 already runs (its MFMAs fill the matrix pipe under the
    // exponentials), and block j+2 is on its way from memory into the third stage.
    const int nblk = (Lk + BCS - 1) / BCS;
    {
        u32x4 kr1[PER], vr1[PER];
        if (nblk > 0 && loader) load_kv(0);
        if (nblk > 1 && loader) load_into(kr1, vr1, BCS);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const half8v t = as_half8(qraw[ks]);
#pragma unroll
            for (int j = 0; j < 8; j++) qf[ks][j] = (half_t)((float)t[j] * c);
        }
        if (nblk > 0 && loader) store_kv(0);
        if (nblk > 1 && loader) store_from(kr1, vr1, 1);
        if constexpr (BIAS == 3) {
            // every block this workgroup walks, whole: keys past the last one read zero (the ragged block's own test
            // excludes them), and so does the slot behind them, which the lanes that feed no mask value read
            const unsigned short *mrow = reinterpret_cast<const unsigned short *>(p.bias) + (long)h * p.bs[2] + (long)b * p.bs[3];
            for (int i = threadIdx.x; i <= nblk * BCS; i += (int)blockDim.x)
                reinterpret_cast<unsigned short *>(Ms)[i] = i < p.Lk ? mrow[(long)i * p.bs[0]] : (unsigned short)0;
        }
    }
    __syncthreads();
    // BIAS 3: where a lane finds the mask value it feeds to the extra k-step (key l32 of a tile, from the lanes that hold
    // k-slots 0..7; the others read the zero behind the row)
    const int msel = hl == 0 ? 1 : 0;
    const int moff = hl == 0 ? gk + l32 : nblk * BCS;

    // lane s of a 16-lane block addresses key (s/4), head-dim 4 (s%4) .. +3 of its 4 x 16 patch
    const int vtoff = (gk + 4 * hl + ((lane & 15) >> 2)) * VLD + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const int ktoff = (gk + l32) * KLD + 8 * hl;
    const float16v zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // t = s*scale*log2(e) - M, straight out of the MFMA chain
    auto qk = [&](float16v (&s)[2], int st, int jblk) {
        const half_t *kbase = &Ks[st][ktoff];
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
            const half_t *kp_ = kbase + 32 * kt * KLD;
            if constexpr (SEED)
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8v *>(kp_), qf[0], negm, 0, 0, 0);
            else
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8v *>(kp_), qf[0], zero16, 0, 0, 0);
#pragma unroll
            for (int ks = 1; ks < KS; ks++)
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8v *>(kp_ + 16 * ks), qf[ks], s[kt], 0, 0, 0);
            if constexpr (BIAS == 3) {
                half8v kx = kext;
                const half_t m = Ms[moff + (min(jblk, nblk - 1) * BCS + 32 * kt) * msel];      // (the product issued after the last block stays inside the row)
                kx[1] = m;
                kx[2] = m;
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kx, qext, s[kt], 0, 0, 0);
            } else if constexpr (!SEED) s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kext, qext, s[kt], 0, 0, 0);
        }
    };
    // p = 2^t as fp16 MFMA operands; the row sum is kept in fp32 with plain adds (v_dot2_f32_f16 on the
    // packed pairs costs fewer instructions but does not run under MFMAs: measured 8 % slower)
    auto probs = [&](const float16v (&s)[2], half8v (&pf)[2][2], float &l) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s[kt][r]), p1 = __builtin_amdgcn_exp2f(s[kt][r + 1]);
                const half2v pk = {(half_t)p0, (half_t)p1};
                pf[kt][r >> 3][r & 7] = pk[0];
                pf[kt][r >> 3][(r & 7) + 1] = pk[1];
                l += p0 + p1;
            }
    };

    // The lane's mask values of one key block: eight runs of four keys (tile kt, register group g: keys
    // key0 + 32 kt + 8 g + 4 hl .. +3), raw as they lie in memory.  Runs past the last key read nothing.
    struct BiasRegs { u32x4 w[BIAS == 2 ? 8 : (BIAS == 1 ? 4 : 1)]; };
    const char *brow = nullptr;
    if constexpr (BIAS == 1 || BIAS == 2) {
        const int qr = min(q0 + l32, p.Lq - 1);
        brow = reinterpret_cast<const char *>(p.bias) + ((long)qr * p.bs[1] + (long)h * p.bs[2] + (long)b * p.bs[3]) * (BIAS == 2 ? 4 : 2);
    }
    auto load_bias = [&](BiasRegs &br, int j) {
        if constexpr (BIAS == 1 || BIAS == 2) {
            const int key0 = j * BCS + gk;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int key = key0 + 32 * kt + 8 * g + 4 * hl, idx = kt * 4 + g;
                    if constexpr (BIAS == 2) {
                        float4v v = {0.f, 0.f, 0.f, 0.f};
                        const float *src = reinterpret_cast<const float *>(brow) + key;
                        if (key + 3 < p.Lk) v = *reinterpret_cast<const float4v *>(src);
                        else for (int e = 0; e < 4; e++) if (key + e < p.Lk) v[e] = src[e];
                        br.w[idx] = __builtin_bit_cast(u32x4, v);
                    } else {
                        u32x2 v = {0u, 0u};
                        const half_t *src = reinterpret_cast<const half_t *>(brow) + key;
                        if (key + 3 < p.Lk) v = *reinterpret_cast<const u32x2 *>(src);
                        else {
                            half4v t = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
                            for (int e = 0; e < 4; e++) if (key + e < p.Lk) t[e] = src[e];
                            v = __builtin_bit_cast(u32x2, t);
                        }
                        br.w[idx >> 1][(idx & 1) * 2] = v[0];
                        br.w[idx >> 1][(idx & 1) * 2 + 1] = v[1];
                    }
                }
        }
    };
    auto add_bias = [&](float16v (&sc)[2], const BiasRegs &br) {
        if constexpr (BIAS == 1 || BIAS == 2) {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int idx = kt * 4 + g;
                    if constexpr (BIAS == 2) {
                        const float4v v = __builtin_bit_cast(float4v, br.w[idx]);
#pragma unroll
                        for (int e = 0; e < 4; e++) sc[kt][4 * g + e] = fmaf(v[e], LOG2E, sc[kt][4 * g + e]);
                    } else {
                        const u32x2 raw = {br.w[idx >> 1][(idx & 1) * 2], br.w[idx >> 1][(idx & 1) * 2 + 1]};
                        const half4v v = __builtin_bit_cast(half4v, raw);
#pragma unroll
                        for (int e = 0; e < 4; e++) sc[kt][4 * g + e] = fmaf((float)v[e], LOG2E, sc[kt][4 * g + e]);
                    }
                }
        }
    };
    BiasRegs ba, bb;
    float16v sa[2], sb[2];
    if constexpr (BIAS == 1 || BIAS == 2) { if (nblk > 0) load_bias(ba, 0); }
    if (nblk > 0) qk(sa, 0, 0);

    // One key block: sc holds its scores (computed one iteration earlier), sn receives the next block's.
    auto iter = [&](auto MASK_, float16v (&sc)[2], float16v (&sn)[2], BiasRegs &bc, BiasRegs &bn, int j) {
        constexpr bool MASK = decltype(MASK_)::value;
        const int key0 = j * BCS + gk;
        const int st = j % 3, st1 = (j + 1) % 3, st2 = (j + 2) % 3;
        const bool next2 = j + 2 < nblk && loader;
        if (next2) load_kv((j + 2) * BCS);
        if constexpr (BIAS == 1 || BIAS == 2) {
            if (j + 1 < nblk) load_bias(bn, j + 1);
            add_bias(sc, bc);
        }
        if constexpr (MASK) {           // the ragged last block: excluded keys get -inf
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = key0 + 32 * kt + 8 * (r >> 2) + 4 * hl + (r & 3);
                    if (key >= Lk) sc[kt][r] = -INFINITY;
                }
        }
        // Fast path: exponentiate against the current reference point.  Without the ping-pong the next block's
        // first product is issued here as well, to run underneath.  (After the last block that product multiplies a
        // stale stage: wasted, harmless, and it keeps this stretch free of branches.)  With the ping-pong it moves
        // behind the second product: a block is then a vector half (the exponentials, ~610 cycles of issue) and a
        // matrix half (both products, 18 MFMAs = 576 cycles) of about equal length, and the two wave groups, half a
        // block apart, always want different units -- 90.7 -> 83.5 us on 16 heads x 4096 x 64; with the first product
        // in the vector half that half was twice as long as the other and set the pace of both.
        __builtin_amdgcn_sched_barrier(0);
        // Without the ping-pong the stretch that mixes exponentials with the next block's first product issues ahead
        // of the other wave of the SIMD, the second product behind it (1-4 % on the measured shapes; the opposite
        // assignment loses 4 %).  Between the ping-pong's halves priorities change nothing.
        if constexpr (!PP) {
            __builtin_amdgcn_s_setprio(1);
            qk(sn, st1, j + 1);
        }
        half8v pf[2][2];
        float l_new = l_run;
        probs(sc, pf, l_new);
        // Four-wave forms: the block's largest exponent, three at a time, found under the next block's first product
        // (these forms sit at the register limit, and the maximum taken here is what lets the scores' registers go
        // early: with the test below on the row sum alone the 96-wide instance spills twice as much).
        float tmax = 0.0f;
        if constexpr (!PP) {
            tmax = fmaxf(sc[0][0], sc[1][0]);
#pragma unroll
            for (int r = 1; r < 16; r++) tmax = fmaxf(fmaxf(tmax, sc[0][r]), sc[1][r]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * KS, 0);
#pragma unroll
        for (int g = 0; g < 2 * KS + 2; g++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 64 / (2 * KS + 2), 0);     // the remaining vector work trails the last MFMA
        }
        __builtin_amdgcn_sched_barrier(0);
        // A probability leaves fp16 range at t >= 16 (2^16 rounds to infinity).  The row sum, kept in fp32 from the
        // unrounded values, tells: it cannot have grown by less than 2^16 - 16 if one of the block's terms did
        // (and if it grew that much through many smaller terms, settling a new reference point is still right, only
        // not needed).  Then, and on the first block, settle a new reference point: the block maximum, for the rows
        // that outgrew the old one by 2^TH; rescale what was accumulated; redo the exponentials.  In the eight-wave
        // forms the maximum is only looked for here: their fast path spends no instruction on it.
        const bool outgrown = PP ? !(l_new - l_run < 65504.0f) : tmax >= 15.9f;
        if (__any(first || outgrown)) {
            if constexpr (PP) {
                tmax = fmaxf(sc[0][0], sc[1][0]);
#pragma unroll
                for (int r = 1; r < 16; r++) tmax = fmaxf(fmaxf(tmax, sc[0][r]), sc[1][r]);
            }
            float mx = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const bool grow = (mx > TH || first) && mx != -INFINITY;
            const half_t m16 = (half_t)(m_ref + (grow ? mx : 0.0f));
            const float d = (float)m16 - m_ref;
            const float alpha = __builtin_amdgcn_exp2f(-d);
            m_ref += d;
            l_run *= alpha;
            if constexpr (SEED) {
#pragma unroll
                for (int r = 0; r < 16; r++) negm[r] = -(float)m16;
            } else if (hl == 0) qext[0] = -m16;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) { sc[kt][r] -= d; if constexpr (!PP) sn[kt][r] -= d; }   // sn was formed against the old M
#pragma unroll
            for (int t = 0; t < ET; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) o_acc[t][r] *= alpha;
            l_new = l_run;
            probs(sc, pf, l_new);
        }
        l_run = l_new;
        first = false;
        if constexpr (PP) {
            // Second half of the block.  Block j+2 goes into the stage whose last readers (the other
            // group's second product of block j-1) finished before the barrier just passed; the barrier
            // that ends this interval publishes it before anyone's first product of block j+2.
            pp_barrier();
            if (next2) store_kv(st2);
            __builtin_amdgcn_sched_barrier(0);
        }
        // O^T += V^T . P^T
        if constexpr (!PP) __builtin_amdgcn_s_setprio(0);
        const half_t *vbase = &Vs[st][vtoff];
#pragma unroll
        for (int t = 0; t < ET; t++) {
            const half_t *vp = vbase + 32 * t;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int bb = 0; bb < 2; bb++) {
                    const half_t *vq = vp + (32 * kt + 16 * bb) * VLD;
                    short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(vq));
                    short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(vq + 8 * VLD));
                    short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    o_acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, both), pf[kt][bb], o_acc[t], 0, 0, 0);
                }
        }
        if constexpr (PP) {
            qk(sn, st1, j + 1);  // the next block's scores, against the reference point as it stands now
            // the matrix half's fragment reads (V for the second product, K for the first) run ten ahead of the MFMAs
            // that consume them: config 3 18.9 -> 18.3 us, config 2 21.5 -> 21.0 us; six ahead or all 24 ahead lose
            constexpr int NRD = 4 * ET * 2 + 2 * KS, NMF = 4 * ET + 2 * KS + 2, AHEAD = 10;
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int g = 0; g < NMF; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, (NRD - AHEAD + NMF - 1) / NMF, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            pp_barrier();
        } else {
            if (next2) store_kv(st2);
            __syncthreads();
        }
    };
    // blocks in which every key of this wave is valid (with KH = 2: its half of the stage)
    const int nfull = KH == 2 ? (Lk - gk + BC) / BCS : Lk / BC;
    if (PP && grp == 1) pp_barrier();    // waves 4-7 run half a block behind waves 0-3
    int j = 0;
    for (; j + 2 <= nfull; j += 2) {
        iter(std::false_type{}, sa, sb, ba, bb, j);
        iter(std::false_type{}, sb, sa, bb, ba, j + 1);
    }
    if constexpr (KH == 1) {
        if (j < nfull) {
            iter(std::false_type{}, sa, sb, ba, bb, j);
            if (j + 1 < nblk) iter(std::true_type{}, sb, sa, bb, ba, j + 1);
        } else if (j < nblk) {
            iter(std::true_type{}, sa, sb, ba, bb, j);
        }
    } else {
        // Both halves of the workgroup run all nblk blocks (every block has a workgroup barrier), whatever
        // share of them is masked for this half: at most one full block is left here, then masked ones.
        if (j < nblk) { if (j < nfull) iter(std::false_type{}, sa, sb, ba, bb, j); else iter(std::true_type{}, sa, sb, ba, bb, j); j++; }
        if (j < nblk) { iter(std::true_type{}, sb, sa, bb, ba, j); j++; }
        if (j < nblk) { iter(std::true_type{}, sa, sb, ba, bb, j); j++; }
    }

    if (PP && grp == 0) pp_barrier();    // ... so waves 0-3 meet their last barrier here
    // Both lanes of a query hold half of its row sum.
    l_run += __shfl_xor(l_run, 32, 64);

    if constexpr (KH == 2) {
        // Waves 4-7 hand their (O, M, l) to the wave that owns the same queries; the last block's barrier has
        // passed, so the stages are idle.  Lane-major slots: the partner's lane holds the same elements.
        constexpr int SLOT = (ET * 16 + 2) * 64;
        constexpr int MOFF = (4 * 32 * (EP + 4) * 4 + 255) / 256 * 256;      // past what the store staging will use
        float *xo = reinterpret_cast<float *>(smem + MOFF) + qw * SLOT;
        static_assert(MOFF + 4 * SLOT * 4 <= 3 * BCS * (KLD + VLD) * 2, "merge slots leave the stages");
        if (grp == 1) {
#pragma unroll
            for (int t = 0; t < ET; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) xo[(t * 16 + r) * 64 + lane] = o_acc[t][r];
            xo[(ET * 16) * 64 + lane] = m_ref;
            xo[(ET * 16 + 1) * 64 + lane] = l_run;
        }
        __syncthreads();
        if (grp == 1) return;
        const float m1 = xo[(ET * 16) * 64 + lane], l1 = xo[(ET * 16 + 1) * 64 + lane];
        // a side that saw no valid key has l = 0 and a meaningless reference point
        const float ma = l_run > 0.0f ? m_ref : -INFINITY, mb = l1 > 0.0f ? m1 : -INFINITY;
        const float mm = fmaxf(ma, mb);
        const float a0 = l_run > 0.0f ? __builtin_amdgcn_exp2f(ma - mm) : 0.0f, a1 = l1 > 0.0f ? __builtin_amdgcn_exp2f(mb - mm) : 0.0f;
#pragma unroll
        for (int t = 0; t < ET; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) o_acc[t][r] = o_acc[t][r] * a0 + xo[(t * 16 + r) * 64 + lane] * a1;
        l_run = l_run * a0 + l1 * a1;
        m_ref = mm;
    }

    // out(e, q, h, b); lane owns query q0 + l32 and, per tile t and group g, the four head-dim values
    // e = 32 t + 8 g + 4 hl + 0..3: stored from the registers, a wave's store instruction would touch 32 rows
    // with 16 or 32 bytes each.  Instead each wave lays its 32 x E tile out in its own stretch of the (now
    // idle) operand LDS and reads it back row-wise, so that every store instruction covers whole rows.
    // A wave reads only what it wrote itself and its LDS operations complete in order: no workgroup barrier.
    const bool partial = !PP && p.nsplit > 1;
    const bool as_f32 = partial || p.out_f32;
    constexpr int SLF = EP + 4, SLH = EP + 8;              // staged row lengths (floats, halves)
    float *stf = reinterpret_cast<float *>(smem) + qw * 32 * SLF;
    half_t *sth = reinterpret_cast<half_t *>(smem) + qw * 32 * SLH;
    const float inv = partial ? 1.0f : (l_run > 0.0f ? 1.0f / l_run : 0.0f);
    const long rows = (long)p.B * p.H * p.Lq;
    if (partial && hl == 0 && q0 + l32 < p.Lq) {
        // the reference point in natural-log units (it was kept in the base-2 domain), -inf for a split without a key
        const long row = ((long)b * p.H + h) * p.Lq + q0 + l32;
        float2v ml = {l_run > 0.0f ? m_ref * 0.6931471805599453f : -INFINITY, l_run};
        *reinterpret_cast<float2v *>(p.part_ml + ((long)split * rows + row) * 2) = ml;
    }
    if (PP && KH == 1 && as_f32) {
        // eight waves of fp32 rows do not fit the operand LDS: this combination stores from the registers
        const int qi = q0 + l32;
        if (qi < p.Lq) {
            const long base = (long)b * p.os[3] + (long)h * p.os[2] + (long)qi * p.os[1];
#pragma unroll
            for (int t = 0; t < ET; t++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int e = 32 * t + 8 * g + 4 * hl;
                    if (e < p.E) {
                        float4v o = {o_acc[t][4 * g] * inv, o_acc[t][4 * g + 1] * inv, o_acc[t][4 * g + 2] * inv, o_acc[t][4 * g + 3] * inv};
                        *reinterpret_cast<float4v *>(reinterpret_cast<float *>(p.out) + base + e) = o;
                    }
                }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < ET; t++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int e = 32 * t + 8 * g + 4 * hl;
            if (as_f32) {
                float4v o = {o_acc[t][4 * g] * inv, o_acc[t][4 * g + 1] * inv, o_acc[t][4 * g + 2] * inv, o_acc[t][4 * g + 3] * inv};
                *reinterpret_cast<float4v *>(stf + l32 * SLF + e) = o;
            } else {
                half4v o = {(half_t)(o_acc[t][4 * g] * inv), (half_t)(o_acc[t][4 * g + 1] * inv),
                            (half_t)(o_acc[t][4 * g + 2] * inv), (half_t)(o_acc[t][4 * g + 3] * inv)};
                *reinterpret_cast<half4v *>(sth + l32 * SLH + e) = o;
            }
        }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (as_f32) {
        constexpr int CPR = EP / 4;                        // 16-byte chunks per row
        float *dst0 = partial ? p.part_o + ((long)split * rows + ((long)b * p.H + h) * p.Lq) * p.E
                              : reinterpret_cast<float *>(p.out) + (long)b * p.os[3] + (long)h * p.os[2];
        const long rstride = partial ? p.E : p.os[1];
        for (int c = lane; c < 32 * CPR; c += 64) {
            const int row = c / CPR, e = (c % CPR) * 4;
            if (q0 + row < p.Lq && e < p.E)
                *reinterpret_cast<float4v *>(dst0 + (long)(q0 + row) * rstride + e) = *reinterpret_cast<const float4v *>(stf + row * SLF + e);
        }
    } else {
        constexpr int CPR = EP / 8;
        half_t *dst0 = reinterpret_cast<half_t *>(p.out) + (long)b * p.os[3] + (long)h * p.os[2];
        for (int c = lane; c < 32 * CPR; c += 64) {
            const int row = c / CPR, e = (c % CPR) * 8;
            if (q0 + row < p.Lq && e < p.E)
                *reinterpret_cast<u32x4 *>(dst0 + (long)(q0 + row) * p.os[1] + e) = *reinterpret_cast<const u32x4 *>(sth + row * SLH + e);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Fused attention for grids that leave most of the chip idle (head size 64, no mask): a workgroup owns 32 queries,
// and its NW waves (8, or 4 so that two workgroups share a CU) each walk their own run of whole 64-key blocks, so the
// chain a wave walks is Lk / NW keys long instead of Lk / 2.  Nothing is shared between the waves until the end, so
// nothing is staged for anyone else and the loop has no workgroup barrier: a wave takes its K fragments straight from
// memory in the layout the first product wants (lane = key, 16 bytes of one row per k-step: every row is read whole over
// the four k-steps), and passes its V block through a private stretch of LDS only for the transposing read of the second
// product (the wave's LDS operations complete in order: the write of block j + 1 follows the reads of block j without a
// wait).  Both are requested a block ahead.  The softmax is flash_fwd_kernel's (lazy reference point).  The waves'
// (O, M, l) meet in LDS and are merged with the rescaling identity of flash.jl:1385-1391, each thread finishing four
// consecutive head-dim values of one query.
template <int NW>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void flash_short_kernel(SdpaArgs p) {
    constexpr int EP = 64, KS = 4, ET = 2, BC = 64, VLD = flash_vld(64);
    constexpr int WREG = BC * VLD * 2;                        // bytes of a wave's V stretch; holds its (O, m, l) afterwards
    static_assert((ET * 16 + 2) * 64 * 4 <= WREG, "a wave's partial fits its own stretch");
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int hl = lane >> 5, l32 = lane & 31;
    half_t *Vw = reinterpret_cast<half_t *>(smem + wave * WREG);
    int qblk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    {
        // all query blocks of a head on one XCD (workgroups are dealt to the XCDs round robin)
        const int nqb = gridDim.x, total = nqb * gridDim.y * gridDim.z;
        if ((total & 7) == 0) {
            int id = blockIdx.x + nqb * (blockIdx.y + gridDim.y * blockIdx.z);
            id = (id & 7) * (total >> 3) + (id >> 3);
            qblk = id % nqb;
            h = (id / nqb) % gridDim.y;
            b = id / (nqb * gridDim.y);
        }
    }
    const int q0 = qblk * 32;
    const half_t *qb = p.q + h * p.qs[2] + b * p.qs[3];
    const half_t *kb = p.k + h * p.ks[2] + b * p.ks[3];
    const half_t *vb = p.v + h * p.vs[2] + b * p.vs[3];
    int Lk = p.Lk;
    if (p.kv_len) Lk = max(0, min(Lk, p.kv_len[b]));
    // this wave's keys: whole 64-key blocks, [kbeg, kend)
    const int per = (((Lk + BC - 1) / BC + NW - 1) / NW) * BC;
    const int kbeg = wave * per, kend = min(Lk, kbeg + per);
    const int nblk = kend > kbeg ? (kend - kbeg + BC - 1) / BC : 0;
    const int last = p.Lk - 1;                                // rows past the end re-read the last key that exists
    const float c = p.scale * LOG2E;

    u32x4 qraw[KS];
    {
        const int qr = min(q0 + l32, p.Lq - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qraw[ks] = ldg16(qb + (long)qr * p.qs[1] + 16 * ks + 8 * hl);
    }
    // K fragments of a block: tile kt (32 keys), k-step ks: key = key0 + 32 kt + l32, head dim 16 ks + 8 hl .. +7
    auto load_k = [&](u32x4 (&kf)[2][KS], int key0) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
            const half_t *row = kb + (long)min(key0 + 32 * kt + l32, last) * p.ks[1] + 8 * hl;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) kf[kt][ks] = ldg16(row + 16 * ks);
        }
    };
    // the wave's V block, 8 chunks of 16 bytes per lane: chunk lane + 64 i = (key, 8 head-dim values)
    u32x4 vr[8];
    auto load_v = [&](int key0) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int cidx = lane + 64 * i;
            vr[i] = ldg16(vb + (long)min(key0 + (cidx >> 3), last) * p.vs[1] + (cidx & 7) * 8);
        }
    };
    auto store_v = [&]() {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int cidx = lane + 64 * i;
            *reinterpret_cast<u32x4 *>(Vw + (cidx >> 3) * VLD + (cidx & 7) * 8) = vr[i];
        }
    };
    u32x4 ka[2][KS], kc[2][KS];
    if (nblk > 0) { load_k(ka, kbeg); load_v(kbeg); }
    half8v qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const half8v t = as_half8(qraw[ks]);
#pragma unroll
        for (int j = 0; j < 8; j++) qf[ks][j] = (half_t)((float)t[j] * c);
    }
    float16v o_acc[ET];
#pragma unroll
    for (int t = 0; t < ET; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[t][r] = 0.0f;
    float m_run = 0.0f, l_run = 0.0f;                        // m_run: the reference point, always exactly representable in fp16
    const int vtoff = (4 * hl + ((lane & 15) >> 2)) * VLD + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const float16v zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // The reference point of the running softmax is subtracted by the first product itself -- one more k-step with the
    // operand pair 1.0 and -M[query] -- and moves lazily, as in flash_fwd_kernel: on a wave's first block, and when a
    // probability would leave fp16 range (seen in the fp32 row sum growing by 2^16 within a block).
    constexpr float TH = 8.0f;
    half8v kext, qext;
#pragma unroll
    for (int jj = 0; jj < 8; jj++) { kext[jj] = (half_t)0.0f; qext[jj] = (half_t)0.0f; }
    if (hl == 0) kext[0] = (half_t)1.0f;
    bool first = true;
    auto probs = [&](const float16v (&sx)[2], half8v (&pf)[2][2], float &l) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(sx[kt][r]), p1 = __builtin_amdgcn_exp2f(sx[kt][r + 1]);
                pf[kt][r >> 3][r & 7] = (half_t)p0;
                pf[kt][r >> 3][(r & 7) + 1] = (half_t)p1;
                l += p0 + p1;
            }
    };
    auto iter = [&](u32x4 (&kcur)[2][KS], u32x4 (&knext)[2][KS], int j) {
        const int key0 = kbeg + j * BC;
        store_v();                                           // block j's V (requested one block ago) into the stretch
        if (j + 1 < nblk) { load_k(knext, key0 + BC); load_v(key0 + BC); }
        float16v sc[2];
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
            sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(kcur[kt][0]), qf[0], zero16, 0, 0, 0);
#pragma unroll
            for (int ks = 1; ks < KS; ks++) sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(kcur[kt][ks]), qf[ks], sc[kt], 0, 0, 0);
            sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kext, qext, sc[kt], 0, 0, 0);
        }
        if (key0 + BC > kend) {                              // the ragged last block: excluded keys get -inf
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (key0 + 32 * kt + 8 * (r >> 2) + 4 * hl + (r & 3) >= kend) sc[kt][r] = -INFINITY;
        }
        half8v pf[2][2];
        float l_new = l_run;
        probs(sc, pf, l_new);
        if (__any(first || !(l_new - l_run < 65504.0f))) {
            float tmax = fmaxf(sc[0][0], sc[1][0]);
#pragma unroll
            for (int r = 1; r < 16; r++) tmax = fmaxf(fmaxf(tmax, sc[0][r]), sc[1][r]);
            const float mx = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const bool grow = (mx > TH || first) && mx != -INFINITY;
            const half_t m16 = (half_t)(m_run + (grow ? mx : 0.0f));
            const float d = (float)m16 - m_run;
            const float alpha = __builtin_amdgcn_exp2f(-d);
            m_run += d;
            l_run *= alpha;
            if (hl == 0) qext[0] = -m16;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) sc[kt][r] -= d;
#pragma unroll
            for (int t = 0; t < ET; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) o_acc[t][r] *= alpha;
            l_new = l_run;
            probs(sc, pf, l_new);
        }
        l_run = l_new;
        first = false;
        // O^T += V^T . P^T
#pragma unroll
        for (int t = 0; t < ET; t++) {
            const half_t *vp = Vw + vtoff + 32 * t;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int bb = 0; bb < 2; bb++) {
                    const half_t *vq = vp + (32 * kt + 16 * bb) * VLD;
                    short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(vq));
                    short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(vq + 8 * VLD));
                    short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    o_acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, both), pf[kt][bb], o_acc[t], 0, 0, 0);
                }
        }
    };
    int j = 0;
    for (; j + 2 <= nblk; j += 2) {
        iter(ka, kc, j);
        iter(kc, ka, j + 1);
    }
    if (j < nblk) iter(ka, kc, j);

    // both lanes of a query hold half of its row sum
    l_run += __shfl_xor(l_run, 32, 64);
    // the wave's partial, lane-major, into its own stretch (its reads of V are behind it)
    float *xo = reinterpret_cast<float *>(smem + wave * WREG);
#pragma unroll
    for (int t = 0; t < ET; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) xo[(t * 16 + r) * 64 + lane] = o_acc[t][r];
    xo[(ET * 16) * 64 + lane] = m_run;
    xo[(ET * 16 + 1) * 64 + lane] = l_run;
    __syncthreads();
    // Thread (src lane, group) finishes query q0 + l32 at head dims 32 t + 8 g + 4 hl .. +3 for its (t, g).
    float aw[NW], mm = -INFINITY, den = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; w++) {
        // a wave that saw no valid key has l = 0 and a meaningless reference point
        const float *xw = reinterpret_cast<const float *>(smem + w * WREG);
        aw[w] = xw[(ET * 16 + 1) * 64 + lane] > 0.0f ? xw[(ET * 16) * 64 + lane] : -INFINITY;
        mm = fmaxf(mm, aw[w]);
    }
#pragma unroll
    for (int w = 0; w < NW; w++) {
        const float *xw = reinterpret_cast<const float *>(smem + w * WREG);
        aw[w] = aw[w] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(aw[w] - mm);
        den += aw[w] * xw[(ET * 16 + 1) * 64 + lane];
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    const int qi = q0 + l32;
    constexpr int COMBOS = 8 / NW;                            // (t, g) pairs per thread: 8 pairs over NW waves
#pragma unroll
    for (int cidx = 0; cidx < COMBOS; cidx++) {
        const int tg = wave * COMBOS + cidx, t = tg >> 2, g = tg & 3;
        float o4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const float *xw = reinterpret_cast<const float *>(smem + w * WREG);
#pragma unroll
            for (int i = 0; i < 4; i++) o4[i] += aw[w] * xw[(t * 16 + 4 * g + i) * 64 + lane];
        }
        if (qi < p.Lq) {
            const long off = (long)b * p.os[3] + (long)h * p.os[2] + (long)qi * p.os[1] + 32 * t + 8 * g + 4 * hl;
            if (p.out_f32) {
                const float4v o = {o4[0] * inv, o4[1] * inv, o4[2] * inv, o4[3] * inv};
                *reinterpret_cast<float4v *>(reinterpret_cast<float *>(p.out) + off) = o;
            } else {
                const half4v o = {(half_t)(o4[0] * inv), (half_t)(o4[1] * inv), (half_t)(o4[2] * inv), (half_t)(o4[3] * inv)};
                *reinterpret_cast<half4v *>(reinterpret_cast<half_t *>(p.out) + off) = o;
            }
        }
    }
}

// The short-chain form on 64-query tiles, for grids whose 32-query tiles would be a few more than the CUs (6 heads x
// 1370: 258) and for the traffic: in flash_short_kernel every 32-query tile reads all of its head's K and V from the L2,
// and with 43 tiles a head that read is what the loop waits for.  Here eight waves share a tile: wave w takes key
// quarter w % 4 for query half w / 4, and the two waves of a quarter share its K and V through LDS -- one of them fetches
// the K block, the other the V block, a block ahead, 8 chunks of 16 bytes a lane -- so a tile of twice the queries reads
// the same bytes.  K lies in LDS row-major with 16 bytes of padding (conflict-free 16-byte fragment reads), V as in
// flash_short_kernel.  One buffer per quarter: a workgroup barrier after the writes of block j, another before the
// writes of block j + 1; every wave takes part in every barrier (quarters with fewer blocks idle through the rest).
__global__ __launch_bounds__(512, 1) void flash_pair_kernel(SdpaArgs p) {
    constexpr int EP = 64, KS = 4, ET = 2, BC = 64, NQ = 4, VLD = flash_vld(64), KLD = EP + 8;
    constexpr int KBYTES = BC * KLD * 2, VBYTES = BC * VLD * 2, QREG = KBYTES + VBYTES;      // a quarter's K and V
    constexpr int WPART = (ET * 16 + 2) * 64 * 4;                                            // a wave's (O, m, l)
    static_assert(8 * WPART <= NQ * QREG, "the partials fit where the stages were");
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kq = wave & 3, qh = wave >> 2;
    const int hl = lane >> 5, l32 = lane & 31;
    half_t *Kw = reinterpret_cast<half_t *>(smem + kq * QREG);
    half_t *Vw = reinterpret_cast<half_t *>(smem + kq * QREG + KBYTES);
    int qblk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    {
        const int nqb = gridDim.x, total = nqb * gridDim.y * gridDim.z;
        if ((total & 7) == 0) {
            int id = blockIdx.x + nqb * (blockIdx.y + gridDim.y * blockIdx.z);
            id = (id & 7) * (total >> 3) + (id >> 3);
            qblk = id % nqb;
            h = (id / nqb) % gridDim.y;
            b = id / (nqb * gridDim.y);
        }
    }
    const int q0 = qblk * 64 + 32 * qh;
    const half_t *qb = p.q + h * p.qs[2] + b * p.qs[3];
    const half_t *kb = p.k + h * p.ks[2] + b * p.ks[3];
    const half_t *vb = p.v + h * p.vs[2] + b * p.vs[3];
    int Lk = p.Lk;
    if (p.kv_len) Lk = max(0, min(Lk, p.kv_len[b]));
    const int per = (((Lk + BC - 1) / BC + NQ - 1) / NQ) * BC;
    const int nmax = per / BC;                                // barriers are counted over this, by every wave
    const int kbeg = kq * per, kend = min(Lk, kbeg + per);
    const int nblk = kend > kbeg ? (kend - kbeg + BC - 1) / BC : 0;
    const int last = p.Lk - 1;
    const float c = p.scale * LOG2E;

    u32x4 qraw[KS];
    {
        const int qr = min(q0 + l32, p.Lq - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qraw[ks] = ldg16(qb + (long)qr * p.qs[1] + 16 * ks + 8 * hl);
    }
    // this wave's share of a block: the K rows (query half 0) or the V rows (query half 1), chunk lane + 64 i = (key, 8 head dims)
    const half_t *src = qh == 0 ? kb : vb;
    const long srow = qh == 0 ? p.ks[1] : p.vs[1];
    half_t *dst = qh == 0 ? Kw : Vw;
    const int dld = qh == 0 ? KLD : VLD;
    u32x4 pre[8];
    auto fetch = [&](int key0) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int cidx = lane + 64 * i;
            pre[i] = ldg16(src + (long)min(key0 + (cidx >> 3), last) * srow + (cidx & 7) * 8);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int cidx = lane + 64 * i;
            *reinterpret_cast<u32x4 *>(dst + (cidx >> 3) * dld + (cidx & 7) * 8) = pre[i];
        }
    };
    if (nblk > 0) fetch(kbeg);
    half8v qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const half8v t = as_half8(qraw[ks]);
#pragma unroll
        for (int j = 0; j < 8; j++) qf[ks][j] = (half_t)((float)t[j] * c);
    }
    float16v o_acc[ET];
#pragma unroll
    for (int t = 0; t < ET; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[t][r] = 0.0f;
    float m_run = 0.0f, l_run = 0.0f;
    const int ktoff = l32 * KLD + 8 * hl;
    const int vtoff = (4 * hl + ((lane & 15) >> 2)) * VLD + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const float16v zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    constexpr float TH = 8.0f;
    // the reference point is the first product's accumulator input: every score of a lane belongs to its one query
    float16v negm = zero16;
    bool first = true;
    auto probs = [&](const float16v (&sx)[2], half8v (&pf)[2][2], float &l) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(sx[kt][r]), p1 = __builtin_amdgcn_exp2f(sx[kt][r + 1]);
                pf[kt][r >> 3][r & 7] = (half_t)p0;
                pf[kt][r >> 3][(r & 7) + 1] = (half_t)p1;
                l += p0 + p1;
            }
    };
    for (int j = 0; j < nmax; j++) {
        const bool live = j < nblk;                          // uniform over the wave, and the same for both waves of a quarter
        const int key0 = kbeg + j * BC;
        if (j > 0) __syncthreads();                          // block j - 1 has been read by everyone
        if (live) stage();
        if (j + 1 < nblk) fetch(key0 + BC);
        __syncthreads();                                     // block j is in place
        if (!live) continue;
        float16v sc[2];
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
            const half_t *kp_ = Kw + ktoff + 32 * kt * KLD;
            sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8v *>(kp_), qf[0], negm, 0, 0, 0);
#pragma unroll
            for (int ks = 1; ks < KS; ks++)
                sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8v *>(kp_ + 16 * ks), qf[ks], sc[kt], 0, 0, 0);
        }
        if (key0 + BC > kend) {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (key0 + 32 * kt + 8 * (r >> 2) + 4 * hl + (r & 3) >= kend) sc[kt][r] = -INFINITY;
        }
        half8v pf[2][2];
        float l_new = l_run;
        probs(sc, pf, l_new);
        if (__any(first || !(l_new - l_run < 65504.0f))) {
            float tmax = fmaxf(sc[0][0], sc[1][0]);
#pragma unroll
            for (int r = 1; r < 16; r++) tmax = fmaxf(fmaxf(tmax, sc[0][r]), sc[1][r]);
            const float mx = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const bool grow = (mx > TH || first) && mx != -INFINITY;
            const half_t m16 = (half_t)(m_run + (grow ? mx : 0.0f));
            const float d = (float)m16 - m_run;
            const float alpha = __builtin_amdgcn_exp2f(-d);
            m_run += d;
            l_run *= alpha;
#pragma unroll
            for (int r = 0; r < 16; r++) negm[r] = -(float)m16;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) sc[kt][r] -= d;
#pragma unroll
            for (int t = 0; t < ET; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) o_acc[t][r] *= alpha;
            l_new = l_run;
            probs(sc, pf, l_new);
        }
        l_run = l_new;
        first = false;
#pragma unroll
        for (int t = 0; t < ET; t++) {
            const half_t *vp = Vw + vtoff + 32 * t;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int bb = 0; bb < 2; bb++) {
                    const half_t *vq = vp + (32 * kt + 16 * bb) * VLD;
                    short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(vq));
                    short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(vq + 8 * VLD));
                    short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    o_acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, both), pf[kt][bb], o_acc[t], 0, 0, 0);
                }
        }
    }
    l_run += __shfl_xor(l_run, 32, 64);
    __syncthreads();                                         // the last blocks have been read: the stages become the partials
    float *xo = reinterpret_cast<float *>(smem + wave * WPART);
#pragma unroll
    for (int t = 0; t < ET; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) xo[(t * 16 + r) * 64 + lane] = o_acc[t][r];
    xo[(ET * 16) * 64 + lane] = m_run;
    xo[(ET * 16 + 1) * 64 + lane] = l_run;
    __syncthreads();
    // the four quarters of this wave's query half meet; wave kq finishes (t, g) pairs 2 kq and 2 kq + 1 of its 32 queries
    float aw[NQ], mm = -INFINITY, den = 0.0f;
#pragma unroll
    for (int w = 0; w < NQ; w++) {
        const float *xw = reinterpret_cast<const float *>(smem + (qh * NQ + w) * WPART);
        aw[w] = xw[(ET * 16 + 1) * 64 + lane] > 0.0f ? xw[(ET * 16) * 64 + lane] : -INFINITY;
        mm = fmaxf(mm, aw[w]);
    }
#pragma unroll
    for (int w = 0; w < NQ; w++) {
        const float *xw = reinterpret_cast<const float *>(smem + (qh * NQ + w) * WPART);
        aw[w] = aw[w] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(aw[w] - mm);
        den += aw[w] * xw[(ET * 16 + 1) * 64 + lane];
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    const int qi = q0 + l32;
#pragma unroll
    for (int cidx = 0; cidx < 2; cidx++) {
        const int tg = kq * 2 + cidx, t = tg >> 2, g = tg & 3;
        float o4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < NQ; w++) {
            const float *xw = reinterpret_cast<const float *>(smem + (qh * NQ + w) * WPART);
#pragma unroll
            for (int i = 0; i < 4; i++) o4[i] += aw[w] * xw[(t * 16 + 4 * g + i) * 64 + lane];
        }
        if (qi < p.Lq) {
            const long off = (long)b * p.os[3] + (long)h * p.os[2] + (long)qi * p.os[1] + 32 * t + 8 * g + 4 * hl;
            if (p.out_f32) {
                const float4v o = {o4[0] * inv, o4[1] * inv, o4[2] * inv, o4[3] * inv};
                *reinterpret_cast<float4v *>(reinterpret_cast<float *>(p.out) + off) = o;
            } else {
                const half4v o = {(half_t)(o4[0] * inv), (half_t)(o4[1] * inv), (half_t)(o4[2] * inv), (half_t)(o4[3] * inv)};
                *reinterpret_cast<half4v *>(reinterpret_cast<half_t *>(p.out) + off) = o;
            }
        }
    }
}


// ------------------------------------------------------------------------------------------
// One workgroup (4 waves) per (query row, key split).  A wave walks keys 8 at a
// time: 8 lanes share a key, each owning 8-element head-dim chunks c, c+8, ...
// (NCH chunks, E <= 64 NCH).  Every 8-lane group keeps its own running
// (m, l, acc); groups, waves and splits are merged with the rescaling identity
// m = max m_s, l = sum e^{m_s-m} l_s, O = sum e^{m_s-m} O_s  (flash.jl:1385-1391).
template <int NCH, bool VEC>
__global__ __launch_bounds__(256) void sdpa_rows_kernel(SdpaArgs p) {
    __shared__ float red_ml[4][2];
    __shared__ float red_o[4][64 * NCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int grp = lane >> 3, cl = lane & 7;
    const int split = blockIdx.x % p.nsplit;
    const int row = blockIdx.x / p.nsplit;      // lq + Lq * h
    const int lq = row % p.Lq, h = row / p.Lq, b = blockIdx.z;
    int Lk = p.Lk;
    if (p.kv_len) Lk = max(0, min(Lk, p.kv_len[b]));
    // split ranges in units of 32 keys (one pass of the workgroup)
    const int units = (Lk + 31) / 32;
    const int per = (units + p.nsplit - 1) / p.nsplit;
    const int kbeg = min(Lk, split * per * 32), kend = min(Lk, (split + 1) * per * 32);

    const half_t *qp = p.q + (long)lq * p.qs[1] + h * p.qs[2] + b * p.qs[3];
    const half_t *kb = p.k + h * p.ks[2] + b * p.ks[3];
    const half_t *vb = p.v + h * p.vs[2] + b * p.vs[3];

    float qv[NCH][8];
#pragma unroll
    for (int ci = 0; ci < NCH; ci++) {
        const int e0 = (cl + 8 * ci) * 8;
        if (VEC) {
            u32x4 z = {0u, 0u, 0u, 0u};
            half8v t = as_half8(e0 < p.E ? ldg16(qp + e0) : z);
#pragma unroll
            for (int j = 0; j < 8; j++) qv[ci][j] = (float)t[j];
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) qv[ci][j] = e0 + j < p.E ? (float)qp[(long)(e0 + j) * p.qs[0]] : 0.0f;
        }
    }

    float m = -INFINITY, l = 0.0f;
    float acc[NCH][8];
#pragma unroll
    for (int ci = 0; ci < NCH; ci++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[ci][j] = 0.0f;

    // Every lane of the wave runs the same number of iterations (the shuffles below need all 64
    // lanes); a key past the end is computed on a clamped row and then given weight zero.  With
    // 16-byte addressable operands the next iteration's K and V chunks are requested before the
    // current ones are used, so a wave waits for memory once, not once per 8 keys.
    u32x4 kc[NCH], vc[NCH];
    auto fetch = [&](int base, u32x4 (&kx)[NCH], u32x4 (&vx)[NCH]) {
        const int key = base + grp;
        const int kk = key < kend ? key : kend - 1;
        const half_t *kp = kb + (long)kk * p.ks[1], *vp = vb + (long)kk * p.vs[1];
#pragma unroll
        for (int ci = 0; ci < NCH; ci++) {
            const int e0 = (cl + 8 * ci) * 8;
            const u32x4 z = {0u, 0u, 0u, 0u};
            kx[ci] = e0 < p.E ? ldg16(kp + e0) : z;
            vx[ci] = e0 < p.E ? ldg16(vp + e0) : z;
        }
    };
    const int base0 = kbeg + wave * 8;
    if (VEC && base0 < kend) fetch(base0, kc, vc);
    for (int base = base0; base < kend; base += 32) {
        const int key = base + grp;
        const bool live = key < kend;
        const int kk = live ? key : kend - 1;
        const half_t *kp = kb + (long)kk * p.ks[1];
        u32x4 kn[NCH], vn[NCH];
        if (VEC && base + 32 < kend) fetch(base + 32, kn, vn);
        float d = 0.0f;
#pragma unroll
        for (int ci = 0; ci < NCH; ci++) {
            const int e0 = (cl + 8 * ci) * 8;
            if (VEC) {
                half8v t = as_half8(kc[ci]);
#pragma unroll
                for (int j = 0; j < 8; j++) d = fmaf(qv[ci][j], (float)t[j], d);
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (e0 + j < p.E) d = fmaf(qv[ci][j], (float)kp[(long)(e0 + j) * p.ks[0]], d);
            }
        }
        d += lane_xor<1>(d);
        d += lane_xor<2>(d);
        d += lane_xor<4>(d);
        float sc = d * p.scale;
        if (p.bias && live) {
            const long bo = (long)kk * p.bs[0] + (long)lq * p.bs[1] + (long)h * p.bs[2] + (long)b * p.bs[3];
            sc += p.bias_f32 ? reinterpret_cast<const float *>(p.bias)[bo] : (float)reinterpret_cast<const half_t *>(p.bias)[bo];
        }
        if (!live) sc = -INFINITY;
        const float mn = fmaxf(m, sc);
        const float mu = mn == -INFINITY ? 0.0f : mn;
        const float al = __expf(m - mu);
        const float pw = __expf(sc - mu);
        l = l * al + pw;
        m = mn;
        const half_t *vp = vb + (long)kk * p.vs[1];
#pragma unroll
        for (int ci = 0; ci < NCH; ci++) {
            const int e0 = (cl + 8 * ci) * 8;
            if (VEC) {
                half8v t = as_half8(vc[ci]);
#pragma unroll
                for (int j = 0; j < 8; j++) acc[ci][j] = fmaf(pw, (float)t[j], acc[ci][j] * al);
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    float vv = e0 + j < p.E ? (float)vp[(long)(e0 + j) * p.vs[0]] : 0.0f;
                    acc[ci][j] = fmaf(pw, vv, acc[ci][j] * al);
                }
            }
        }
        if (VEC) {
#pragma unroll
            for (int ci = 0; ci < NCH; ci++) { kc[ci] = kn[ci]; vc[ci] = vn[ci]; }
        }
    }

    // merge the 8 groups of the wave
#pragma unroll
    for (int o = 8; o < 64; o <<= 1) {
        const float mo = __shfl_xor(m, o, 64), lo = __shfl_xor(l, o, 64);
        const float mn = fmaxf(m, mo);
        const float mu = mn == -INFINITY ? 0.0f : mn;
        const float a0 = __expf(m - mu), a1 = __expf(mo - mu);
        l = l * a0 + lo * a1;
#pragma unroll
        for (int ci = 0; ci < NCH; ci++)
#pragma unroll
            for (int j = 0; j < 8; j++) acc[ci][j] = acc[ci][j] * a0 + __shfl_xor(acc[ci][j], o, 64) * a1;
        m = mn;
    }
    // merge the 4 waves through LDS
    if (lane < 8) {
#pragma unroll
        for (int ci = 0; ci < NCH; ci++)
#pragma unroll
            for (int j = 0; j < 8; j++) red_o[wave][(cl + 8 * ci) * 8 + j] = acc[ci][j];
        if (lane == 0) { red_ml[wave][0] = m; red_ml[wave][1] = l; }
    }
    __syncthreads();
    if (tid < 64 * NCH && tid < p.E) {
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; w++) mm = fmaxf(mm, red_ml[w][0]);
        const float mu = mm == -INFINITY ? 0.0f : mm;
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float a = __expf(red_ml[w][0] - mu);
            L += a * red_ml[w][1];
            O += a * red_o[w][tid];
        }
        const long orow = ((long)b * p.H + h) * p.Lq + lq;
        if (p.nsplit == 1) {
            const float r = L > 0.0f ? O / L : 0.0f;
            const long oo = (long)b * p.os[3] + (long)h * p.os[2] + (long)lq * p.os[1] + (long)tid * p.os[0];
            if (p.out_f32) reinterpret_cast<float *>(p.out)[oo] = r;
            else reinterpret_cast<half_t *>(p.out)[oo] = (half_t)r;
        } else {
            const long rows = (long)p.B * p.H * p.Lq;
            p.part_o[((long)split * rows + orow) * p.E + tid] = O;
            if (tid == 0) {
                p.part_ml[((long)split * rows + orow) * 2] = mm;
                p.part_ml[((long)split * rows + orow) * 2 + 1] = L;
            }
        }
    }
}

// Single query row per (head, batch): 8-wave workgroups, `nsplit` of them per row, each over its share of the key
// range.  A wave takes keys 8 at a time (8 lanes per key, one 16-byte chunk of the head dim each) with a stride of
// 64 keys, in rounds of SD_U passes whose K and V loads are all issued before the first is used, the next round's
// before the current round is consumed: about 190 KB in flight per workgroup.
//
// Such a launch moves a few MB, so its duration is a chain of trips to memory.  Every address is therefore made
// independent of loaded data: the key range is cut by the cache's capacity (p.Lk), not by kv_len, and keys are
// requested up to the capacity -- valid memory whatever the length -- together with the length itself, the query
// and the new row; the length only masks scores afterwards.  One trip, then arithmetic.
//
// nsplit > 1: the workgroups of one row run on one XCD (workgroup ids are dealt to XCDs round robin, so ids that
// differ by multiples of 8 share an L2), write their partial (max, sum, o[E]) to part_o / part_ml, and take a ticket;
// whoever draws the last ticket merges the partials in split order -- so the result does not depend on who that
// is -- writes the row and puts the ticket counter back to zero.  Nobody waits for anybody: every workgroup exits
// after its own work.  The exchange stays inside that one L2: a partial is written with plain stores, waited for
// (vmcnt) and followed by the ticket, an atomic the L2 performs; the merging workgroup reads with loads that go to
// the L2.  A device-scope release per workgroup instead (__threadfence) writes the whole L2 back each time: measured
// 63 us for 320 workgroups against 6 us unsplit.  The host only splits on a device whose probe showed the round-robin
// placement this relies on.
constexpr int SD_U = 6;
__global__ __launch_bounds__(512) void sdpa_decode_kernel(SdpaArgs p) {
    __shared__ float red_ml[8][2];
    __shared__ float red_o[8][64];
    __shared__ int is_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int grp = lane >> 3, cl = lane & 7;
    const int S = p.nsplit;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int split = slot % S, unit = (slot / S) * 8 + xcd;
    if (unit >= p.H * p.B) return;                       // the grid is padded to whole groups of 8 rows
    const int h = unit % p.H, b = unit / p.H;
    const int cap = p.Lk;
    const int npass = (cap + 63) / 64, per = (npass + S - 1) / S;
    const int t_lo = split * per, t_hi = min(npass, t_lo + per);
    const half_t *qp = p.q + h * p.qs[2] + b * p.qs[3];
    half_t *kb = const_cast<half_t *>(p.k) + h * p.ks[2] + b * p.ks[3];
    half_t *vb = const_cast<half_t *>(p.v) + h * p.vs[2] + b * p.vs[3];
    const int e0 = cl * 8;
    const bool eok = e0 < p.E;
    const u32x4 z = {0u, 0u, 0u, 0u};
    const int n_raw = p.kv_len ? p.kv_len[b] : cap;
    u32x4 kc[2][SD_U], vc[2][SD_U];
    // pass t of this wave covers keys 64 t + 8 wave + grp
    auto fetch = [&](int set, int t0) {
#pragma unroll
        for (int u = 0; u < SD_U; u++) {
            const int kk = min(64 * (t0 + u) + 8 * wave + grp, cap - 1);
            const bool on = eok && t0 + u < t_hi;
            kc[set][u] = on ? ldg16(kb + (long)kk * p.ks[1] + e0) : z;
            vc[set][u] = on ? ldg16(vb + (long)kk * p.vs[1] + e0) : z;
        }
    };
    if (t_lo < t_hi) fetch(0, t_lo);
    if (t_lo + SD_U < t_hi) fetch(1, t_lo + SD_U);
    u32x4 kn = z, vn = z;                                // the row that this step appends
    if (p.k_new && eok) {
        kn = ldg16(p.k_new + h * p.ns[2] + b * p.ns[3] + e0);
        vn = ldg16(p.v_new + h * p.ns[2] + b * p.ns[3] + e0);
    }
    float qv[8];
    {
        const half8v t = as_half8(eok ? ldg16(qp + e0) : z);
#pragma unroll
        for (int j = 0; j < 8; j++) qv[j] = (float)t[j] * p.scale;
    }
    // a length past the capacity: the cache is full, the new row is neither stored nor attended
    const int Lk = max(0, min(cap, n_raw));
    const int fresh = p.k_new && n_raw <= cap ? Lk - 1 : -1;
    float m = -INFINITY, l = 0.0f, acc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] = 0.0f;
    auto consume = [&](int set, int t0) {
#pragma unroll
        for (int u = 0; u < SD_U; u++) {
            if (t0 + u < t_hi && 64 * (t0 + u) < Lk) {           // uniform: the shuffles below need the whole wave
                const int key = 64 * (t0 + u) + 8 * wave + grp;
                u32x4 kr = kc[set][u], vr = vc[set][u];
                if (key == fresh) {                              // exactly eight lanes of one workgroup own it
                    kr = kn; vr = vn;
                    if (eok) {
                        *reinterpret_cast<u32x4 *>(kb + (long)key * p.ks[1] + e0) = kn;
                        *reinterpret_cast<u32x4 *>(vb + (long)key * p.vs[1] + e0) = vn;
                    }
                }
                const half8v kt = as_half8(kr), vt = as_half8(vr);
                float d = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; j++) d = fmaf(qv[j], (float)kt[j], d);
                d += lane_xor<1>(d);
                d += lane_xor<2>(d);
                d += lane_xor<4>(d);
                const float sc = key < Lk ? d : -INFINITY;
                const float mn = fmaxf(m, sc);
                const float mu = mn == -INFINITY ? 0.0f : mn;
                const float al = __expf(m - mu), pw = __expf(sc - mu);
                l = l * al + pw;
                m = mn;
#pragma unroll
                for (int j = 0; j < 8; j++) acc[j] = fmaf(pw, (float)vt[j], acc[j] * al);
            }
        }
    };
    for (int t0 = t_lo; t0 < t_hi; t0 += 2 * SD_U) {
        consume(0, t0);
        if (t0 + 2 * SD_U < t_hi) fetch(0, t0 + 2 * SD_U);
        if (t0 + SD_U < t_hi) consume(1, t0 + SD_U);
        if (t0 + 3 * SD_U < t_hi) fetch(1, t0 + 3 * SD_U);
    }
    // merge the 8 groups of the wave, then the 8 waves through LDS (flash.jl:1385-1391)
#pragma unroll
    for (int o = 8; o < 64; o <<= 1) {
        const float mo = __shfl_xor(m, o, 64), lo = __shfl_xor(l, o, 64);
        const float mn = fmaxf(m, mo);
        const float mu = mn == -INFINITY ? 0.0f : mn;
        const float a0 = __expf(m - mu), a1 = __expf(mo - mu);
        l = l * a0 + lo * a1;
#pragma unroll
        for (int j = 0; j < 8; j++) acc[j] = acc[j] * a0 + __shfl_xor(acc[j], o, 64) * a1;
        m = mn;
    }
    if (lane < 8) {
#pragma unroll
        for (int j = 0; j < 8; j++) red_o[wave][cl * 8 + j] = acc[j];
        if (lane == 0) { red_ml[wave][0] = m; red_ml[wave][1] = l; }
    }
    __syncthreads();
    float mm = -INFINITY, L = 0.0f, O = 0.0f;
    if (tid < 64) {
#pragma unroll
        for (int w = 0; w < 8; w++) mm = fmaxf(mm, red_ml[w][0]);
        const float mu = mm == -INFINITY ? 0.0f : mm;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const float a = __expf(red_ml[w][0] - mu);
            L += a * red_ml[w][1];
            O += a * red_o[w][tid];
        }
    }
    if (S > 1) {                                         // uniform
        const long row = (long)unit * S + split;
        if (tid < p.E) p.part_o[row * p.E + tid] = O;
        if (tid == 0) { p.part_ml[row * 2] = mm; p.part_ml[row * 2 + 1] = L; }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's part of the partial has reached the L2 ...
        __syncthreads();                                  // ... and so has everybody's, before the ticket is drawn
        if (tid == 0) {
            const unsigned t = __hip_atomic_fetch_add(p.tickets + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = t == (unsigned)(S - 1);
            if (is_last) __hip_atomic_store(p.tickets + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
        }
        __syncthreads();
        if (!is_last) return;
        mm = -INFINITY; L = 0.0f; O = 0.0f;
        if (tid < p.E) {
            const long r0 = (long)unit * S;
            for (int s0 = 0; s0 < S; s0 += 8) {
                float ms[8], ls[8], os_[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const long r = r0 + min(s0 + j, S - 1);
                    // read at the L2, past this compute unit's own cache
                    ms[j] = s0 + j < S ? __hip_atomic_load(p.part_ml + r * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -INFINITY;
                    ls[j] = __hip_atomic_load(p.part_ml + r * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    os_[j] = __hip_atomic_load(p.part_o + r * p.E + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                float mb = mm;
#pragma unroll
                for (int j = 0; j < 8; j++) mb = fmaxf(mb, ms[j]);
                const float mu = mb == -INFINITY ? 0.0f : mb;
                const float a0 = __expf(mm - mu);
                L *= a0; O *= a0;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float a = __expf(ms[j] - mu);  // a split past the end has m = -inf: weight 0
                    L += a * ls[j];
                    O += a * os_[j];
                }
                mm = mb;
            }
        }
    }
    if (tid < p.E) {
        const float r = L > 0.0f ? O / L : 0.0f;
        const long oo = (long)b * p.os[3] + (long)h * p.os[2] + (long)tid * p.os[0];
        if (p.out_f32) reinterpret_cast<float *>(p.out)[oo] = r;
        else reinterpret_cast<half_t *>(p.out)[oo] = (half_t)r;
    }
}

// One thread per (row, e): merges the key splits (attn_flash_cm_merge!, flash.jl:1398-1421).
__global__ void sdpa_merge_kernel(SdpaArgs p) {
    const long rows = (long)p.B * p.H * p.Lq;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * p.E) return;
    const long row = idx / p.E;
    const int e = (int)(idx % p.E);
    // Splits are taken eight at a time with every load of a batch issued before the first is used;
    // the running maximum is carried from batch to batch by the rescaling identity.
    float mm = -INFINITY, L = 0.0f, O = 0.0f;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float ms[8], ls[8], os_[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = min(s0 + j, p.nsplit - 1);
            const float2v ml = *reinterpret_cast<const float2v *>(p.part_ml + ((long)s * rows + row) * 2);
            ms[j] = s0 + j < p.nsplit ? ml[0] : -INFINITY;
            ls[j] = ml[1];
            os_[j] = p.part_o[((long)s * rows + row) * p.E + e];
        }
        float mb = mm;
#pragma unroll
        for (int j = 0; j < 8; j++) mb = fmaxf(mb, ms[j]);
        const float mu = mb == -INFINITY ? 0.0f : mb;
        const float a0 = __expf(mm - mu);
        L *= a0; O *= a0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float a = __expf(ms[j] - mu);     // a split past the end has m = -inf: weight 0
            L += a * ls[j];
            O += a * os_[j];
        }
        mm = mb;
    }
    const float r = L > 0.0f ? O / L : 0.0f;
    const long lq = row % p.Lq, hb = row / p.Lq, h = hb % p.H, b = hb / p.H;
    const long oo = b * p.os[3] + h * p.os[2] + lq * p.os[1] + (long)e * p.os[0];
    if (p.out_f32) reinterpret_cast<float *>(p.out)[oo] = r;
    else reinterpret_cast<half_t *>(p.out)[oo] = (half_t)r;
}

// ------------------------------------------------------------------------------------------
constexpr int flash_lds_bytes(int EP) { return 3 * 64 * (EP + 8) * 2 + 3 * 64 * flash_vld(EP) * 2; }
// A mask that depends on the key only rides in LDS behind the stages: whole key blocks (of `bcs` keys) and one zero
constexpr int FLASH_KEYMASK_MAX = 4096;
constexpr int flash_keymask_bytes(int64_t Lk, int bcs) { return (int)(((Lk + bcs - 1) / bcs * bcs + 1) * 2 + 15) / 16 * 16; }
constexpr int flash_short_lds_bytes(int NW) { return NW * 64 * flash_vld(64) * 2; }
constexpr int flash_pair_lds_bytes() { return 4 * (64 * (64 + 8) * 2 + 64 * flash_vld(64) * 2); }

bool vec_addressable(const half_t *ptr, const long st[4], int E) {
    return st[0] == 1 && E % 8 == 0 && st[1] % 8 == 0 && st[2] % 8 == 0 && st[3] % 8 == 0 && aligned_to(ptr, 16);
}

int rows_splits(int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    // Aim at two workgroups per compute unit, as the reference's splitcount does (flash.jl:1288-1303); a split is
    // at least 64 keys.  The wanted count is rounded up and not re-derived from equal chunks: the reference's
    // rounding gives 3 splits instead of 4 for 160 rows over 1500 keys and measured 20.0 us against 17.7 us.
    int64_t rows = Lq * H * B;
    if (rows <= 0) return 1;
    int64_t want = ceil_div(2 * (int64_t)mi_num_cus(), rows);
    int64_t maxs = ceil_div(Lk, 64);
    if (want > maxs) want = maxs;
    if (want < 1) want = 1;
    if (want > 64) want = 64;
    return (int)want;
}

// Between 8 and 63 queries over a long key range -- the reference's flash-decoding case, 23 queries over 4096 keys
// (SAM 2.1's mask decoder attending the image; flash.jl:1288-1303, kernelplans.jl:300-312): one 128-query tile per
// (head, batch) of the fused kernel with the keys cut over workgroups, two workgroups per compute unit as the
// reference's splitcount aims for, every split at least four 64-key blocks; sdpa_merge_kernel joins the partials.
// (One workgroup per query row -- sdpa_rows_kernel -- re-reads K and V once per row.)
// Only while the (head, batch) tiles alone leave the chip mostly idle: beyond that a workgroup per query row fills it.
bool flash_few_queries(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    return Lq >= 8 && Lq < 64 && Lk >= 512 && E <= 128 && H * B * 2 <= (int64_t)mi_num_cus();
}
int few_query_splits(int64_t Lk, int64_t H, int64_t B) {
    const int64_t tiles = H * B, blocks = ceil_div(Lk, 64);
    int64_t want = ceil_div(2 * (int64_t)mi_num_cus(), tiles);
    if (want > blocks / 4) want = blocks / 4;
    if (want > 32) want = 32;
    if (want < 1) want = 1;
    while (want > 1 && ceil_div(blocks, want) * (want - 1) >= blocks) want--;      // no empty split
    return (int)want;
}

// Key splits for the fused kernel.  A workgroup spends about 1 us per 64-key block plus 3 us of start-up,
// and the merge is a second launch of about 6 us, so splitting pays only when the query blocks leave most
// of the chip idle and every split still walks a dozen blocks (config 3's 66 workgroups x 22 blocks do
// not: 21.9 us unsplit, 21.1 us at best split three ways).
int flash_splits_over_workgroups(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B);

// Head sizes 65 .. 96 over 1024 keys or more, at most one 128-query workgroup per CU: the eight-wave key-halves form at
// 96 wide (two waves per SIMD in ping-pong, no second launch) where the grid covers more than half of the chip or the
// keys would not be split over workgroups anyway -- 8 heads x 4096 x 72 (the reference's SAM 2.1 global attention):
// 87.8 us as two key splits + merge launch, 76.0 us so; 12 heads x 1024 x 80: 28.8 -> 25.1 us.  Shorter key ranges stay
// with four waves (16 windows x 8 heads x 256 x 72: 13.4 us against 16.0 us).
bool flash_halves96(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    const int64_t wgs = ceil_div(Lq, 128) * H * B, cus = mi_num_cus();
    if (E <= 64 || E > 96 || Lk < 1024 || wgs > cus) return false;
    return wgs * 2 > cus || flash_splits_over_workgroups(E, Lq, Lk, H, B) == 1;
}

int flash_splits(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    if (flash_few_queries(E, Lq, Lk, H, B)) return few_query_splits(Lk, H, B);
    return flash_halves96(E, Lq, Lk, H, B) ? 1 : flash_splits_over_workgroups(E, Lq, Lk, H, B);
}

int flash_splits_over_workgroups(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    const int64_t wgs = ceil_div(Lq, 128) * H * B, cus = mi_num_cus();
    // At head size 64 a grid of up to one workgroup per CU runs the eight-wave key-halves variant instead; wider
    // heads have no such variant, and two workgroups per CU is what gives their SIMDs a second wave.
    if (E <= 64 ? wgs * 2 > cus : wgs > cus) return 1;
    int64_t want = ceil_div(cus * 3 / 2, wgs);
    const int64_t blocks = ceil_div(Lk, 64);
    if (want > blocks / 12) want = blocks / 12;
    if (want > 16) want = 16;
    if (want < 2) return 1;
    // no empty split: with `per` blocks each, the last one must still start inside the keys
    while (want > 1 && ceil_div(blocks, want) * (want - 1) >= blocks) want--;
    return (int)want;
}

// Head size 64, no mask, and at most about one 32-query workgroup per compute unit: flash_short_kernel, unless key
// splits over workgroups are estimated faster still (a handful of tiles over thousands of keys).  A SIMD finishes a 32 x 64 block of it in
// about 1.3 us whether it holds one of its waves or two, so what counts is that every SIMD gets one wave: 6 heads x 1344
// (252 workgroups) 18.5 -> 11.8 us, 12 heads x 577 12.3 -> 7.6 us, 4 heads x 640 over 300 keys 10.6 -> 6.3 us; at 6
// heads x 1370 two CUs of 256 hold two workgroups, which then take twice as long (17.6 us against 18.5 us), and
// beyond that the 128-query forms are as fast or faster.
bool flash_short(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    const int64_t tiles = ceil_div(Lq, 32) * H * B, cus = mi_num_cus();
    if (E != 64 || Lk < 128 || tiles > cus + cus / 16) return false;
    // against key splits over workgroups (few tiles, many keys): 4.5 us + 1.3 us per block of a wave's quarter here,
    // 3 us + 1 us per block of a split + the 6 us merge launch there
    const int64_t blocks = ceil_div(Lk, 64), ns = flash_splits(E, Lq, Lk, H, B);
    return ns == 1 || 4.5 + 1.3 * (double)ceil_div(blocks, 4) <= 9.0 + 1.0 * (double)ceil_div(blocks, ns);
}

// The same on 64-query tiles (flash_pair_kernel) where the 32-query tiles would not all find a CU of their own but the
// 64-query tiles do.  Replayed, against what ran there before (key halves on 128-query tiles, or 32-query tiles two to a
// CU): 6 heads x 1370 17.8 -> 14.3 us, 16 x 1024 15.8 -> 11.3, 10 x 1500 26.5 -> 14.8, 8 x 2048 31.1 -> 19.6, 6 x 2500
// 34.5 -> 21.1, 4 x 4096 44.1 -> 30.0; where the 32-query tiles fit they are faster (6 x 1344 11.7 against 13.4 us), and
// at 12 x 1370 (264 tiles of 64) the key-halves form is (19.4 against 26.5 us).
bool flash_pair(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    const int64_t tiles32 = ceil_div(Lq, 32) * H * B, tiles64 = ceil_div(Lq, 64) * H * B, cus = mi_num_cus();
    return E == 64 && Lk >= 128 && tiles32 > cus && tiles64 <= cus;
}
// either of the two: one launch, keys not split over workgroups
bool flash_unsplit(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B) {
    return !flash_few_queries(E, Lq, Lk, H, B) && (flash_pair(E, Lq, Lk, H, B) || flash_short(E, Lq, Lk, H, B));
}

// A single query row (a decode step) runs in one launch of sdpa_decode_kernel: the work follows the device-side kv_len
// and the cache write can ride along (mi_sdpa_append_f16).  Twenty heads alone leave most of the chip idle and give each
// workgroup a long chain of keys, so a long key range is cut over several workgroups per row -- at most one workgroup
// per compute unit, a round of six 64-key passes each -- which merge inside the launch.  Head dim <= 64, 16-byte addressable
// operands, no additive mask; the rest goes to sdpa_rows_kernel (+ sdpa_merge_kernel).
constexpr int SD_BANKS = 16, SD_TICKETS = 4096, SD_PART_FLOATS = 1 << 16;
// Arrival counters and partials of the split form: a launch takes the next of SD_BANKS banks, so launches in flight
// together on one GPU (up to SD_BANKS of them) do not touch each other's.  Zero when the module loads; every launch
// leaves its counters at zero.
static __device__ unsigned sd_ticket_words[SD_BANKS * SD_TICKETS];
static __device__ __align__(256) float sd_part_words[SD_BANKS * SD_PART_FLOATS];
constexpr int SD_MAX_DEVICES = 64;
unsigned *g_sd_tickets[SD_MAX_DEVICES] = {};
float *g_sd_parts[SD_MAX_DEVICES] = {};
std::atomic<unsigned> g_sd_launch{0};

bool one_pass_decode(const SdpaArgs &a, bool vec) {
    return a.Lq == 1 && vec && !a.bias && a.E <= 64 && a.Lk >= 1 && (int64_t)a.H * a.B <= SD_TICKETS;
}

int decode_splits(int64_t E, int64_t Lk, int64_t H, int64_t B) {
    const int64_t units = H * B, passes = ceil_div(Lk, 64);
    // The exchange adds about 3 us of its own (partial out, ticket, partials in: three trips in a row), a workgroup
    // walks six passes in about one trip: 448 keys stay whole (5.9 us either way at batch 1), 1500 keys are cut
    // four ways at batch 1 (11.1 us whole, 7.2 us cut in 4, 10.2 us cut in 12) and three ways at batch 4.
    int64_t want = mi_num_cus() / units;                 // at most one workgroup per compute unit
    if (want > ceil_div(passes, SD_U)) want = ceil_div(passes, SD_U);      // one round of passes each
    if (passes <= 8) want = 1;
    if (want > 32) want = 32;
    while (want > 1 && units * want * (E + 2) > SD_PART_FLOATS) want--;
    if (want < 1) want = 1;
    // no empty split: with `per` passes each, the last one must still start inside the range
    while (want > 1 && ceil_div(passes, want) * (want - 1) >= passes) want--;
    return (int)want;
}

// Fills in the split count and, for a split launch, this launch's bank of counters and partials, and launches.
int launch_decode(SdpaArgs &a, hipStream_t st) {
    a.nsplit = decode_splits(a.E, a.Lk, a.H, a.B);
    if (a.nsplit > 1) {
        int dev = -1;
        if (!mi_xcd_round_robin() || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SD_MAX_DEVICES || !g_sd_tickets[dev]) a.nsplit = 1;
        else {
            const unsigned bank = g_sd_launch++ % SD_BANKS;
            a.tickets = g_sd_tickets[dev] + (size_t)bank * SD_TICKETS;
            a.part_o = g_sd_parts[dev] + (size_t)bank * SD_PART_FLOATS;
            a.part_ml = a.part_o + (size_t)a.H * a.B * a.nsplit * a.E;
        }
    }
    const unsigned units8 = (unsigned)ceil_div((int64_t)a.H * a.B, 8);
    hipLaunchKernelGGL(sdpa_decode_kernel, dim3(units8 * 8 * a.nsplit), dim3(512), 0, st, a);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

// A mask the fused kernel can carry: keys contiguous (a lane reads runs of four), the other axes any stride including
// broadcast; fp16 runs are read as two dwords, so every row must start on a 4-byte boundary.  An fp16 mask with the
// query axis broadcast has no such conditions.
bool flash_bias_ok(const SdpaArgs &a) {
    if (!a.bias_f32 && (a.bs[1] == 0 || a.Lq == 1) && a.Lk <= FLASH_KEYMASK_MAX) return aligned_to(a.bias, 2);      // the same for every query: copied to LDS a value at a time
    if (a.bs[0] != 1 && a.Lk != 1) return false;
    if (a.bias_f32) return aligned_to(a.bias, 4);
    return aligned_to(a.bias, 4) && a.bs[1] % 2 == 0 && a.bs[2] % 2 == 0 && a.bs[3] % 2 == 0;
}

int sdpa_path(const SdpaArgs &a) {
    if (a.E < 1 || a.E > 256 || a.Lq < 0 || a.Lk < 0 || a.H < 1 || a.B < 1) return MI_SDPA_DECLINE;
    if (a.H > 65535 || a.B > 65535 || (int64_t)a.Lq * a.H * 64 > INT32_MAX) return MI_SDPA_DECLINE;
    bool vec = vec_addressable(a.q, a.qs, a.E) && vec_addressable(a.k, a.ks, a.E) && vec_addressable(a.v, a.vs, a.E);
    bool out_ok = (aligned_to(a.out, 16) || a.out == nullptr) && a.os[0] == 1 && a.os[1] % 8 == 0 && a.os[2] % 8 == 0 && a.os[3] % 8 == 0;
    const bool enough_queries = a.Lq >= 64 || (!a.bias && flash_few_queries(a.E, a.Lq, a.Lk, a.H, a.B));
    if (mi_plan_mfma() && vec && out_ok && (!a.bias || flash_bias_ok(a)) && a.scale > 0.0f && a.E <= 128 && enough_queries && a.Lk >= 1) return MI_SDPA_FLASH;
    return MI_SDPA_ROWS;
}

int fill(SdpaArgs &a, void *out, int out_dtype, const int64_t *os, const void *q, const int64_t *qs, const void *k, const int64_t *ks,
         const void *v, const int64_t *vs, const void *bias, int bias_dtype, const int64_t *bs, const int32_t *kv_len,
         int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale) {
    if (!q || !k || !v || !qs || !ks || !vs) return MI_DECLINE_OPERANDS;
    if (bias && !bs) return MI_DECLINE_BIAS;
    if (out_dtype != MI_F16 && out_dtype != MI_F32) return MI_DECLINE_OPERANDS;
    if (E > INT32_MAX || Lq > INT32_MAX || Lk > INT32_MAX || H > INT32_MAX || B > INT32_MAX) return MI_DECLINE_EXTENT;
    a.out = out; a.q = (const half_t *)q; a.k = (const half_t *)k; a.v = (const half_t *)v;
    for (int i = 0; i < 4; i++) { a.qs[i] = qs[i]; a.ks[i] = ks[i]; a.vs[i] = vs[i]; a.bs[i] = bias ? bs[i] : 0; }
    if (os) { for (int i = 0; i < 4; i++) a.os[i] = os[i]; }
    else { a.os[0] = 1; a.os[1] = E; a.os[2] = E * Lq; a.os[3] = E * Lq * H; }
    a.bias = bias; a.bias_f32 = bias_dtype == MI_F32; a.kv_len = kv_len;
    a.part_o = a.part_ml = nullptr;
    a.tickets = nullptr;
    a.k_new = a.v_new = nullptr;
    for (int i = 0; i < 4; i++) a.ns[i] = 0;
    a.E = (int)E; a.Lq = (int)Lq; a.Lk = (int)Lk; a.H = (int)H; a.B = (int)B;
    a.out_f32 = out_dtype == MI_F32; a.nsplit = 1; a.scale = scale;
    return MI_OK;
}

template <int NCH>
void launch_rows(const SdpaArgs &a, bool vec, dim3 grid, hipStream_t st) {
    if (vec) hipLaunchKernelGGL((sdpa_rows_kernel<NCH, true>), grid, dim3(256), 0, st, a);
    else     hipLaunchKernelGGL((sdpa_rows_kernel<NCH, false>), grid, dim3(256), 0, st, a);
}

}  // namespace

// Called once from mi_init: the 128-wide head-dim variant needs more than the
// default 64 KiB of dynamic LDS.
int mi_sdpa_init() {
    int bad = 0;
    {   // this device's copies of the decode kernel's counters and partials (zeroed at load; never named in host code again)
        int dev = -1;
        void *t = nullptr, *pw = nullptr;
        if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < SD_MAX_DEVICES &&
            hipGetSymbolAddress(&t, HIP_SYMBOL(sd_ticket_words)) == hipSuccess && hipGetSymbolAddress(&pw, HIP_SYMBOL(sd_part_words)) == hipSuccess) {
            g_sd_tickets[dev] = reinterpret_cast<unsigned *>(t);
            g_sd_parts[dev] = reinterpret_cast<float *>(pw);
        }
    }
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, false>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, true>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, true, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, 2 * flash_lds_bytes(64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, true, 2, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, 2 * flash_lds_bytes(64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<96, true, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, 2 * flash_lds_bytes(96)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_short_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_short_lds_bytes(4)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_pair_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, flash_pair_lds_bytes()) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<96, false>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(96)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<128, false>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(128)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, false, 1, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, false, 1, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<96, false, 1, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(96)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<96, false, 1, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(96)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<128, false, 1, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(128)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<128, false, 1, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(128)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, true, 2, 3>), hipFuncAttributeMaxDynamicSharedMemorySize, 2 * flash_lds_bytes(64) + flash_keymask_bytes(FLASH_KEYMASK_MAX, 128)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, false, 1, 3>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(64) + flash_keymask_bytes(FLASH_KEYMASK_MAX, 64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<64, true, 1, 3>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(64) + flash_keymask_bytes(FLASH_KEYMASK_MAX, 64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<96, false, 1, 3>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(96) + flash_keymask_bytes(FLASH_KEYMASK_MAX, 64)) != hipSuccess;
    bad |= hipFuncSetAttribute(reinterpret_cast<const void *>(flash_fwd_kernel<128, false, 1, 3>), hipFuncAttributeMaxDynamicSharedMemorySize, flash_lds_bytes(128) + flash_keymask_bytes(FLASH_KEYMASK_MAX, 64)) != hipSuccess;
    return bad;
}

extern "C" {

size_t mi_sdpa_f16_workspace(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, int has_bias) {
    // sized for the path the call will most likely take: the fused kernel's key splits for Lq >= 64 without
    // an additive mask (unused if the operands turn out not to be 16-byte addressable), the rows kernel's below
    int ns = Lq >= 64 ? ((has_bias || flash_unsplit(E, Lq, Lk, H, B)) ? 1 : flash_splits(E, Lq, Lk, H, B)) : rows_splits(Lq, Lk, H, B);
    // few queries over many keys: whichever of the two routes the operands allow must find its partials' room
    if (!has_bias && flash_few_queries(E, Lq, Lk, H, B) && few_query_splits(Lk, H, B) > ns) ns = few_query_splits(Lk, H, B);
    if (ns <= 1) return 0;
    size_t rows = (size_t)Lq * H * B;
    return round_up((size_t)ns * rows * E * sizeof(float), 256) + round_up((size_t)ns * rows * 2 * sizeof(float), 256);
}

int mi_sdpa_f16_plan(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                     const void *v, const int64_t v_strides[4], int has_bias, int has_kv_len,
                     int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale, int *nsplit_out) {
    (void)has_kv_len;
    SdpaArgs a;
    static const int64_t zero4[4] = {0, 0, 0, 0};
    // a mask is planned as a dense fp16 (Lk, Lq, H, B) array: what an exported graph hands over
    const int64_t dense4[4] = {1, Lk, Lk * Lq, Lk * Lq * H};
    int rc = fill(a, nullptr, MI_F16, nullptr, q, q_strides, k, k_strides, v, v_strides, has_bias ? (const void *)q : nullptr, MI_F16,
                  has_bias ? dense4 : zero4, nullptr, E, Lq, Lk, H, B, scale);
    if (rc != MI_OK) return MI_SDPA_DECLINE;
    int path = sdpa_path(a);
    const bool vec = vec_addressable(a.q, a.qs, a.E) && vec_addressable(a.k, a.ks, a.E) && vec_addressable(a.v, a.vs, a.E);
    if (nsplit_out) *nsplit_out = (path == MI_SDPA_ROWS && Lq < 64) ? (one_pass_decode(a, vec) ? decode_splits(E, Lk, H, B) : rows_splits(Lq, Lk, H, B))
                                  : (path == MI_SDPA_FLASH && !has_bias && !flash_unsplit(E, Lq, Lk, H, B)) ? flash_splits(E, Lq, Lk, H, B) : 1;
    return path;
}

int mi_sdpa_f16_plan_caps(const int64_t caps[6], const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                          const void *v, const int64_t v_strides[4], int has_bias, int has_kv_len,
                          int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale, int *nsplit_out) {
    mi_plan_caps_begin(caps);
    const int path = mi_sdpa_f16_plan(q, q_strides, k, k_strides, v, v_strides, has_bias, has_kv_len, E, Lq, Lk, H, B, scale, nsplit_out);
    mi_plan_caps_end();
    return path;
}

int mi_sdpa_f16(void *out, int out_dtype, const int64_t out_strides[4],
                const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                const void *v, const int64_t v_strides[4],
                const void *bias, int bias_dtype, const int64_t bias_strides[4], const int32_t *kv_len,
                int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale,
                void *ws, size_t ws_bytes, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out) return MI_DECLINE_OPERANDS;
    SdpaArgs a;
    int rc = fill(a, out, out_dtype, out_strides, q, q_strides, k, k_strides, v, v_strides, bias, bias_dtype, bias_strides, kv_len, E, Lq, Lk, H, B, scale);
    if (rc != MI_OK) return rc;
    if (Lq == 0 || H == 0 || B == 0 || E == 0) return MI_OK;
    hipStream_t st = (hipStream_t)stream;
    int path = sdpa_path(a);
    if (path == MI_SDPA_DECLINE) return MI_DECLINE_EXTENT;
    if (path == MI_SDPA_FLASH) {
        // The 8-wave ping-pong kernel when 256-query workgroups still cover most of the chip.
        const bool pp = !a.bias && E <= 64 && ceil_div(Lq, 256) * H * B * 4 >= (int64_t)mi_num_cus() * 3;
        if (a.bias) {
            // the mask rides in the four-wave form, keys unsplit
            a.nsplit = 1;
            dim3 grid((unsigned)ceil_div(Lq, 128), (unsigned)H, (unsigned)B);
            const bool f32 = a.bias_f32 != 0;
            const bool halves = E <= 64 && ceil_div(Lq, 128) * H * B <= (int64_t)mi_num_cus() && Lk >= 256;
            // an fp16 mask that is the same for every query (a padding mask, a per-head key bias) enters with the first
            // product's extra k-step and costs no vector work
            if (!f32 && (a.bs[1] == 0 || Lq == 1) && Lk <= FLASH_KEYMASK_MAX) {
                const int m64 = flash_keymask_bytes(Lk, 64), m128 = flash_keymask_bytes(Lk, 128);
                // (the 256-query ping-pong form on the grids that run it unmasked: its first product, seeded with the
                // reference point, gets the extra k-step for the mask alone)
                if (E <= 64 && ceil_div(Lq, 256) * H * B * 4 >= (int64_t)mi_num_cus() * 3) {
                    grid = dim3((unsigned)ceil_div(Lq, 256), (unsigned)H, (unsigned)B);
                    hipLaunchKernelGGL((flash_fwd_kernel<64, true, 1, 3>), grid, dim3(512), flash_lds_bytes(64) + m64, st, a);
                }
                else if (halves)  hipLaunchKernelGGL((flash_fwd_kernel<64, true, 2, 3>), grid, dim3(512), 2 * flash_lds_bytes(64) + m128, st, a);
                else if (E <= 64) hipLaunchKernelGGL((flash_fwd_kernel<64, false, 1, 3>), grid, dim3(256), flash_lds_bytes(64) + m64, st, a);
                else if (E <= 96) hipLaunchKernelGGL((flash_fwd_kernel<96, false, 1, 3>), grid, dim3(256), flash_lds_bytes(96) + m64, st, a);
                else              hipLaunchKernelGGL((flash_fwd_kernel<128, false, 1, 3>), grid, dim3(256), flash_lds_bytes(128) + m64, st, a);
            }
            // an fp16 mask on a grid of at most one workgroup per CU: the key-halves form carries it too
            else if (halves && !f32)
                hipLaunchKernelGGL((flash_fwd_kernel<64, true, 2, 1>), grid, dim3(512), 2 * flash_lds_bytes(64), st, a);
            else if (E <= 64) { if (f32) hipLaunchKernelGGL((flash_fwd_kernel<64, false, 1, 2>), grid, dim3(256), flash_lds_bytes(64), st, a);
                                else     hipLaunchKernelGGL((flash_fwd_kernel<64, false, 1, 1>), grid, dim3(256), flash_lds_bytes(64), st, a); }
            else if (E <= 96) { if (f32) hipLaunchKernelGGL((flash_fwd_kernel<96, false, 1, 2>), grid, dim3(256), flash_lds_bytes(96), st, a);
                                else     hipLaunchKernelGGL((flash_fwd_kernel<96, false, 1, 1>), grid, dim3(256), flash_lds_bytes(96), st, a); }
            else              { if (f32) hipLaunchKernelGGL((flash_fwd_kernel<128, false, 1, 2>), grid, dim3(256), flash_lds_bytes(128), st, a);
                                else     hipLaunchKernelGGL((flash_fwd_kernel<128, false, 1, 1>), grid, dim3(256), flash_lds_bytes(128), st, a); }
        } else if (pp) {
            dim3 grid((unsigned)ceil_div(Lq, 256), (unsigned)H, (unsigned)B);
            hipLaunchKernelGGL((flash_fwd_kernel<64, true>), grid, dim3(512), flash_lds_bytes(64), st, a);
        } else if (!flash_few_queries(E, Lq, Lk, H, B) && flash_pair(E, Lq, Lk, H, B)) {
            a.nsplit = 1;
            dim3 grid((unsigned)ceil_div(Lq, 64), (unsigned)H, (unsigned)B);
            hipLaunchKernelGGL(flash_pair_kernel, grid, dim3(512), flash_pair_lds_bytes(), st, a);
        } else if (!flash_few_queries(E, Lq, Lk, H, B) && flash_short(E, Lq, Lk, H, B)) {
            a.nsplit = 1;
            dim3 grid((unsigned)ceil_div(Lq, 32), (unsigned)H, (unsigned)B);
            hipLaunchKernelGGL(flash_short_kernel<4>, grid, dim3(256), flash_short_lds_bytes(4), st, a);
        } else {
            // few query blocks: split the keys over workgroups too, if the caller brought the workspace for it
            a.nsplit = flash_splits(E, Lq, Lk, H, B);
            const size_t rows = (size_t)Lq * H * B;
            const size_t o_bytes = round_up((size_t)a.nsplit * rows * E * sizeof(float), 256);
            if (a.nsplit > 1 && ws && aligned_to(ws, 256) && ws_bytes >= o_bytes + round_up((size_t)a.nsplit * rows * 2 * sizeof(float), 256)) {
                a.part_o = reinterpret_cast<float *>(ws);
                a.part_ml = reinterpret_cast<float *>(reinterpret_cast<char *>(ws) + o_bytes);
            } else {
                a.nsplit = 1;
            }
            dim3 grid((unsigned)(ceil_div(Lq, 128) * a.nsplit), (unsigned)H, (unsigned)B);
            // no CU would hold two workgroups anyway: eight waves per workgroup, each with half of the keys
            // (head size 64 only: the 96-wide instance of this variant measured slower than four waves, 115 us
            // against 106 us on 8 heads x 4096 x 72)
            const bool halves = E <= 64 && a.nsplit == 1 && ceil_div(Lq, 128) * H * B <= (int64_t)mi_num_cus() && Lk >= 256;
            // (its two key-half groups in ping-pong: 25.1 -> 23.8 us on 20 heads x 1500, 20.1 -> 19.4 us on 6 heads x 1370)
            if (halves)       hipLaunchKernelGGL((flash_fwd_kernel<64, true, 2>), grid, dim3(512), 2 * flash_lds_bytes(64), st, a);
            else if (a.nsplit == 1 && flash_halves96(E, Lq, Lk, H, B))
                hipLaunchKernelGGL((flash_fwd_kernel<96, true, 2>), grid, dim3(512), 2 * flash_lds_bytes(96), st, a);
            else if (E <= 64) hipLaunchKernelGGL((flash_fwd_kernel<64, false>), grid, dim3(256), flash_lds_bytes(64), st, a);
            else if (E <= 96) hipLaunchKernelGGL((flash_fwd_kernel<96, false>), grid, dim3(256), flash_lds_bytes(96), st, a);
            else         hipLaunchKernelGGL((flash_fwd_kernel<128, false>), grid, dim3(256), flash_lds_bytes(128), st, a);
            if (a.nsplit > 1) {
                const long total = (long)Lq * H * B * E;
                hipLaunchKernelGGL(sdpa_merge_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, a);
            }
        }
        return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
    }
    // rows path
    bool vec = vec_addressable(a.q, a.qs, a.E) && vec_addressable(a.k, a.ks, a.E) && vec_addressable(a.v, a.vs, a.E);
    if (one_pass_decode(a, vec)) return launch_decode(a, st);
    a.nsplit = Lq < 64 ? rows_splits(Lq, Lk, H, B) : 1;
    if (a.nsplit > 1) {
        size_t rows = (size_t)Lq * H * B;
        size_t o_bytes = round_up((size_t)a.nsplit * rows * E * sizeof(float), 256);
        size_t need = o_bytes + round_up((size_t)a.nsplit * rows * 2 * sizeof(float), 256);
        if (!ws || ws_bytes < need || !aligned_to(ws, 256)) return MI_DECLINE_WORKSPACE;
        a.part_o = reinterpret_cast<float *>(ws);
        a.part_ml = reinterpret_cast<float *>(reinterpret_cast<char *>(ws) + o_bytes);
    }
    dim3 grid((unsigned)(a.nsplit * Lq * H), 1, (unsigned)B);
    int nch = (int)ceil_div(E, 64);
    if (nch == 1) launch_rows<1>(a, vec, grid, st);
    else if (nch == 2) launch_rows<2>(a, vec, grid, st);
    else launch_rows<4>(a, vec, grid, st);
    if (a.nsplit > 1) {
        long total = (long)Lq * H * B * E;
        hipLaunchKernelGGL(sdpa_merge_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, a);
    }
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

// Decode step, self-attention: append the newest key/value row to the cache and attend over the cache in one launch.
int mi_sdpa_append_f16(void *out, int out_dtype, const int64_t out_strides[4],
                       const void *q, const int64_t q_strides[4],
                       void *cache_k, const int64_t k_strides[4], void *cache_v, const int64_t v_strides[4],
                       const void *k_new, const void *v_new, const int64_t new_strides[4],
                       const int32_t *kv_len, int64_t E, int64_t Lk, int64_t H, int64_t B, float scale, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !k_new || !v_new || !new_strides) return MI_DECLINE_OPERANDS;
    SdpaArgs a;
    int rc = fill(a, out, out_dtype, out_strides, q, q_strides, cache_k, k_strides, cache_v, v_strides, nullptr, MI_F16, nullptr, kv_len, E, 1, Lk, H, B, scale);
    if (rc != MI_OK) return rc;
    if (H == 0 || B == 0 || E == 0) return MI_OK;
    a.k_new = (const half_t *)k_new; a.v_new = (const half_t *)v_new;
    for (int i = 0; i < 4; i++) a.ns[i] = new_strides[i];
    if (sdpa_path(a) == MI_SDPA_DECLINE) return MI_DECLINE_EXTENT;
    const bool vec = vec_addressable(a.q, a.qs, a.E) && vec_addressable(a.k, a.ks, a.E) && vec_addressable(a.v, a.vs, a.E) &&
                     vec_addressable(a.k_new, a.ns, a.E) && vec_addressable(a.v_new, a.ns, a.E);
    if (!one_pass_decode(a, vec)) return MI_DECLINE_UNSUPPORTED;      // the caller appends and attends in two calls
    return launch_decode(a, (hipStream_t)stream);
}

}  // extern "C"
