/*
 * mi355dnn: C ABI of the MI355X (gfx950) dense-contraction kernels.
 *
 * This is the drop-in boundary under the reference's kernel entry points
 *   matmul!/batchedmatmul!   DNNKernels/src/kernels/extern/matmul.jl:78-79,383
 *   sdpa / sdpa!             DNNKernels/src/kernels/extern/attention.jl:712,773-834
 *   convolution!             DNNKernels/src/kernels/extern/conv.jl:100-101
 *   layernorm!               DNNKernels/src/kernels/layernorm.jl:125
 * which the op handlers call (DNNKernels/src/ops.jl:575-647,1114-1222,1347-1399).
 *
 * Conventions
 *   - Every data pointer is a DEVICE pointer (hipMalloc); `stream` is a
 *     hipStream_t passed as void* (NULL = the default stream).  Calls enqueue
 *     work and return; they never synchronise and never allocate.
 *   - Arrays are row-major C arrays.  The reference's column-major Julia array
 *     (a,b,c,d) is the same bytes as the row-major [d][c][b][a]
 *     (DNNKernels/src/safetensors.jl:7-12), so nothing is copied at the boundary.
 *   - Leading dimensions and strides are in ELEMENTS.
 *   - Return value: MI_OK, or a decline code.  A decline is the C form of the
 *     reference's `Decline(reason)` (DNNKernels/src/kernelplans.jl:21-35): no
 *     work was enqueued and the caller takes its own fallback.  Nothing throws.
 *   - Scratch comes from the caller (`ws`, `ws_bytes`): the reference hands
 *     kernels per-op scratch from its bump workspace, valid until the next op
 *     (DNNKernels/src/workspace.jl:63-106); the *_workspace functions say how
 *     much a call needs.  ws must be 256-byte aligned.
 */
#ifndef MI355DNN_H
#define MI355DNN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355DNN_VERSION 1

enum mi_status {
    MI_OK = 0,
    MI_DECLINE_OPERANDS = 1,    /* null / misaligned / unsupported layout        (Decline(:operands)) */
    MI_DECLINE_EXTENT = 2,      /* an extent the kernels do not cover            (Decline(:extent))   */
    MI_DECLINE_WORKSPACE = 3,   /* ws too small or misaligned                                          */
    MI_DECLINE_BIAS = 4,        /* a bias/mask shape the call cannot apply       (Decline(:bias))     */
    MI_DECLINE_UNSUPPORTED = 5, /* e.g. grouped convolution                                            */
    MI_ERROR_LAUNCH = 6,        /* HIP reported an error at launch                                     */
    MI_ERROR_DEVICE = 7,        /* no gfx950 device / library not initialised                          */
    MI_DECLINE_SCRATCH_LIMIT = 8 /* mi_gemm_f16_noalloc: the call needs more than MI_NOALLOC_SCRATCH_BYTES */
};

enum mi_epilogue { MI_EPI_NONE = 0, MI_EPI_GELU_ERF = 1, MI_EPI_GELU_TANH = 2, MI_EPI_RELU = 3 };
enum mi_dtype { MI_F16 = 0, MI_F32 = 1 };
enum mi_wlayout { MI_W_KF = 0, MI_W_FK = 1 };
enum mi_bias_mode { MI_BIAS_NONE = 0, MI_BIAS_COL = 1, MI_BIAS_ROW = 2 };

/* Which kernel a GEMM call takes; returned by mi_gemm_f16_plan so a host-side
 * planner (the reference's `mmplan`, matmul.jl:87-95) can be tested without a launch. */
enum mi_gemm_path { MI_GEMM_DECLINE = 0, MI_GEMM_MFMA = 1, MI_GEMM_SKINNY = 2, MI_GEMM_SCALAR = 3 };
enum mi_sdpa_path { MI_SDPA_DECLINE = 0, MI_SDPA_FLASH = 1, MI_SDPA_ROWS = 2 };
enum mi_conv_path { MI_CONV_DECLINE = 0, MI_CONV_GEMM_1X1 = 1, MI_CONV_IM2COL_GEMM = 2, MI_CONV_DIRECT = 3, MI_CONV_IMPLICIT_GEMM = 4 };
enum mi_convt_path { MI_CONVT_DECLINE = 0, MI_CONVT_GEMM_SHUFFLE = 1, MI_CONVT_GATHER = 2 };

/* Library / device. */
int mi_version(void);
/* Selects nothing and allocates nothing: checks that the current HIP device is
 * gfx950 and raises the kernels' dynamic-LDS limits.  Idempotent.  Replaces the
 * reference's `caps(backend)` device query (DNNKernels/src/context.jl:55,68). */
int mi_init(void);
/* Device facts a planner needs (the fields of Lava.DeviceCaps the reference
 * reads, context.jl:68): out[0]=mfma available, [1]=tile (16), [2]=wavefront (64),
 * [3]=LDS bytes per workgroup, [4]=max workgroup size, [5]=compute units. */
int mi_device_caps(int64_t out[6]);

/* Measurement aid (no counterpart in the reference).  While a device buffer of four uint64 is registered (NULL
 * clears it), workgroup 0 of every launch of the four-wave GEMM kernel (the 128 x 256, 192 x 128 and split
 * 128 x 128 tiles of mi_gemm_f16 and its variants) stores {shader clock, constant 100 MHz clock} there when it starts and again after
 * its last store: buf = {clk0, ref0, clk1, ref1}, and (clk1 - clk0) / (ref1 - ref0) x 100 MHz is the shader clock the
 * launch ran at.  The caller keeps the buffer alive while it is registered.  Process-wide, not thread safe. */
int mi_set_clock_probe(void *dev_u64x4);
/* A second measurement aid of the same kind.  While a device buffer of workgroups x 4 x 4 uint64 is registered (NULL
 * clears it), matrix wave w of workgroup g < workgroups of every four-wave GEMM launch stores at buf[(g * 4 + w) * 4 ..]
 * the shader clocks it spent {from its start to its K loop, in the K loop, issuing its store (for the split-K
 * instance: exchange and store), waiting for the store to be acknowledged}.  Costs the launch five clock reads a wave
 * while registered, a scalar branch otherwise.  Process-wide, not thread safe. */
int mi_set_phase_probe(void *dev_u64, int64_t workgroups);

/* Ceiling probes (measurement aids, no counterpart in the reference).
 * mi_probe_mfma: `workgroups` workgroups of eight waves run `steps` 64-deep steps of the 128 x 256 GEMM tile's
 * arithmetic -- sixteen v_mfma_f32_32x32x16_f16 per wave and step, 2 x 8 x 16 x 32768 flop per workgroup and step --
 * on operand fragments held in registers, with no memory operation in the loop; gelu != 0 adds the GEMM epilogue's
 * arithmetic (bias, rounding, erf-GELU) on every accumulator value.  seed_f16: 65536 fp16 values the fragments are
 * taken from (random values make the multipliers toggle as on real data); sink: 512 x workgroups floats that are never
 * actually written.  240 workgroups x 20 steps with gelu is config 1's launch minus its memory traffic; a grid of many
 * rounds is what the matrix units sustain at the clock the chip holds under that load.
 * mi_probe_copy: out[0 .. bytes) = in[0 .. bytes), 16 bytes per lane and step; bytes % 16 == 0.  A kernel of known HBM
 * traffic (bytes read + bytes written).
 * mi_probe_grid_barrier: `workgroups` (<= compute units) workgroups meet `rounds` times at a barrier across the whole
 * grid -- an agent-scope atomic add on a counter in device memory and a bounded poll -- and, with bit 0 of payload set,
 * exchange 16 bytes each around it (write-through stores before, reads past the L2 after): what one phase boundary inside
 * a multi-phase persistent kernel would cost.  Bit 1 of payload: the barrier in two levels (eight groups of workgroups
 * with a counter and a release flag each, so that no address sees more than 32 arrivals or pollers).  scratch_u32:
 * 2304 + 32 x workgroups bytes of device memory, 16-byte aligned; word 4 is nonzero afterwards if some workgroup gave up
 * waiting (it then ran on without waiting).  Not for use under graph capture (it clears its counters with a memset). */
int mi_probe_mfma(void *sink, const void *seed_f16, int64_t workgroups, int64_t steps, int gelu, void *stream);
int mi_probe_grid_barrier(void *scratch_u32, int64_t workgroups, int64_t rounds, int payload, void *stream);
int mi_probe_copy(void *out, const void *in, size_t bytes, void *stream);

/* Device-side failures (no counterpart in the reference, whose kernels never wait for one another).  A few kernels
 * here exchange data between workgroups inside one launch and wait for each other a bounded time; a wait that gives
 * up cannot be reported by the call that enqueued the launch, so it is recorded in a sticky word in device memory.
 * mi_device_status SYNCHRONISES the current device (the one exception to "calls never synchronise") and returns the
 * OR of enum mi_device_status_bits raised since the last reset, or -1 if the device cannot be read.  With reset != 0
 * it also clears the word and zeroes the exchange's flag banks (a workgroup that gave up has not released them): do
 * that before reusing the device after a nonzero status, and re-run the affected work -- its outputs hold NaN where
 * a workgroup gave up. */
enum mi_device_status_bits {
    MI_DEVSTAT_EXCHANGE_TIMEOUT = 1,  /* split-K exchange of mi_gemm_f16: a partner workgroup did not arrive in time   */
    MI_DEVSTAT_EXCHANGE_XCD = 2,      /* split-K exchange: partner workgroups did not share an XCD (one L2)            */
    MI_DEVSTAT_STEP_BARRIER = 4       /* a workgroup gave up at a barrier across the grid (mi_probe_grid_barrier's word) */
};
int mi_device_status(int reset);
/* Process-wide switch for the in-launch split-K exchange of mi_gemm_f16 and its variants (on by default where the
 * device passed the XCD probe at mi_init).  Off: split K goes through fp32 planes in ws and a summing launch; plans
 * and workspace sizes follow the switch, so query workspaces after setting it. */
int mi_set_in_launch_exchange(int enabled);
/* Test aid: makes the exchange's bounded waits fail from the host side, so that the failure path can be exercised
 * with every kernel still exiting normally.  spin_limit: polls before a wave gives up (<= 0 restores the default);
 * publish_xor: XORed into the epoch a wave publishes (nonzero: no partner ever sees the epoch it waits for);
 * xcc_xor: XORed into the XCD id a wave expects of its partners (nonzero: every partner looks misplaced).
 * (0, 0, 0) restores ordinary operation.  Process-wide, not thread safe. */
int mi_test_exchange_faults(int spin_limit, unsigned publish_xor, unsigned xcc_xor);

/* ---------------------------------------------------------------- GEMM
 * Y[T x F] = epi(round(X[T x K] . W + bias)) (+ residual)
 *   X   fp16 [T][K], ldX.
 *   W   fp16, MI_W_KF: [K][F] (the reference's hoisted weight,
 *       DNNKernels/src/hoistcasts.jl:47-112) or MI_W_FK: [F][K]; ldW.
 *   bias fp16 or NULL; MI_BIAS_COL: bias[F] (addmm), MI_BIAS_ROW: bias[T]
 *       (the reference GEMM's per-row bias of the column-major C, matmul.jl:188-217).
 *   fp32 accumulation seeded with the bias (matmul.jl:21,230-233), one rounding
 *   to out_dtype, the activation applied to the ROUNDED value (matmul.jl:210-214).
 *   residual (fp16, same layout as Y, or NULL; fp16 output only) is added after the
 *   activation with one more rounding: the graph's own add.Tensor (ops.jl:186-197).
 * Replaces matmul!(ctx, out, A, B, bias; epi) -- matmul.jl:78-79,99-100,133-137,235-273.
 * Concurrency: a launch that splits K inside the kernel (the workgroups of a tile exchange partial tiles through
 * arrival flags) takes the next of 16 banks of flag words held in static device memory, and leaves its bank zeroed.
 * Such a launch assumes that all its workgroups become resident together, which holds on an otherwise idle GPU (the
 * grid is at most one workgroup per compute unit) and is NOT guaranteed while kernels of other streams occupy
 * compute units: a workgroup waits for its partners a bounded time only, and if the bound is reached -- or a partner
 * turns out to run on another XCD -- it stores NaN over its part of Y and raises the sticky status word that
 * mi_device_status reads; the call itself has long returned MI_OK.  A caller that overlaps streams should either
 * check mi_device_status at its synchronisation points or switch the exchange off (mi_set_in_launch_exchange(0):
 * K-slices then go through fp32 planes in ws and a second launch, as on a device that fails the XCD probe).
 * Up to 16 such launches may be in flight on one GPU; a captured launch keeps the bank it was given at capture, so
 * two captured graphs that hold the same bank must not be replayed at the same time. */
int mi_gemm_f16(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                int w_layout, int bias_mode, int epi, int out_dtype,
                void *ws, size_t ws_bytes, void *stream);

/* The same over `nbatch` planes: element strides sY, sX, sW, sBias between planes
 * (0 = operand shared).  Replaces batchedmatmul!(ctx, out, A, B) -- matmul.jl:364-392
 * and the nbatch form of the GEMMs in sdpa_coopmat! -- attention.jl:697-699.  With
 * sX = 0 it also runs several addmm ops that read the same activations (the q, k, v
 * projections of one attention, ops.jl:1347-1356 three times) as one launch. */
int mi_gemm_f16_batched(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                        int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                        int w_layout, int bias_mode, int epi, int out_dtype,
                        int64_t nbatch, int64_t sY, int64_t sX, int64_t sW, int64_t sBias,
                        void *ws, size_t ws_bytes, void *stream);

/* Decode-sized T (<= 8; more declines with MI_DECLINE_EXTENT): the
 * bandwidth-bound form.  [K][F] weights: K split across workgroups, fp32
 * partial planes in ws, a reducing epilogue (ws from mi_gemm_f16_workspace).
 * [F][K] weights: one launch, no workspace.  mi_gemm_f16 takes the same route
 * by itself for T <= 8; this entry forces it.
 * The reference's counterpart is the fp32-only Lava.gemv! path
 * (matmul.jl:108-137) and mm_epilogue_kernel! (matmul.jl:192-217). */
int mi_gemv_f16(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                int w_layout, int bias_mode, int epi, int out_dtype,
                void *ws, size_t ws_bytes, void *stream);

/* Y = epi(layernorm(X) . W + bias) (+ residual) for T <= 8 in one pass over the weights:
 * the rows of X are normalised over K (fp32 statistics, gamma/beta fp16 or NULL, the
 * result rounded to fp16) while they are staged, in the arithmetic and summation order
 * of mi_layernorm_f16, so the result is bit-identical to that call followed by
 * mi_gemv_f16.  The reference runs the two as separate ops (layernorm!,
 * layernorm.jl:125, then matmul!, matmul.jl:78-79); folding the norm into the GEMM's
 * prologue is item 3 of its plans/kernels-to-port.md.  Workspace as for mi_gemv_f16. */
int mi_ln_gemv_f16(void *Y, const void *X, const void *gamma, const void *beta, float eps,
                   const void *W, const void *bias, const void *residual,
                   int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                   int w_layout, int bias_mode, int epi, int out_dtype,
                   void *ws, size_t ws_bytes, void *stream);

/* The same fold for any T: Y = epi(layernorm(X) . W + bias) (+ residual), bit-identical to mi_layernorm_f16 followed
 * by mi_gemm_f16 on its result.  T <= 8 is mi_ln_gemv_f16.  Larger T runs the tiled MFMA kernel with the norm as its
 * prologue: every workgroup normalises its 64 rows of X into an LDS panel (one wave per row, the lane / summation
 * order of mi_layernorm_f16) and then streams W alone; this needs 128 <= K <= 512 and K % 64 == 0 (a ViT-S block's
 * d = 384), anything else returns MI_DECLINE_EXTENT and the caller runs the two ops.  No workspace is used for T > 8.
 * The reference runs layernorm! (layernorm.jl:125) and matmul! (matmul.jl:78-79) as separate ops; the fold is item 3
 * of its plans/kernels-to-port.md. */
int mi_ln_gemm_f16(void *Y, const void *X, const void *gamma, const void *beta, float eps,
                   const void *W, const void *bias, const void *residual,
                   int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                   int w_layout, int bias_mode, int epi, int out_dtype,
                   void *ws, size_t ws_bytes, void *stream);

/* mi_gemm_f16 followed by mi_layernorm_f16 of its output rows: Y[T][F] (fp16, dense rows) as mi_gemm_f16 writes
 * it, and H[T][F] = layer norm of Y over F with gamma / beta (either may be NULL).  When the GEMM splits K the norm
 * rides in the pass that sums the planes (one launch less); otherwise the two kernels run back to back.  Either way
 * Y and H carry the bits of the two separate calls.  The graph shape it serves: a linear op (+ residual) whose
 * result is both the residual stream and the input of the next block's first norm (layer_norm, ops.jl:575-647,
 * after addmm + add.Tensor, ops.jl:1347-1363,186-197); the reference runs the three ops one by one.
 * Workspace as for mi_gemm_f16. */
int mi_gemm_ln_f16(void *Y, void *H, const void *X, const void *W, const void *bias, const void *residual,
                   const void *gamma, const void *beta, float eps,
                   int64_t T, int64_t K, int64_t F, int64_t ldX, int64_t ldW,
                   int w_layout, int bias_mode, int epi, void *ws, size_t ws_bytes, void *stream);
/* mi_gemm_ln_f16 with the result clamped to [-clamp, clamp] (clamp > 0) after the residual add, as a separate
 * aten::clamp on Y would leave it -- the fp16 overflow guard that exported encoder layers carry after every block
 * (ops.jl:300-310) -- and H, the layer norm of the clamped rows, optional (null: none).  The tiled kernels and the
 * split-K plane sum clamp in their stores; decode-sized and unaligned shapes clamp in a pass of their own.  Bits as
 * the separate ops give them. */
int mi_gemm_clamp_ln_f16(void *Y, void *H, const void *X, const void *W, const void *bias, const void *residual,
                         const void *gamma, const void *beta, float eps, float clamp,
                         int64_t T, int64_t K, int64_t F, int64_t ldX, int64_t ldW,
                         int w_layout, int bias_mode, int epi, void *ws, size_t ws_bytes, void *stream);

size_t mi_gemm_f16_workspace(int64_t T, int64_t K, int64_t F, int w_layout, int64_t nbatch);

/* ---- a layer norm with no pass of its own
 * layernorm! followed by matmul! (layernorm.jl:125, matmul.jl:78-79) is, algebraically,
 *     LN(x) . W + b  =  r (x . W') - r mu colsum(W') + b',      W'[k][n] = gamma[k] W[k][n],  b' = b + beta . W,
 * with (mu, r) the row's mean and 1 / sqrt(var + eps): the GEMM can run on the RAW rows and apply a per-row scale and
 * a rank-one correction in its store, if it knows (mu, r) -- and the GEMM that WROTE the rows can leave what is needed
 * behind.  Three pieces:
 *   mi_lnfold_prepare_f16   once per weight, at load: Wp = fp16(gamma W) in W's layout, colsum[F] (of the rounded Wp)
 *                           and biasp[F] in fp32.  gamma, beta, bias may be NULL.
 *   row statistics          stats[ceil(C / 32)][rows][2] fp32: for every 32-column segment of a row, the sum and the
 *                           squares about the segment's own mean (segment-major, so that a wave reads the segments of
 *                           64 consecutive rows as contiguous 512 bytes).  Written by mi_gemm_rowstats_f16 (mi_gemm_f16 with
 *                           dense rows of Y, ldY = F, that also leaves the statistics of the final fp16 rows, after
 *                           residual and clamp), by mi_lnfold_gemm_f16 (stats_out), or by mi_rowstats_f16 for rows that
 *                           no GEMM of this library wrote (a block's first input).
 *   mi_lnfold_gemm_f16      Y = epi(round(r (X . Wp) - r mu colsum + biasp)) (+ residual), (mu, r) combined per row
 *                           from stats_in (segment sums -> mean; squares about that mean by the pairwise update, never
 *                           as sum(x^2) - n mu^2).  nbatch planes share X and stats_in (sY, sW, sVec = plane strides of
 *                           Y, Wp, colsum / biasp): q, k, v in one launch.  T > 8, K % 64 == 0, K >= 128, 16-byte rows;
 *                           anything else returns a decline and the caller runs the two ops.
 * What differs from the two ops: the reference rounds the normalised row to fp16 before the product; here the rounding
 * sits on gamma W instead and the normalised row is never formed.  Same order of error (one fp16 rounding of one
 * factor per product term), not the same bits: held to the 1e-2 / 0.9999 gate against layernorm -> GEMM, not to
 * bit-identity (mi_ln_gemm_f16 is the bit-identical fold).  The reference's own plans name the fold of the norm into
 * the GEMM as open work (plans/kernels-to-port.md item 3; plans/perf-plan.md:4074-4095). */
int mi_lnfold_prepare_f16(void *Wp, float *colsum, float *biasp, const void *W, const void *gamma, const void *beta, const void *bias,
                          int64_t K, int64_t F, int64_t ldW, int w_layout, void *stream);
int mi_rowstats_f16(float *stats, const void *a, int64_t ld, int64_t C, int64_t rows, void *stream);
int mi_gemm_rowstats_f16(void *Y, float *stats, const void *X, const void *W, const void *bias, const void *residual, float clamp,
                         int64_t T, int64_t K, int64_t F, int64_t ldX, int64_t ldW,
                         int w_layout, int bias_mode, int epi, void *ws, size_t ws_bytes, void *stream);
int mi_lnfold_gemm_f16(void *Y, float *stats_out, const void *X, const float *stats_in, float eps,
                       const void *Wp, const float *colsum, const float *biasp, const void *residual, float clamp,
                       int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                       int w_layout, int epi, int out_dtype,
                       int64_t nbatch, int64_t sY, int64_t sW, int64_t sVec, void *ws, size_t ws_bytes, void *stream);

/* mi_gemm_f16 without the workspace arguments, for callers that cannot allocate device memory and have no
 * workspace to hand over: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference (whose kernels always draw scratch from the caller's bump workspace,
 * workspace.jl:63-106).  The split-K / decode planes go to a static device array of MI_NOALLOC_SCRATCH_BYTES that
 * every GPU the library runs on holds until the process ends; a call that would need more (what
 * mi_gemm_f16_workspace(T, K, F, w_layout, 1) returns) is refused with MI_DECLINE_SCRATCH_LIMIT and enqueues
 * nothing.  Calls no hipMalloc / hipFree / allocating routine.  Same kernels, same plan and same bits as
 * mi_gemm_f16.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams
 * without ordering between them) race on it. */
#define MI_NOALLOC_SCRATCH_BYTES (32 * 1024 * 1024)
int mi_gemm_f16_noalloc(void *Y, const void *X, const void *W, const void *bias, const void *residual,
                        int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                        int w_layout, int bias_mode, int epi, int out_dtype, void *stream);
/* Returns an mi_gemm_path; never launches.  Replaces mmplan / mm_coopmat_plan /
 * mm_gemv_plan -- matmul.jl:87-95,121-131,172-179. */
int mi_gemm_f16_plan(const void *Y, const void *X, const void *W,
                     int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                     int w_layout, int out_dtype, int64_t nbatch, int64_t sY, int64_t sX, int64_t sW);

/* mi_gemm_f16_plan for a device the caller describes: caps are the six values of mi_device_caps (NULL: the current
 * device), of which the planner reads [0] (matrix unit present; without it the tiled MFMA path is not offered) and
 * [5] (compute units, which decide tiles and K-splits).  ksplit_out (optional) receives the number of K-slices the
 * plan would use.  The reference's planners take a DeviceCaps value for the same purpose: tests ask about hardware
 * they do not have (DNNKernels/test/test_flash.jl:328,363,373-377; context.jl:68).  Never launches, needs no GPU. */
int mi_gemm_f16_plan_caps(const int64_t caps[6], const void *Y, const void *X, const void *W,
                          int64_t T, int64_t K, int64_t F, int64_t ldY, int64_t ldX, int64_t ldW,
                          int w_layout, int out_dtype, int64_t nbatch, int64_t sY, int64_t sX, int64_t sW, int *ksplit_out);

/* ---------------------------------------------------------------- attention
 * out(E,Lq,H,B) = softmax_over_keys(scale * q.k + bias) . v
 *   q (E,Lq,H,B), k (E,Lk,H,B), v (E,Lk,H,B): fp16, each given as a base pointer
 *   plus four element strides in (E, L, H, B) order -- the reference passes
 *   root pointer + offsets + strides the same way (flash.jl:1353-1365,1448-1474).
 *   out is (E,Lq,H,B), fp16 or fp32 (the graph's declared type, ops.jl:1365-1391);
 *   out_strides NULL means dense = row-major [B][H][Lq][E], which is what the
 *   reference allocates (attention.jl:762-765).  Element strides in (E,L,H,B)
 *   order let the caller have the result written token-major ([B][Lq][H][E]),
 *   i.e. already in the layout the graph's following permute + reshape produces.
 *   bias: optional additive mask laid out (Lk,Lq,H,B) with element strides
 *   bias_strides[4]; a stride of 0 broadcasts that axis (attention.jl:55-59,
 *   launch.jl:72-75); bias_dtype MI_F16 / MI_F32.  An fp16 mask whose query
 *   stride is 0 (a padding mask (B,1,1,Lk), a per-head key bias) over at most 4096
 *   keys costs the fused kernel no time: give a padding mask in that form rather
 *   than written out per query.
 *   kv_len: optional device int32[B]; keys >= kv_len[b] get weight exactly 0
 *   (what the decoder's 0 / finfo.min mask does, tools/export_whisper_decoder.py:158-165).
 *   A row with every key excluded yields zeros, not NaN (attention.jl:82-87).
 * Replaces sdpa(ctx, q, k, v, bias, scale; out) -- attention.jl:712-834 -- and the
 * fused kernels behind it: attn_flash_cm! + attn_flash_cm_merge! (flash.jl:459-1036,
 * 1398-1421), attn_softmax_rows! / sdpa_coopmat! (attention.jl:514-705). */
int mi_sdpa_f16(void *out, int out_dtype, const int64_t out_strides[4],
                const void *q, const int64_t q_strides[4],
                const void *k, const int64_t k_strides[4],
                const void *v, const int64_t v_strides[4],
                const void *bias, int bias_dtype, const int64_t bias_strides[4],
                const int32_t *kv_len,
                int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale,
                void *ws, size_t ws_bytes, void *stream);
size_t mi_sdpa_f16_workspace(int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, int has_bias);
/* Returns an mi_sdpa_path; replaces sdpaplan / flashcm_plan -- attention.jl:735-759,
 * flash.jl:1322-1374.  nsplit_out (optional) receives the key-split count
 * (splitcount, flash.jl:1288-1303). */
int mi_sdpa_f16_plan(const void *q, const int64_t q_strides[4],
                     const void *k, const int64_t k_strides[4],
                     const void *v, const int64_t v_strides[4],
                     int has_bias, int has_kv_len,
                     int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale,
                     int *nsplit_out);

/* mi_sdpa_f16_plan for a device the caller describes (see mi_gemm_f16_plan_caps): without a matrix unit the fused
 * kernel is not offered, and the compute-unit count decides the key splits (splitcount(dev, ...), flash.jl:1288-1303). */
int mi_sdpa_f16_plan_caps(const int64_t caps[6], const void *q, const int64_t q_strides[4],
                          const void *k, const int64_t k_strides[4],
                          const void *v, const int64_t v_strides[4],
                          int has_bias, int has_kv_len,
                          int64_t E, int64_t Lq, int64_t Lk, int64_t H, int64_t B, float scale,
                          int *nsplit_out);

/* ---------------------------------------------------------------- convolution
 * Reference layout: x (W,H,Cin,N) = row-major [N][Cin][H][W]; w (KW,KH,Cin,Cout) =
 * [Cout][Cin][KH][KW]; out (OW,OH,Cout,N); bias[Cout] or NULL; stride / padding /
 * dilation as (x, y) pairs; act MI_EPI_NONE or MI_EPI_RELU (anything else returns
 * MI_DECLINE_UNSUPPORTED).  groups = 1 runs as a GEMM (1x1, implicit, or im2col: see
 * mi_conv2d_f16_plan); groups > 1 -- w then holds Cin / groups input channels per filter --
 * runs a direct kernel, one thread per output element, as the reference routes
 * grouped convolutions to its direct kernel (conv.jl:100-145); Cin or Cout not
 * divisible by groups declines.  fp32 accumulation seeded with the bias, one rounding,
 * relu on the rounded value.
 * Replaces convolution!(ctx, out, x, w, bias, stride, padding, dilation, groups; act)
 * -- conv.jl:100-145 -- and convolution_coopmat! / im2col_kernel! /
 * conv_epilogue_kernel! -- conv_coopmat.jl:246-392; the implicit-GEMM path (stride_x 1,
 * OW % 8 == 0, Cin*KH*KW % 64 == 0) is the MFMA counterpart of conv2d_igemm! --
 * conv_implicit.jl:53-355: the im2col matrix is never written, the GEMM gathers its
 * operand from a zero-padded copy of x in the workspace. */
int mi_conv2d_f16(void *out, const void *x, const void *w, const void *bias,
                  int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                  int64_t KW, int64_t KH, int64_t Cout,
                  int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                  int64_t dil_x, int64_t dil_y, int64_t groups, int act,
                  void *ws, size_t ws_bytes, void *stream);
size_t mi_conv2d_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                               int64_t KW, int64_t KH, int64_t Cout,
                               int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                               int64_t dil_x, int64_t dil_y);
/* Returns an mi_conv_path; replaces conv_coopmat_plan / onebyone -- conv_coopmat.jl:83-155,
 * conv.jl:63-66. */
int mi_conv2d_f16_plan(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                       int64_t KW, int64_t KH, int64_t Cout,
                       int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                       int64_t dil_x, int64_t dil_y, int64_t groups);
/* The same convolution over channels-last tensors: x [N][H][W][Cin], w [Cout][KH][KW][Cin], out [N][OH][OW][Cout]
 * (groups = 1).  An implicit GEMM with nothing staged: out[(n,oh,ow)][Cout] = patch . w^T, the patch matrix gathered
 * from x by the GEMM's own operand loads, the weights read as they lie; split-K planes in ws where the output tiles
 * are few.  Needs Cin % 64 == 0 and Cout % 8 == 0 (MI_DECLINE_UNSUPPORTED otherwise: use the layout above).
 * The reference has no channels-last path -- its arrays are (W,H,C,N) throughout (safetensors.jl:7-12) -- but its
 * implicit-GEMM kernel walks K the same way, conv2d_igemm!, conv_implicit.jl:53-355. */
int mi_conv2d_nhwc_f16(void *out, const void *x, const void *w, const void *bias,
                       int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                       int64_t KW, int64_t KH, int64_t Cout,
                       int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                       int64_t dil_x, int64_t dil_y, int act,
                       void *ws, size_t ws_bytes, void *stream);
size_t mi_conv2d_nhwc_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                                    int64_t KW, int64_t KH, int64_t Cout,
                                    int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                                    int64_t dil_x, int64_t dil_y);
/* The convolution of mi_conv2d_f16 (groups = 1) with its output token-major: out[n][m][co], m = oh * OW + ow, one row
 * of Cout values per output pixel at pitch ld_out, images out_image_stride elements apart -- what a ViT's
 * flatten(2).transpose(1, 2) makes of the channel-major result -- plus, if given, residual[n][m][co] (fp16, the same
 * pitch, images res_image_stride apart; 0 = one residual for every image, the position embedding), added to the
 * rounded result with one more rounding, as an add after the convolution would.  ld_out and the strides are
 * multiples of 8, out and residual 16-byte aligned.  The im2col matrix is written token-major and is the GEMM's
 * row-major operand, the weights are its K-contiguous operand as they lie, the bias is per column: patch embedding
 * + position embedding in two launches (im2col with the weight padding in its last blocks, GEMM) instead of
 * convolution, transpose and add.
 * The reference runs these as separate ops: convolution! (conv.jl:100-145), its permute, add (ops.jl); its fold
 * passes merge neighbours of this kind into one kernel's epilogue (foldrelu.jl:60-125). */
int mi_conv2d_tokens_f16(void *out, int64_t ld_out, int64_t out_image_stride,
                         const void *x, const void *w, const void *bias, const void *residual, int64_t res_image_stride,
                         int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                         int64_t KW, int64_t KH, int64_t Cout,
                         int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                         int64_t dil_x, int64_t dil_y, int act,
                         void *ws, size_t ws_bytes, void *stream);
size_t mi_conv2d_tokens_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                                      int64_t KW, int64_t KH, int64_t Cout,
                                      int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                                      int64_t dil_x, int64_t dil_y);
/* ATen's output extent -- convsize, conv.jl:309. */
int64_t mi_convsize(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d);

/* Transposed convolution.  x as above; w (KW,KH,Cout/groups,Cin) = row-major
 * [Cin][Cout/groups][KH][KW] (torch's conv_transpose2d weight); out (OW,OH,Cout,N) with
 * OW = mi_convtransposesize(...); bias[Cout] or NULL.  fp32 accumulation seeded with the
 * bias, one rounding.  kernel == stride with no padding / dilation / output padding and one
 * group is one MFMA GEMM (Cout*KH*KW x Cin x H*W per image) followed by a pixel shuffle,
 * workspace from mi_convtranspose2d_f16_workspace; every other case is the gather kernel
 * and needs no workspace.
 * Replaces convolutiontranspose!(ctx, out, x, w, bias, stride, padding, dilation, outpad,
 * groups) -- conv.jl:226-294 -- with shufflecase / shuffleout (conv.jl:204-222) and the
 * gather kernel convtranspose2d (conv.jl:149-191). */
int mi_convtranspose2d_f16(void *out, const void *x, const void *w, const void *bias,
                           int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                           int64_t KW, int64_t KH, int64_t Cout,
                           int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                           int64_t dil_x, int64_t dil_y, int64_t outpad_x, int64_t outpad_y,
                           int64_t groups, void *ws, size_t ws_bytes, void *stream);
size_t mi_convtranspose2d_f16_workspace(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                                        int64_t KW, int64_t KH, int64_t Cout,
                                        int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                                        int64_t dil_x, int64_t dil_y, int64_t outpad_x, int64_t outpad_y,
                                        int64_t groups);
/* Returns an mi_convt_path; replaces shufflecase -- conv.jl:204-209. */
int mi_convtranspose2d_f16_plan(int64_t Wi, int64_t Hi, int64_t Cin, int64_t N,
                                int64_t KW, int64_t KH, int64_t Cout,
                                int64_t stride_x, int64_t stride_y, int64_t pad_x, int64_t pad_y,
                                int64_t dil_x, int64_t dil_y, int64_t outpad_x, int64_t outpad_y,
                                int64_t groups);
/* ATen's transposed-convolution output extent -- convtransposesize, conv.jl:201. */
int64_t mi_convtransposesize(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d, int64_t op);

/* ---------------------------------------------------------------- layout
 * in is an (E,L,H,B) fp16 operand given by its four element strides (any non-negative
 * values; a zero broadcasts); out receives it as (L,E,H,B), L contiguous: dense when
 * out_strides is NULL, else by its own strides (out_strides[0] must be 1).  With H = B = 1
 * this is the 2-D transpose out[e][l] = in[l][e].
 * Replaces transposeLE(ctx, a) / toLE_tiled_Float16! -- attention.jl:342-396.  The
 * reference's other layout pass, padcols_kernel! (matmul.jl:182-185), has no counterpart:
 * mi_gemm_f16 takes ragged T, K, F as they are. */
int mi_transpose_le_f16(void *out, const int64_t out_strides[4], const void *in, const int64_t in_strides[4],
                        int64_t E, int64_t L, int64_t H, int64_t B, void *stream);

/* w_fk[F][K] (pitch ld_fk) = transpose of w_kf[K][F] (pitch ld_kf): a weight in the reference's hoisted layout
 * (hoistpermutes, DNNKernels/src/hoistcasts.jl:47-112) re-laid K-contiguous, to be done ONCE where the model uploads
 * its weights (Model, DNNKernels/src/driver.jl:165-168) and passed from then on with w_layout = MI_W_FK.  Values
 * are unchanged, so every product is bit-identical to the one over the original; what changes is the route: decode-
 * sized linears (T <= 8) run as one launch without a workspace instead of K-slices plus a summing launch, and the
 * tiled GEMM reads both operands K-contiguous.  One launch of the transpose kernel of mi_transpose_le_f16. */
int mi_relayout_weight_f16(void *w_fk, int64_t ld_fk, const void *w_kf, int64_t ld_kf, int64_t K, int64_t F, void *stream);

/* ---------------------------------------------------------------- layer norm + glue
 * `groups` rows of C contiguous fp16 elements; mean in fp32, variance about that
 * mean in fp32, out = (x-mean)*rstd*gamma + beta rounded to fp16; mean/rstd
 * (fp32[groups], either may be NULL) returned as native_layer_norm does.
 * Replaces layernorm!(ctx, out, mean, rstd, a, gamma, beta, C, eps) -- layernorm.jl:44-135. */
int mi_layernorm_f16(void *out, float *mean, float *rstd, const void *a,
                     const void *gamma, const void *beta,
                     int64_t C, int64_t groups, float eps, void *stream);

/* Softmax over the last, contiguous axis of `rows` rows of n elements, fp16 or fp32 (dtype) in and out:
 * out = exp(scale * a - max) / sum in fp32, one rounding; a row of -inf gives zeros.  The reference's softmax_kernel!
 * (ops.jl:474-573, aten::_softmax; scale = 1 there) and the softmax of its two-GEMM attention, attn_softmax_rows!
 * (attention.jl:528-615), which takes the scale. */
int mi_softmax_f16(void *out, const void *a, int dtype, int64_t n, int64_t rows, float scale, void *stream);
/* out = fp16(a * c) over n contiguous elements: aten::mul.Tensor / div.Tensor with a constant (the emit() broadcast of
 * ops.jl's elementwise handlers). */
int mi_scale_f16(void *out, const void *a, float c, int64_t n, void *stream);
/* out = fp16(act(a)) over n contiguous elements, act one of enum mi_epilogue: an activation no GEMM or convolution
 * store could take (aten::gelu / relu after a strided convolution; ops.jl:1698-1702, 1683). */
int mi_act_f16(void *out, const void *a, int epi, int64_t n, void *stream);
/* out = min(max(a, lo), hi): aten::clamp, the fp16 overflow guard of exported encoder layers (ops.jl:300-310). */
int mi_clamp_f16(void *out, const void *a, float lo, float hi, int64_t n, void *stream);
/* out = fp16(a + b), n elements: the residual add.Tensor in the operand type
 * (ops.jl:186-197), for callers that do not fold it into the GEMM store. */
int mi_add_f16(void *out, const void *a, const void *b, int64_t n, void *stream);

/* ---- decode-step cache maintenance ------------------------------------------
 * The reference's decoder step is functional: the exported graph writes the new
 * token's K/V with index_put, returns the whole cache through cat, and
 * decodestep! copies ~18 MB back per token (WhisperRunner/src/decode.jl:186-203).
 * These two calls replace that round trip with an in-place write driven by a
 * device-resident length per batch row, the same int32 array mi_sdpa_f16 takes
 * as kv_len -- so a step enqueues identical work whatever the position, and a
 * captured graph of it can be replayed (the reference's Lava.capture/replay,
 * plans/whisper-decoder.md:244-259).
 *
 * Order within a step: mi_kv_advance(+1) once, then per layer mi_kv_append_f16
 * (writes slot kv_len[b]-1) and attention with kv_len.
 *
 * cache_k/cache_v: (E, Lmax, H, B) with element strides cache_strides, E contiguous.
 * k_new/v_new: (E, 1, H, B) with element strides new_strides (the L stride is unused).
 * A row whose kv_len is 0 or exceeds Lmax is left untouched: a caller that advances with cap = Lmax + 1 gets
 * "length Lmax + 1" as the mark of a step that found the cache full -- nothing stored (here and in
 * mi_sdpa_append_f16), attention over the Lmax stored keys -- and can read it back; with cap = Lmax the counter
 * saturates silently and each further step overwrites the last slot. */
int mi_kv_append_f16(void *cache_k, void *cache_v, const int64_t cache_strides[4], int64_t Lmax,
                     const void *k_new, const void *v_new, const int64_t new_strides[4],
                     const int32_t *kv_len, int64_t E, int64_t H, int64_t B, void *stream);

/* mi_kv_append_f16 and mi_sdpa_f16 (Lq = 1) in one launch, for the decoder's self-attention: the key/value row of
 * the newest token (k_new, v_new: 1 x E per head and batch, element strides new_strides as (E, L, H, B)) is taken
 * as key kv_len[b] - 1 and written into that slot of the cache on the way; out = attention of q over the first
 * kv_len[b] keys.  cache_k / cache_v are written to.  Only what the single-launch kernel covers (E <= 64, at most
 * 4096 (head, batch) rows, 16-byte addressable rows); MI_DECLINE_UNSUPPORTED otherwise, and the caller makes the two
 * calls.  The key range may be cut over several workgroups per row that merge inside the launch through counters and
 * partials in a static device array (16 banks taken in turn: more than 16 such launches -- this call or mi_sdpa_f16
 * with Lq = 1 -- in flight together on one GPU would share a bank and race).
 * Replaces index_put + cat + scaled_dot_product_attention of the exported decoder step
 * (WhisperRunner/src/decode.jl:186-203, tools/export_whisper_decoder.py). */
int mi_sdpa_append_f16(void *out, int out_dtype, const int64_t out_strides[4],
                       const void *q, const int64_t q_strides[4],
                       void *cache_k, const int64_t k_strides[4], void *cache_v, const int64_t v_strides[4],
                       const void *k_new, const void *v_new, const int64_t new_strides[4],
                       const int32_t *kv_len, int64_t E, int64_t Lk, int64_t H, int64_t B, float scale, void *stream);
/* kv_len[b] = clamp(kv_len[b] + delta, 0, cap) for b < B, on the device
 * (KVCache.position += 1, decode.jl:201, without the host in the loop). */
int mi_kv_advance(int32_t *kv_len, int64_t B, int32_t delta, int32_t cap, void *stream);
/* kv_len[b] = clamp(position[b] + 1, 0, cap) for b < B, on the device; npos = 1 (one position for every row, as
 * the exported step's cache_position input has it) or B.  The exported decoder step names the slot its new token
 * is written to (cache_position, int64; tools/export_whisper_decoder.py:158-181, decode.jl:186-203); the kernels
 * here count valid keys, which is that slot + 1.  mi_kv_advance saturates at cap, and so does this: a caller that
 * steps past the capacity overwrites the last slot, unless cap = capacity + 1 is passed (see mi_kv_append_f16). */
int mi_kv_len_from_position(int32_t *kv_len, const int64_t *position, int64_t npos, int64_t B, int32_t cap, void *stream);

/* out[i, :] = table[ids[i], :] (+ table2[ids2[i], :], or table2[ids2[0], :] when n2 = 1) for i < n: rows of D
 * contiguous fp16 elements, int64 ids, tables V x D and V2 x D, table2 = NULL for a plain gather; the sum is fp32,
 * rounded once.  aten::embedding (embedding_kernel!, ops.jl:1754-1783), the row gather of aten::index.Tensor along
 * the first axis (ops.jl:1524-1640), and -- with both tables -- the decoder step's token embedding + position
 * embedding (tools/export_whisper_decoder.py:150-152) in one launch.  An id outside its table contributes a row
 * of zeros (torch raises there; the reference reads out of bounds). */
int mi_embedding_f16(void *out, const void *table, const int64_t *ids, int64_t n, int64_t D, int64_t V,
                     const void *table2, const int64_t *ids2, int64_t n2, int64_t V2, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355DNN_H */
