// Measurement kernels (no counterpart in the reference): what the matrix units and the memory system of THIS box
// deliver when nothing else is in the way, so that a benchmark can print the ceilings next to its results instead
// of assuming the vendor's figures.
//
//   probe_mfma_kernel   the arithmetic of the 128 x 256 GEMM tile with every memory operation removed: eight waves
//                       per workgroup, two per SIMD, each with a 2 x 2 block of 32 x 32 accumulators and, per 64-deep
//                       step, sixteen v_mfma_f32_32x32x16_f16 on operand fragments that sit in registers (random
//                       fp16 values, so the multipliers toggle as they do on real data); optionally the GEMM's
//                       epilogue arithmetic (bias, rounding, erf-GELU on the rounded value) on all 64 values a lane
//                       holds.  Nothing is stored unless the results are impossible, which the compiler cannot know.
//   probe_copy_kernel   out[i] = in[i], sixteen bytes per lane and step: a kernel of known HBM traffic, for timing
//                       the memory system and for scaling the FETCH_SIZE / WRITE_SIZE counters of rocprofv3.
#include "common.hpp"

namespace {

__global__ __launch_bounds__(512, 2) void probe_mfma_kernel(float *sink, const half_t *seed, int steps, int gelu) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // operand fragments of the four k-steps of a 64-deep step: 2 of A and 2 of B each, distinct random values per lane
    half8v fa[4][2], fb[4][2];
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            fa[ks][j] = *reinterpret_cast<const half8v *>(seed + (((ks * 2 + j) * 8 + wave) * 64 + lane) * 8);
            fb[ks][j] = *reinterpret_cast<const half8v *>(seed + (((8 + ks * 2 + j) * 8 + wave) * 64 + lane) * 8);
        }
    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    for (int s = 0; s < steps; s++) {
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ks][i], fa[ks][j], acc[i][j], 0, 0, 0);
        // keeps the loop a loop (no hoisting of the whole chain) without touching memory
        asm volatile("" : "+v"(fa[0][0]));
    }
    float t = 0.0f;
    const float bias = (float)fa[0][0][0];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float v = acc[i][j][r] * 1e-3f;
                if (gelu) v = (float)(half_t)gelu_erf((float)(half_t)(v + bias));
                t += v;
            }
    if (t == 12345.6789f) sink[blockIdx.x * 512 + threadIdx.x] = t;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(u32x4 *out, const u32x4 *in, long n16) {
    const long stride = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) out[i] = in[i];
}

// What a barrier across the whole grid costs on this device: `rounds` times, every workgroup adds itself to a counter
// in device memory (an agent-scope atomic: the XCDs' L2s are not coherent with each other, so it is performed beyond
// them) and polls it until all have arrived; with `payload`, every workgroup first publishes 16 bytes with write-through
// stores and afterwards reads all of them back past its L2 -- the exchange a multi-phase kernel would need between phases
// (a decode step's 2.5 KB activation row).  Every wait is bounded: a workgroup that gives up raises the sticky status word
// and runs on without waiting, so the grid drains whatever happens.  The grid must be resident at once (<= one
// workgroup per compute unit).
__global__ __launch_bounds__(64) void probe_grid_barrier_kernel(unsigned *counter, unsigned *data, unsigned *status, int rounds, int payload, int spin_limit) {
    const unsigned G = gridDim.x;
    bool gave_up = false;
    unsigned acc = 0;
    for (int r = 0; r < rounds; r++) {
        if (payload && threadIdx.x < 4)
            __hip_atomic_store(data + ((r & 1) * G + blockIdx.x) * 4 + threadIdx.x, (unsigned)(r * 131 + blockIdx.x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (threadIdx.x == 0 && !gave_up) {
            __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned want = (unsigned)(r + 1) * G;
            int spins = 0;
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
                if (++spins > spin_limit) { gave_up = true; __hip_atomic_fetch_or(status, (unsigned)MI_DEVSTAT_STEP_BARRIER, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break; }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
        if (payload) {
            for (unsigned i = threadIdx.x; i < G * 4; i += 64) acc += __hip_atomic_load(data + (r & 1) * G * 4 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (acc == 0x12345u) data[0] = acc;
}

// The same barrier in two levels, so that no address sees more than 32 arrivals or 32 pollers: a workgroup adds itself to
// the counter of its group (workgroup index mod 8: on a device that deals workgroups to its XCDs round robin, its XCD),
// the last arrival of a group adds the group to the counter of groups, the last group releases everyone by writing the
// round's number into each group's flag, and a workgroup polls its own group's flag.  Counters and flags sit 128 bytes
// apart (`lines`: word 32 x (1 + g) the counter of group g, word 32 x 9 the counter of groups, word 32 x (10 + g) the
// flag of group g); they only ever grow, so nothing is reset between rounds.  Waits are bounded like the flat form's.
__global__ __launch_bounds__(64) void probe_grid_barrier2_kernel(unsigned *lines, unsigned *data, unsigned *status, int rounds, int payload, int spin_limit) {
    const unsigned G = gridDim.x, grp = blockIdx.x & 7u;
    const unsigned ngrp = G < 8u ? G : 8u, members = (G - grp + 7u) / 8u;
    unsigned *mine = lines + 32 * (1 + grp), *groups = lines + 32 * 9, *flag = lines + 32 * (10 + grp);
    bool gave_up = false;
    unsigned acc = 0;
    for (int r = 0; r < rounds; r++) {
        if (payload && threadIdx.x < 4)
            __hip_atomic_store(data + ((r & 1) * G + blockIdx.x) * 4 + threadIdx.x, (unsigned)(r * 131 + blockIdx.x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (threadIdx.x == 0 && !gave_up) {
            const unsigned round1 = (unsigned)(r + 1);
            if (__hip_atomic_fetch_add(mine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == round1 * members - 1u) {
                if (__hip_atomic_fetch_add(groups, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == round1 * ngrp - 1u) {
                    for (unsigned g = 0; g < ngrp; g++)
                        __hip_atomic_store(lines + 32 * (10 + g), round1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            int spins = 0;
            while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < round1) {
                if (++spins > spin_limit) { gave_up = true; __hip_atomic_fetch_or(status, (unsigned)MI_DEVSTAT_STEP_BARRIER, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break; }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
        if (payload) {
            for (unsigned i = threadIdx.x; i < G * 4; i += 64) acc += __hip_atomic_load(data + (r & 1) * G * 4 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (acc == 0x12345u) data[0] = acc;
}

}  // namespace

extern "C" {

int mi_probe_mfma(void *sink, const void *seed_f16, int64_t workgroups, int64_t steps, int gelu, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!sink || !seed_f16 || !aligned_to(seed_f16, 16)) return MI_DECLINE_OPERANDS;
    if (workgroups < 1 || workgroups > (1 << 20) || steps < 1 || steps > (1 << 24)) return MI_DECLINE_EXTENT;
    hipLaunchKernelGGL(probe_mfma_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,
                       reinterpret_cast<float *>(sink), reinterpret_cast<const half_t *>(seed_f16), (int)steps, gelu);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_probe_grid_barrier(void *scratch_u32, int64_t workgroups, int64_t rounds, int payload, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!scratch_u32 || !aligned_to(scratch_u32, 16)) return MI_DECLINE_OPERANDS;
    if (workgroups < 1 || workgroups > mi_num_cus() || rounds < 1 || rounds > 100000 || payload < 0 || payload > 3) return MI_DECLINE_EXTENT;
    // [0]: counter, [4]: status; flat form: two rounds of payload from word 16; two-level form: its counters and flags in
    // words 32 .. 32 x 18, the payload behind them
    unsigned *base = reinterpret_cast<unsigned *>(scratch_u32);
    hipStream_t st = (hipStream_t)stream;
    const bool two_level = (payload & 2) != 0;
    if (hipMemsetAsync(base, 0, two_level ? 32 * 18 * 4 : 64, st) != hipSuccess) return MI_ERROR_LAUNCH;
    if (two_level) hipLaunchKernelGGL(probe_grid_barrier2_kernel, dim3((unsigned)workgroups), dim3(64), 0, st, base, base + 32 * 18, base + 4, (int)rounds, payload & 1, 1 << 16);
    else           hipLaunchKernelGGL(probe_grid_barrier_kernel, dim3((unsigned)workgroups), dim3(64), 0, st, base, base + 16, base + 4, (int)rounds, payload & 1, 1 << 16);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_probe_copy(void *out, const void *in, size_t bytes, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !in || !aligned_to(out, 16) || !aligned_to(in, 16) || bytes % 16) return MI_DECLINE_OPERANDS;
    if (bytes == 0) return MI_OK;
    const long n16 = (long)(bytes / 16);
    const long want = ceil_div(n16, 256 * 8), cap = (long)mi_num_cus() * 16;
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)(want < cap ? want : cap)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<u32x4 *>(out), reinterpret_cast<const u32x4 *>(in), n16);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

}  // extern "C"
