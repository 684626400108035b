// In-place KV-cache maintenance for a decode step.
//
// The reference's decoder graph is functional: it takes the self-attention cache, writes the new
// token's K and V with index_put, returns the whole cache through cat, and the host copies ~18 MB
// back per token (WhisperRunner/src/decode.jl:186-203, tools/export_whisper_decoder.py).  Here the
// cache is device state: a length counter per batch row lives in device memory, a step first
// advances it, then writes the new rows at slot length-1, and the attention kernels read the same
// counter as their kv_len.  Nothing on the host changes from step to step, so a captured graph of
// the step replays as is.
#include "common.hpp"

namespace {

// grid (H, B); one 16-byte chunk (or one element) of the new K row and V row per thread.
template <bool VEC>
__global__ __launch_bounds__(64) void kv_append_kernel(half_t *ck, half_t *cv, const half_t *nk, const half_t *nv,
                                                       long cs1, long cs2, long cs3, long ns2, long ns3,
                                                       const int *kv_len, int E, int Lmax) {
    const int h = blockIdx.x, b = blockIdx.y;
    const int slot = kv_len[b] - 1;
    if (slot < 0 || slot >= Lmax) return;      // length 0 (never advanced) or a corrupt counter: nothing is written
    const long dst = (long)b * cs3 + (long)h * cs2 + (long)slot * cs1;
    const long src = (long)b * ns3 + (long)h * ns2;
    if (VEC) {
        for (int c = threadIdx.x; c < E / 8; c += 64) {
            *reinterpret_cast<u32x4 *>(ck + dst + c * 8) = ldg16(nk + src + c * 8);
            *reinterpret_cast<u32x4 *>(cv + dst + c * 8) = ldg16(nv + src + c * 8);
        }
    } else {
        for (int e = threadIdx.x; e < E; e += 64) { ck[dst + e] = nk[src + e]; cv[dst + e] = nv[src + e]; }
    }
}

__global__ void kv_advance_kernel(int *kv_len, int n, int delta, int cap) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int v = kv_len[i] + delta;
        kv_len[i] = v < 0 ? 0 : v > cap ? cap : v;
    }
}

// kv_len[b] = position + 1 (the new token's slot counts), one position for every row or one per row.
__global__ void kv_len_from_position_kernel(int *kv_len, const long long *pos, int npos, int n, int cap) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const long long v = pos[npos == 1 ? 0 : i] + 1;
        kv_len[i] = v < 0 ? 0 : v > cap ? cap : (int)v;
    }
}

// One workgroup per gathered row; 16-byte chunks where the row length and the pointers allow, else single elements.
// An id outside its table contributes a row of zeros.
template <bool VEC>
__global__ __launch_bounds__(256) void embedding_kernel(half_t *out, const half_t *t1, const long long *ids1, long V1,
                                                        const half_t *t2, const long long *ids2, long n2, long V2, int D) {
    const long i = blockIdx.x;
    const long long r1 = ids1[i];
    const bool ok1 = r1 >= 0 && r1 < V1;
    const half_t *a = t1 + (ok1 ? r1 : 0) * (long)D;
    const half_t *b = nullptr;
    if (t2) {
        const long long r2 = ids2[n2 == 1 ? 0 : i];
        if (r2 >= 0 && r2 < V2) b = t2 + r2 * (long)D;
    }
    half_t *o = out + i * (long)D;
    if (VEC) {
        for (int c = threadIdx.x; c < D / 8; c += 256) {
            half8v x = {0, 0, 0, 0, 0, 0, 0, 0};
            if (ok1) x = *reinterpret_cast<const half8v *>(a + c * 8);
            if (b) {
                const half8v y = *reinterpret_cast<const half8v *>(b + c * 8);
#pragma unroll
                for (int j = 0; j < 8; j++) x[j] = (half_t)((float)x[j] + (float)y[j]);
            }
            *reinterpret_cast<half8v *>(o + c * 8) = x;
        }
    } else {
        for (int e = threadIdx.x; e < D; e += 256) {
            float x = ok1 ? (float)a[e] : 0.f;
            if (b) x += (float)b[e];
            o[e] = (half_t)x;
        }
    }
}

}  // namespace

extern "C" {

int mi_kv_append_f16(void *cache_k, void *cache_v, const int64_t cache_strides[4], int64_t Lmax,
                     const void *k_new, const void *v_new, const int64_t new_strides[4],
                     const int32_t *kv_len, int64_t E, int64_t H, int64_t B, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!cache_k || !cache_v || !k_new || !v_new || !cache_strides || !new_strides || !kv_len) return MI_DECLINE_OPERANDS;
    if (E < 1 || H < 1 || B < 1 || Lmax < 1 || H > 65535 || B > 65535 || E > INT32_MAX || Lmax > INT32_MAX) return MI_DECLINE_EXTENT;
    if (cache_strides[0] != 1 || new_strides[0] != 1) return MI_DECLINE_OPERANDS;     // head-dim contiguous on both sides
    const bool vec = E % 8 == 0 && cache_strides[1] % 8 == 0 && cache_strides[2] % 8 == 0 && cache_strides[3] % 8 == 0 &&
                     new_strides[2] % 8 == 0 && new_strides[3] % 8 == 0 &&
                     aligned_to(cache_k, 16) && aligned_to(cache_v, 16) && aligned_to(k_new, 16) && aligned_to(v_new, 16);
    dim3 grid((unsigned)H, (unsigned)B);
    hipStream_t st = (hipStream_t)stream;
    if (vec) hipLaunchKernelGGL(kv_append_kernel<true>, grid, dim3(64), 0, st, (half_t *)cache_k, (half_t *)cache_v, (const half_t *)k_new, (const half_t *)v_new,
                                (long)cache_strides[1], (long)cache_strides[2], (long)cache_strides[3], (long)new_strides[2], (long)new_strides[3], kv_len, (int)E, (int)Lmax);
    else     hipLaunchKernelGGL(kv_append_kernel<false>, grid, dim3(64), 0, st, (half_t *)cache_k, (half_t *)cache_v, (const half_t *)k_new, (const half_t *)v_new,
                                (long)cache_strides[1], (long)cache_strides[2], (long)cache_strides[3], (long)new_strides[2], (long)new_strides[3], kv_len, (int)E, (int)Lmax);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_kv_advance(int32_t *kv_len, int64_t B, int32_t delta, int32_t cap, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!kv_len) return MI_DECLINE_OPERANDS;
    if (B < 1 || B > INT32_MAX || cap < 0) return MI_DECLINE_EXTENT;
    hipLaunchKernelGGL(kv_advance_kernel, dim3((unsigned)ceil_div(B, 64)), dim3(64), 0, (hipStream_t)stream, kv_len, (int)B, delta, cap);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_kv_len_from_position(int32_t *kv_len, const int64_t *position, int64_t npos, int64_t B, int32_t cap, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!kv_len || !position) return MI_DECLINE_OPERANDS;
    if (B < 1 || B > INT32_MAX || cap < 0 || (npos != 1 && npos != B)) return MI_DECLINE_EXTENT;
    hipLaunchKernelGGL(kv_len_from_position_kernel, dim3((unsigned)ceil_div(B, 64)), dim3(64), 0, (hipStream_t)stream, kv_len,
                       (const long long *)position, (int)npos, (int)B, cap);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

int mi_embedding_f16(void *out, const void *table, const int64_t *ids, int64_t n, int64_t D, int64_t V,
                     const void *table2, const int64_t *ids2, int64_t n2, int64_t V2, void *stream) {
    if (!mi_ready()) return MI_ERROR_DEVICE;
    if (!out || !table || !ids || (table2 && !ids2)) return MI_DECLINE_OPERANDS;
    if (n < 1 || n > INT32_MAX || D < 1 || D > INT32_MAX || V < 1) return MI_DECLINE_EXTENT;
    if (table2 && (V2 < 1 || (n2 != 1 && n2 != n))) return MI_DECLINE_EXTENT;
    const bool vec = D % 8 == 0 && aligned_to(out, 16) && aligned_to(table, 16) && (!table2 || aligned_to(table2, 16));
    hipStream_t st = (hipStream_t)stream;
    if (vec) hipLaunchKernelGGL(embedding_kernel<true>, dim3((unsigned)n), dim3(256), 0, st, (half_t *)out, (const half_t *)table, (const long long *)ids,
                                (long)V, (const half_t *)table2, (const long long *)ids2, (long)n2, (long)V2, (int)D);
    else     hipLaunchKernelGGL(embedding_kernel<false>, dim3((unsigned)n), dim3(256), 0, st, (half_t *)out, (const half_t *)table, (const long long *)ids,
                                (long)V, (const half_t *)table2, (const long long *)ids2, (long)n2, (long)V2, (int)D);
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERROR_LAUNCH;
}

}  // extern "C"
