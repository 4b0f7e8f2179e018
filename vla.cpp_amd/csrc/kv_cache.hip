// Resident KV cache: in-place suffix append and gather (bit-exact copies).
//
// Replaces the per-layer, per-step ggml_concat(cached_K, k_rope, 2) /
// ggml_concat(cached_V, v_h, 2) of the reference (src/models/smolvla.cpp:832-833,
// src/models/pi0.cpp:198-201): the prefix stays where it was written, only the
// S suffix tokens move.
//
// Layouts: K [B][Hkv][t_max][D] (a head's keys are one contiguous block, so an
// attention workgroup streams it with full 128-byte lines); V^T
// [B][Hkv][D][t_max] (keys innermost, the order the P.V contraction reads).
// Sources / destinations of these two kernels are token-major
// [B][n_tok][Hkv][D].

#include "common.h"
#include "vla_kernels.h"

namespace {

using namespace vk;

// One thread per element of the token-major tensor; both caches in one pass.
template <typename T, bool kToCache>
__global__ void kv_move_kernel(T* __restrict__ k_cache, T* __restrict__ vt_cache, T* __restrict__ k_tok,
                               T* __restrict__ v_tok, int Hkv, int D, int t_max, int tok_offset, int n_tok,
                               long total) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int d = (int)(i % D);
    long r = i / D;
    const int h = (int)(r % Hkv);
    r /= Hkv;
    const int t = (int)(r % n_tok);
    const int b = (int)(r / n_tok);
    const long bh = (long)b * Hkv + h;
    const long ki = (bh * t_max + tok_offset + t) * D + d;
    const long vi = (bh * D + d) * t_max + tok_offset + t;
    if (kToCache) {
        if (k_tok) k_cache[ki] = k_tok[i];
        if (v_tok) vt_cache[vi] = v_tok[i];
    } else {
        if (k_tok) k_tok[i] = k_cache[ki];
        if (v_tok) v_tok[i] = vt_cache[vi];
    }
}

template <bool kToCache>
int kv_move(void* k_cache, void* vt_cache, void* k_tok, void* v_tok, int dtype, int batch, int Hkv, int D,
            int t_max, int tok_offset, int n_tok, vla_stream_t stream) {
    if (batch < 0 || Hkv <= 0 || D <= 0 || t_max <= 0 || tok_offset < 0 || n_tok < 0) return VLA_K_ERR_ARG;
    if ((k_tok && !k_cache) || (v_tok && !vt_cache)) return VLA_K_ERR_ARG;
    if (tok_offset + n_tok > t_max) return VLA_K_ERR_SHAPE;
    if (dtype != VLA_DT_F32 && dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    const long total = (long)batch * n_tok * Hkv * D;
    if (total == 0 || (!k_tok && !v_tok)) return VLA_K_OK;
    const int threads = 256;
    const unsigned blocks = (unsigned)((total + threads - 1) / threads);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VLA_DT_F32)
        kv_move_kernel<float, kToCache><<<blocks, threads, 0, st>>>((float*)k_cache, (float*)vt_cache, (float*)k_tok,
                                                                  (float*)v_tok, Hkv, D, t_max, tok_offset, n_tok,
                                                                  total);
    else
        kv_move_kernel<uint16_t, kToCache><<<blocks, threads, 0, st>>>((uint16_t*)k_cache, (uint16_t*)vt_cache,
                                                                     (uint16_t*)k_tok, (uint16_t*)v_tok, Hkv, D,
                                                                     t_max, tok_offset, n_tok, total);
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

}  // namespace

extern "C" int vla_kv_append(void* k_cache, void* vt_cache, const void* k_src, const void* v_src, int dtype,
                             int batch, int n_kv_heads, int head_dim, int t_max, int tok_offset, int n_tok,
                             vla_stream_t stream) {
    return kv_move<true>(k_cache, vt_cache, const_cast<void*>(k_src), const_cast<void*>(v_src), dtype, batch,
                         n_kv_heads, head_dim, t_max, tok_offset, n_tok, stream);
}

extern "C" int vla_kv_gather(const void* k_cache, const void* vt_cache, void* k_dst, void* v_dst, int dtype,
                             int batch, int n_kv_heads, int head_dim, int t_max, int tok_offset, int n_tok,
                             vla_stream_t stream) {
    return kv_move<false>(const_cast<void*>(k_cache), const_cast<void*>(vt_cache), k_dst, v_dst, dtype, batch,
                          n_kv_heads, head_dim, t_max, tok_offset, n_tok, stream);
}
