// Masked prefix+suffix attention over the resident KV cache (gfx950).
//
// out = softmax(scale * Q K^T + mask) V, one pass over the keys with an online
// softmax, fp32 scores / statistics / accumulation in every mode (the
// reference's precision split, src/act_dtype.h:29-35).
//
// Work decomposition.  A workgroup owns one (batch, kv head) and a group of
// 32-row tiles of that head's query rows; the rows of all g = Hq/Hkv query
// heads sharing the kv head are flattened (row = head_in_group * S + s), so a
// K/V tile staged in LDS is read once per query-head group (GQA / MQA sharing)
// instead of being copied per query head as bitvla_repeat_kv_bf16 does
// (src/kernels/bitvla/bitvla_lm_cuda.cu:181-190).  Each 64-lane wavefront owns
// one row tile.
//
// The cache layout makes both tiles plain block copies: K [t][D] of one head is
// contiguous, V^T [D][t] has the keys innermost.
//
// MFMA formulation (transposed, so softmax statistics are per lane):
//   S^T[key][row] = K . Q^T     A = K tile rows (lane r <-> key), B = Q rows
//   O^T[d][row]  += V^T . P^T   A = V^T rows (lane r <-> d),      B = P^T
// The 32x32 accumulator gives lane (g, r) the 16 keys 8j+4g+i of query row r,
// so row max / sum are 15 in-lane ops plus one exchange with lane r+32, and the
// probabilities are already in B-operand position for the second product: the
// k-slot (g, e) of that product is bound to key 8(e/4)+4g+(e%4), and V^T is
// fetched from LDS in the same order.  No score matrix is ever written
// (the reference's explicit path writes and re-reads Hq*S*T scores).

#include <math.h>

#include "common.h"
#include "vla_kernels.h"

namespace {

using namespace vk;

constexpr int TK = 64;  // keys per LDS tile

struct AttnArgs {
    const void* q;
    const void* k_cache;
    const void* vt_cache;
    void* out;
    int batch, S, Hq, Hkv, t_max, n_keys;
    float scale;
    int mask_kind, n_prefix, pad_start, pad_end;
    const float* mask;
};

template <typename T> struct AT;
template <> struct AT<bf16_t> {
    static constexpr int EB = 2;
    static constexpr int CE = 16;  // k elements per MFMA group
    __device__ static __forceinline__ void mma(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                      acc, 0, 0, 0);
    }
    __device__ static __forceinline__ float fexp(float x) { return __expf(x); }
};
template <> struct AT<float> {
    static constexpr int EB = 4;
    static constexpr int CE = 8;
    __device__ static __forceinline__ void mma(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
        const f32x4_t fa = __builtin_bit_cast(f32x4_t, a), fb = __builtin_bit_cast(f32x4_t, b);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[t], fb[t], acc, 0, 0, 0);
    }
    __device__ static __forceinline__ float fexp(float x) { return expf(x); }
};

template <typename T, int D, int NW>
__global__ void __launch_bounds__(NW * 64) attn_kernel(AttnArgs a) {
    typedef AT<T> A;
    constexpr int EB = A::EB, CE = A::CE;
    constexpr int DP = (D + 31) / 32 * 32;  // head_dim padded to whole 32-row output blocks
    constexpr int NQ = D / CE;              // MFMA groups along head_dim
    constexpr int NDB = DP / 32;            // 32-row blocks of O^T
    constexpr int KS = D * EB + 16;         // LDS stride of a K row (bytes)
    constexpr int VS = TK * EB + 16;        // LDS stride of a V^T row (bytes)
    constexpr int NT = NW * 64;
    static_assert(D % CE == 0 && (D * EB) % 16 == 0, "head_dim must be whole MFMA groups and 16-byte rows");

    __shared__ __attribute__((aligned(16))) unsigned char ldsK[TK * KS];
    __shared__ __attribute__((aligned(16))) unsigned char ldsV[DP * VS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 5, r = lane & 31;
    const int hk = blockIdx.y, b = blockIdx.z;
    const int grp = a.Hq / a.Hkv;
    const int R = grp * a.S;
    const int row = (blockIdx.x * NW + wave) * 32 + r;
    const bool wave_active = (blockIdx.x * NW + wave) * 32 < R;
    const bool row_valid = row < R;
    const int hg = row_valid ? row / a.S : 0;
    const int s = row_valid ? row % a.S : 0;
    const int h = hk * grp + hg;

    // Q fragments: B operand, lane (g, r) holds 16 bytes of query row r per group.
    u32x4_t qf[NQ];
    {
        const unsigned char* qrow = (const unsigned char*)a.q + (((long)b * a.S + s) * a.Hq + h) * D * EB;
#pragma unroll
        for (int c = 0; c < NQ; ++c) {
            u32x4_t z = {0u, 0u, 0u, 0u};
            qf[c] = row_valid ? *reinterpret_cast<const u32x4_t*>(qrow + (c * CE + g * (CE / 2)) * EB) : z;
        }
    }

    f32x16_t o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const unsigned char* kbase = (const unsigned char*)a.k_cache + ((long)b * a.Hkv + hk) * a.t_max * D * EB;
    const unsigned char* vbase = (const unsigned char*)a.vt_cache + ((long)b * a.Hkv + hk) * D * (long)a.t_max * EB;

    for (int k0 = 0; k0 < a.n_keys; k0 += TK) {
        __syncthreads();  // previous tile fully consumed
        // K tile: TK rows of D*EB contiguous bytes.
        constexpr int KV_PER_ROW = D * EB / 16;
        for (int v = tid; v < TK * KV_PER_ROW; v += NT) {
            const int key = v / KV_PER_ROW, c = v % KV_PER_ROW;
            u32x4_t val = {0u, 0u, 0u, 0u};
            if (k0 + key < a.n_keys) val = *reinterpret_cast<const u32x4_t*>(kbase + ((long)(k0 + key) * D * EB) + c * 16);
            *reinterpret_cast<u32x4_t*>(ldsK + key * KS + c * 16) = val;
        }
        // V^T tile: D rows of TK keys; keys past n_keys are zeroed element-wise so
        // that stale cache contents cannot reach the accumulators.
        constexpr int VV_PER_ROW = TK * EB / 16;
        constexpr int EPV = 16 / EB;  // elements per vector
        for (int v = tid; v < D * VV_PER_ROW; v += NT) {
            const int d = v / VV_PER_ROW, c = v % VV_PER_ROW;
            const int key = k0 + c * EPV;
            u32x4_t val = {0u, 0u, 0u, 0u};
            if (key < a.n_keys) {
                val = *reinterpret_cast<const u32x4_t*>(vbase + ((long)d * a.t_max + key) * EB);
                if (key + EPV > a.n_keys) {
                    const int nvalid = a.n_keys - key;
                    if (EB == 2) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t lo = (2 * e < nvalid) ? 0xffffu : 0u, hi = (2 * e + 1 < nvalid) ? 0xffff0000u : 0u;
                            val[e] &= (lo | hi);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (e >= nvalid) val[e] = 0u;
                    }
                }
            }
            *reinterpret_cast<u32x4_t*>(ldsV + d * VS + c * 16) = val;
        }
        __syncthreads();
        if (!wave_active) continue;

        // ---- scores S^T for the two 32-key blocks of the tile
        float p[2][16];
        float m_tile = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            f32x16_t sc;
#pragma unroll
            for (int i = 0; i < 16; ++i) sc[i] = 0.f;
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(ldsK + (kb * 32 + r) * KS + (c * CE + g * (CE / 2)) * EB);
                A::mma(sc, kf, qf[c]);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = k0 + kb * 32 + 8 * j + 4 * g + i;
                    float v = sc[4 * j + i] * a.scale;
                    bool blocked = key >= a.n_keys;
                    if (a.mask) {
                        if (!blocked) v += a.mask[(long)s * a.n_keys + key];
                    } else if (key < a.n_prefix) {
                        blocked |= (key >= a.pad_start && key < a.pad_end);
                    } else {
                        const int si = key - a.n_prefix;
                        if (a.mask_kind == VLA_MASK_CAUSAL_SUFFIX) blocked |= si > s;
                        else if (a.mask_kind == VLA_MASK_PI0_STATE) blocked |= (s == 0 && si != 0);
                    }
                    v = blocked ? -INFINITY : v;
                    p[kb][4 * j + i] = v;
                    m_tile = fmaxf(m_tile, v);
                }
        }
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
        const float m_new = fmaxf(m_run, m_tile);
        // m_new == -inf: nothing visible yet, keep everything at zero.
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = A::fexp(m_run - m_use);  // exp(-inf) = 0 on the first visible tile
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = A::fexp(p[kb][i] - m_use);
                p[kb][i] = e;
                psum += e;
            }
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[db][i] *= alpha;

        // ---- O^T += V^T . P^T
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (EB == 2) {
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    // The probabilities enter the bf16 MFMA as hi + lo (two bf16 terms,
                    // ~16 mantissa bits): the P.V product then matches an fp32-probability
                    // reference instead of carrying an extra 2^-9 rounding per weight.
                    const float* pp = &p[kb][hh * 8];
                    float lo[8];
                    uint32_t hi16[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        hi16[e] = f2bf(pp[e]);
                        lo[e] = pp[e] - bf2f((bf16_t)hi16[e]);
                    }
                    const u32x4_t pf = {hi16[0] | (hi16[1] << 16), hi16[2] | (hi16[3] << 16), hi16[4] | (hi16[5] << 16),
                                        hi16[6] | (hi16[7] << 16)};
                    const u32x4_t pl = {pack_bf2(lo[0], lo[1]), pack_bf2(lo[2], lo[3]), pack_bf2(lo[4], lo[5]),
                                        pack_bf2(lo[6], lo[7])};
                    const int key_off = (kb * 32 + hh * 16 + 4 * g) * EB;
#pragma unroll
                    for (int db = 0; db < NDB; ++db) {
                        const unsigned char* vr = ldsV + (db * 32 + r) * VS + key_off;
                        const u32x2_t v0 = *reinterpret_cast<const u32x2_t*>(vr);
                        const u32x2_t v1 = *reinterpret_cast<const u32x2_t*>(vr + 8 * EB);
                        const u32x4_t vf = {v0[0], v0[1], v1[0], v1[1]};
                        A::mma(o[db], vf, pf);
                        A::mma(o[db], vf, pl);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float* pp = &p[kb][4 * j];
                    const u32x4_t pf = {__float_as_uint(pp[0]), __float_as_uint(pp[1]), __float_as_uint(pp[2]),
                                        __float_as_uint(pp[3])};
                    const int key_off = (kb * 32 + 8 * j + 4 * g) * EB;
#pragma unroll
                    for (int db = 0; db < NDB; ++db) {
                        const u32x4_t vf = *reinterpret_cast<const u32x4_t*>(ldsV + (db * 32 + r) * VS + key_off);
                        A::mma(o[db], vf, pf);
                    }
                }
            }
        }
    }

    if (!row_valid) return;
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    unsigned char* orow = (unsigned char*)a.out + (((long)b * a.S + s) * a.Hq + h) * D * EB;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = db * 32 + 8 * j + 4 * g;
            if (d >= D) continue;
            const float v0 = o[db][4 * j] * inv, v1 = o[db][4 * j + 1] * inv, v2 = o[db][4 * j + 2] * inv,
                        v3 = o[db][4 * j + 3] * inv;
            if (EB == 2) {
                const u32x2_t pk = {pack_bf2(v0, v1), pack_bf2(v2, v3)};
                *reinterpret_cast<u32x2_t*>(orow + d * EB) = pk;
            } else {
                const f32x4_t pk = {v0, v1, v2, v3};
                *reinterpret_cast<f32x4_t*>(orow + d * EB) = pk;
            }
        }
}

template <typename T, int D>
int launch_d(const AttnArgs& a, vla_stream_t stream) {
    const int R = (a.Hq / a.Hkv) * a.S;
    const int n_tiles = (R + 31) / 32;
    // Fewer wavefronts per workgroup -> more workgroups; go down until the grid
    // covers the 256 compute units, but keep at least two wavefronts loading.
    const long pairs = (long)a.batch * a.Hkv;
    int nw = 4;
    if (n_tiles < 4 || pairs * ((n_tiles + 3) / 4) < 512) nw = 2;
    if (n_tiles < 2) nw = 1;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((n_tiles + nw - 1) / nw, a.Hkv, a.batch);
    if (nw == 4) attn_kernel<T, D, 4><<<grid, 256, 0, st>>>(a);
    else if (nw == 2) attn_kernel<T, D, 2><<<grid, 128, 0, st>>>(a);
    else attn_kernel<T, D, 1><<<grid, 64, 0, st>>>(a);
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

template <typename T>
int launch_t(const AttnArgs& a, int D, vla_stream_t stream) {
    switch (D) {
        case 48: return launch_d<T, 48>(a, stream);
        case 64: return launch_d<T, 64>(a, stream);
        case 128: return launch_d<T, 128>(a, stream);
        case 256:
            // fp32 tiles of 256-wide heads would not fit the LDS budget; only bf16 is built.
            if constexpr (sizeof(T) == 2) return launch_d<T, 256>(a, stream);
            else return VLA_K_ERR_SHAPE;
        default: return VLA_K_ERR_SHAPE;
    }
}

}  // namespace

extern "C" int vla_attn_prefix_suffix(const void* q, const void* k_cache, const void* vt_cache, void* out, int dtype,
                                      int batch, int S, int n_q_heads, int n_kv_heads, int head_dim, int t_max,
                                      int n_keys, float scale, int mask_kind, int n_prefix, int pad_start, int pad_end,
                                      const float* mask, vla_stream_t stream) {
    if (!q || !k_cache || !vt_cache || !out || batch < 0 || S <= 0 || n_q_heads <= 0 || n_kv_heads <= 0)
        return VLA_K_ERR_ARG;
    if (n_q_heads % n_kv_heads || t_max % 8 || n_keys <= 0 || n_keys > t_max) return VLA_K_ERR_SHAPE;
    if (mask_kind < VLA_MASK_NONE || mask_kind > VLA_MASK_PI0_STATE) return VLA_K_ERR_ARG;
    if (batch == 0) return VLA_K_OK;
    AttnArgs a;
    a.q = q; a.k_cache = k_cache; a.vt_cache = vt_cache; a.out = out;
    a.batch = batch; a.S = S; a.Hq = n_q_heads; a.Hkv = n_kv_heads; a.t_max = t_max; a.n_keys = n_keys;
    a.scale = scale; a.mask_kind = mask_kind;
    a.n_prefix = n_prefix < 0 ? 0 : (n_prefix > n_keys ? n_keys : n_prefix);
    a.pad_start = pad_start; a.pad_end = pad_end; a.mask = mask;
    if (dtype == VLA_DT_BF16) return launch_t<bf16_t>(a, head_dim, stream);
    if (dtype == VLA_DT_F32) return launch_t<float>(a, head_dim, stream);
    return VLA_K_ERR_ARG;
}
