// MFMA projections for the attention path on gfx950.
//
// One 64x64 output tile per 256-thread workgroup (four 64-lane wavefronts, each
// a 32x32 MFMA accumulator), A and W tiles staged through padded LDS rows of
// 128 bytes, the next tile's global loads in flight while the current one is
// multiplied.  Three instantiations share the loop:
//
//   bf16 : v_mfma_f32_32x32x16_bf16                       (configs 1-3)
//   fp32 : v_mfma_f32_32x32x2_f32, full fp32 products     (config 0, 1e-5 bar)
//   int8 : v_mfma_i32_32x32x32_i8 against 2-bit ternary weights decoded while
//          they are staged (BitVLA, exact int32 accumulators)
//
// and three epilogues, all run from an LDS copy of the accumulator tile:
//
//   PLAIN   y = x.W^T + bias + residual        (ggml_mul_mat + add; Wo)
//   QKV     bias, NeoX RoPE on the Q and K columns, Q to a token-major buffer,
//           K / V straight into the resident cache at token tok_offset + s
//   TERNARY acc - 2*rowsum (code offset), optional raw int32 dump, bf16 out =
//           float(acc) / s[m] * ws[group]
//
// MFMA operand layout used throughout (64 lanes, g = lane / 32, r = lane % 32):
// a lane supplies 16 bytes of row r of its operand at k offset
// chunk*kChunk + g*(kChunk/2); the 32x32 result holds, in element 4j+i of lane
// (g, r), C[8j + 4g + i][r].

#include "common.h"
#include "vla_kernels.h"

namespace {

using namespace vk;

constexpr int BM = 64, BN = 64;
constexpr int ROW_BYTES = 128;             // bytes of K per tile row
constexpr int LDS_STRIDE = ROW_BYTES + 16; // padded row, keeps 16-byte reads conflict-free
constexpr int C_STRIDE = BN + 4;           // floats

enum { EPI_PLAIN = 0, EPI_QKV = 1, EPI_TERNARY = 2 };

struct GemmArgs {
    const void* A;
    const void* W;
    const float* bias;
    int M, N, K;
    // PLAIN
    const void* residual;
    void* Y;
    int out_bf16;
    // QKV
    int S, Hq, nk, nv, D;
    const float* cos_t;
    const float* sin_t;
    void* q_out;
    void* k_cache;
    void* vt_cache;
    int t_max, tok_offset, Hkv;
    // TERNARY
    int32_t* acc_out;
    const float* s;
    const int32_t* rowsum;
    const float* ws;
    int ws_num;
};

template <typename T> struct Traits;
template <> struct Traits<bf16_t> {
    typedef f32x16_t Acc;
    static constexpr int kElemBytes = 2;
    static constexpr int kChunkBytes = 32;  // bytes of k per MFMA group per row
    __device__ static __forceinline__ void mma(Acc& acc, const u32x4_t& a, const u32x4_t& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                      acc, 0, 0, 0);
    }
};
template <> struct Traits<float> {
    typedef f32x16_t Acc;
    static constexpr int kElemBytes = 4;
    static constexpr int kChunkBytes = 32;
    __device__ static __forceinline__ void mma(Acc& acc, const u32x4_t& a, const u32x4_t& b) {
        const f32x4_t fa = __builtin_bit_cast(f32x4_t, a), fb = __builtin_bit_cast(f32x4_t, b);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[t], fb[t], acc, 0, 0, 0);
    }
};
template <> struct Traits<int8_t> {
    typedef i32x16_t Acc;
    static constexpr int kElemBytes = 1;
    static constexpr int kChunkBytes = 32;
    __device__ static __forceinline__ void mma(Acc& acc, const u32x4_t& a, const u32x4_t& b) {
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, a), __builtin_bit_cast(i32x4_t, b), acc,
                                                   0, 0, 0);
    }
};

// Accumulator element -> raw 32-bit LDS cell (by value: a bit_cast applied
// directly to a vector element expression reads element 0).
__device__ __forceinline__ uint32_t acc_bits(float v) { return __float_as_uint(v); }
__device__ __forceinline__ uint32_t acc_bits(int v) { return (uint32_t)v; }

// W-row bases of the two 32-column halves of output tile `nt`.
struct TileCols {
    int base0, base1;  // rows of W feeding tile columns [0,32) and [32,64)
    int seg;           // 0 Q, 1 K, 2 V (QKV mode)
    int col0, col1;    // segment-local column of tile column 0 and of tile column 32
    bool rope;
};

template <int kEpi>
__device__ __forceinline__ TileCols tile_cols(const GemmArgs& a, int nt) {
    TileCols t;
    if (kEpi != EPI_QKV) {
        t.base0 = nt * BN;
        t.base1 = t.base0 + 32;
        t.seg = 0;
        t.col0 = t.base0;
        t.col1 = t.base1;
        t.rope = false;
        return t;
    }
    const int tq = a.Hq * a.D / BN, tk = a.nk * a.D / BN;
    int lt = nt, seg_base = 0;
    t.seg = 0;
    if (nt >= tq + tk) {
        t.seg = 2;
        lt = nt - tq - tk;
        seg_base = (a.Hq + a.nk) * a.D;
    } else if (nt >= tq) {
        t.seg = 1;
        lt = nt - tq;
        seg_base = a.Hq * a.D;
    }
    t.rope = (a.cos_t != nullptr) && t.seg != 2;
    if (t.rope) {
        const int tph = a.D / BN;  // tiles per head
        const int head = lt / tph, chunk = lt % tph;
        t.col0 = head * a.D + chunk * 32;
        t.col1 = t.col0 + a.D / 2;
    } else {
        t.col0 = lt * BN;
        t.col1 = t.col0 + 32;
    }
    t.base0 = seg_base + t.col0;
    t.base1 = seg_base + t.col1;
    return t;
}

template <typename T, int kEpi>
__global__ void __launch_bounds__(256) gemm_kernel(GemmArgs a) {
    typedef Traits<T> TR;
    constexpr int EB = TR::kElemBytes;
    constexpr int BK = ROW_BYTES / EB;  // k elements per tile

    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * BM * LDS_STRIDE];
    unsigned char* ldsA = lds;
    unsigned char* ldsW = lds + BM * LDS_STRIDE;
    static_assert(sizeof(float) * BM * C_STRIDE <= sizeof(lds), "C tile must fit in the operand buffers");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int g = lane >> 5, r = lane & 31;
    const int m0 = blockIdx.y * BM;
    const int nt = blockIdx.x;
    const TileCols tc = tile_cols<kEpi>(a, nt);

    typename TR::Acc acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0;

    const int nkt = (a.K + BK - 1) / BK;

    // Global -> register staging: two 16-byte vectors of A and of W per thread.
    u32x4_t ra[2], rw[2];
    auto load_tile = [&](int kt) {
        const int k0 = kt * BK;
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int idx = tid + v * 256;
            const int row = idx >> 3, c = idx & 7;
            const int k = k0 + c * (16 / EB);
            const int m = m0 + row;
            u32x4_t z = {0u, 0u, 0u, 0u};
            ra[v] = z;
            if (m < a.M && k < a.K)
                ra[v] = *reinterpret_cast<const u32x4_t*>((const unsigned char*)a.A + ((long)m * a.K + k) * EB);
            if (kEpi == EPI_TERNARY) continue;
            const int n = (row < 32) ? tc.base0 + row : tc.base1 + row - 32;
            rw[v] = z;
            if (n < a.N && k < a.K)
                rw[v] = *reinterpret_cast<const u32x4_t*>((const unsigned char*)a.W + ((long)n * a.K + k) * EB);
        }
        if (kEpi == EPI_TERNARY) {
            // 64 rows x 128 k of 2-bit codes = 64 x 8 words; two words per thread.
            const int row = tid >> 2, q = tid & 3;
            const int n = nt * BN + row;
            const int kw = k0 / 16 + q * 2;
            u32x4_t z = {0u, 0u, 0u, 0u};
            rw[0] = z;
            if (n < a.N && kw * 16 < a.K) {
                const u32x2_t w2 = *reinterpret_cast<const u32x2_t*>((const uint32_t*)a.W + (long)n * (a.K / 16) + kw);
                rw[0][0] = w2[0];
                rw[0][1] = w2[1];
            }
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int idx = tid + v * 256;
            const int row = idx >> 3, c = idx & 7;
            *reinterpret_cast<u32x4_t*>(ldsA + row * LDS_STRIDE + c * 16) = ra[v];
            if (kEpi != EPI_TERNARY) *reinterpret_cast<u32x4_t*>(ldsW + row * LDS_STRIDE + c * 16) = rw[v];
        }
        if (kEpi == EPI_TERNARY) {
            // Decode 2 words -> 32 codes (unsigned 0..3; the -2 offset is folded
            // into the epilogue as -2*rowsum).  Word layout: value b+4j sits at
            // bits 8b+2j, so (w >> 2j) & 0x03030303 is values 4j..4j+3.
            const int row = tid >> 2, q = tid & 3;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t w = rw[0][h];
                u32x4_t d;
                d[0] = w & 0x03030303u;
                d[1] = (w >> 2) & 0x03030303u;
                d[2] = (w >> 4) & 0x03030303u;
                d[3] = (w >> 6) & 0x03030303u;
                *reinterpret_cast<u32x4_t*>(ldsW + row * LDS_STRIDE + q * 32 + h * 16) = d;
            }
        }
    };

    load_tile(0);
    for (int kt = 0; kt < nkt; ++kt) {
        store_tile();
        __syncthreads();
        if (kt + 1 < nkt) load_tile(kt + 1);
#pragma unroll
        for (int ch = 0; ch < ROW_BYTES / TR::kChunkBytes; ++ch) {
            const int off = ch * TR::kChunkBytes + g * 16;
            const u32x4_t fa = *reinterpret_cast<const u32x4_t*>(ldsA + (wm * 32 + r) * LDS_STRIDE + off);
            const u32x4_t fw = *reinterpret_cast<const u32x4_t*>(ldsW + (wn * 32 + r) * LDS_STRIDE + off);
            TR::mma(acc, fa, fw);
        }
        __syncthreads();
    }

    // Accumulators -> LDS C tile (4-byte cells).
    uint32_t* C = reinterpret_cast<uint32_t*>(lds);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = wm * 32 + 8 * j + 4 * g + i;
            const int col = wn * 32 + r;
            C[row * C_STRIDE + col] = acc_bits(acc[4 * j + i]);
        }
    __syncthreads();

    // Epilogue: thread t owns row t/4 and tile columns jg..jg+7 and 32+jg..32+jg+7.
    const int erow = tid >> 2, jg = (tid & 3) * 8;
    const int m = m0 + erow;
    if (m >= a.M) return;
    const uint32_t* crow = C + erow * C_STRIDE;

    if (kEpi == EPI_TERNARY) {
        const int rs2 = 2 * a.rowsum[m];
        const float sm = a.s ? a.s[m] : 1.f;
        const int group = a.N / a.ws_num;
#pragma unroll
        for (int hlf = 0; hlf < 2; ++hlf)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int n = nt * BN + hlf * 32 + jg + e;
                if (n >= a.N) continue;
                const int v = (int)crow[hlf * 32 + jg + e] - rs2;
                if (a.acc_out) a.acc_out[(long)m * a.N + n] = v;
                if (a.Y) ((bf16_t*)a.Y)[(long)m * a.N + n] = f2bf((float)v / sm * a.ws[n / group]);
            }
        return;
    }

    float lo[8], hi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        lo[e] = __uint_as_float(crow[jg + e]);
        hi[e] = __uint_as_float(crow[32 + jg + e]);
    }

    if (kEpi == EPI_PLAIN) {
#pragma unroll
        for (int hlf = 0; hlf < 2; ++hlf)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int n = nt * BN + hlf * 32 + jg + e;
                if (n >= a.N) continue;
                float v = hlf ? hi[e] : lo[e];
                if (a.bias) v += a.bias[n];
                const long o = (long)m * a.N + n;
                if (a.out_bf16) {
                    if (a.residual) v += bf2f(((const bf16_t*)a.residual)[o]);
                    ((bf16_t*)a.Y)[o] = f2bf(v);
                } else {
                    if (a.residual) v += ((const float*)a.residual)[o];
                    ((float*)a.Y)[o] = v;
                }
            }
        return;
    }

    // QKV: bias, rotation, scatter.
    const int b = m / a.S, s = m % a.S;
    if (a.bias) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            lo[e] += a.bias[tc.base0 + jg + e];
            hi[e] += a.bias[tc.base1 + jg + e];
        }
    }
    if (tc.rope) {
        const int half = a.D >> 1;
        const int p0 = (tc.col0 % a.D) + jg;  // pair index inside the head
        const float* cr = a.cos_t + (long)s * half + p0;
        const float* sr = a.sin_t + (long)s * half + p0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float c = cr[e], sn = sr[e];
            const float x0 = lo[e], x1 = hi[e];
            lo[e] = x0 * c - x1 * sn;
            hi[e] = x1 * c + x0 * sn;
        }
    }
    const bool is_bf16 = (sizeof(T) == 2);
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
        const float* v = hlf ? hi : lo;
        const int col = (hlf ? tc.col1 : tc.col0) + jg;  // segment-local, 8 consecutive columns
        if (tc.seg == 0) {
            const long o = (long)m * (a.Hq * a.D) + col;
            if (is_bf16) {
                u32x4_t pk = {pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
                *reinterpret_cast<u32x4_t*>((bf16_t*)a.q_out + o) = pk;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) ((float*)a.q_out)[o + e] = v[e];
            }
        } else if (tc.seg == 1) {
            const int head = col / a.D, d0 = col % a.D;
            const long o = (((long)b * a.Hkv + head) * a.t_max + a.tok_offset + s) * a.D + d0;
            if (is_bf16) {
                u32x4_t pk = {pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
                *reinterpret_cast<u32x4_t*>((bf16_t*)a.k_cache + o) = pk;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) ((float*)a.k_cache)[o + e] = v[e];
            }
        } else {
            const int head = col / a.D, d0 = col % a.D;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const long o = (((long)b * a.Hkv + head) * a.D + d0 + e) * a.t_max + a.tok_offset + s;
                if (is_bf16) ((bf16_t*)a.vt_cache)[o] = f2bf(v[e]);
                else ((float*)a.vt_cache)[o] = v[e];
            }
        }
    }
}

template <typename T, int kEpi>
int launch(const GemmArgs& a, int n_tiles, vla_stream_t stream) {
    if (a.M == 0 || n_tiles == 0) return VLA_K_OK;
    dim3 grid(n_tiles, (a.M + BM - 1) / BM);
    gemm_kernel<T, kEpi><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

// Row sums for the exact-signature BitVLA entry points.
__global__ void rowsum_i8_kernel(const int8_t* __restrict__ A, int32_t* __restrict__ rowsum, int K) {
    const int8_t* r = A + (long)blockIdx.x * K;
    int s = 0;
    for (int k = threadIdx.x; k < K; k += 64) s += r[k];
    s = wave_sum_i(s);
    if (threadIdx.x == 0) rowsum[blockIdx.x] = s;
}

int32_t* g_rowsum = nullptr;
int g_rowsum_cap = 0;

}  // namespace

extern "C" {

int vla_linear(const void* x, const void* W, const float* bias, const void* residual, void* y, int dtype,
               int out_dtype, int M, int N, int K, vla_stream_t stream) {
    if (!x || !W || !y || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out_dtype != VLA_DT_F32 && out_dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    GemmArgs a = {};
    a.A = x; a.W = W; a.bias = bias; a.M = M; a.N = N; a.K = K;
    a.residual = residual; a.Y = y; a.out_bf16 = (out_dtype == VLA_DT_BF16);
    const int nt = (N + BN - 1) / BN;
    if (dtype == VLA_DT_BF16) {
        if (K % 8) return VLA_K_ERR_SHAPE;
        return launch<bf16_t, EPI_PLAIN>(a, nt, stream);
    }
    if (dtype == VLA_DT_F32) {
        if (K % 4) return VLA_K_ERR_SHAPE;
        return launch<float, EPI_PLAIN>(a, nt, stream);
    }
    return VLA_K_ERR_ARG;
}

int vla_attn_qkv_rope(const void* x, const void* W, const float* bias, int dtype, int M, int K, int S, int n_q_heads,
                      int n_kv_heads, int has_k, int has_v, int head_dim, const float* cos_tab, const float* sin_tab,
                      void* q_out, void* k_cache, void* vt_cache, int t_max, int tok_offset, vla_stream_t stream) {
    if (!x || !W || M < 0 || K <= 0 || S <= 0 || n_q_heads < 0 || n_kv_heads < 0 || head_dim <= 0) return VLA_K_ERR_ARG;
    const int nk = has_k ? n_kv_heads : 0, nv = has_v ? n_kv_heads : 0;
    if (n_q_heads > 0 && !q_out) return VLA_K_ERR_ARG;
    if ((nk > 0 && !k_cache) || (nv > 0 && !vt_cache)) return VLA_K_ERR_ARG;
    if ((cos_tab == nullptr) != (sin_tab == nullptr)) return VLA_K_ERR_ARG;
    if (M % S) return VLA_K_ERR_SHAPE;
    if (nk + nv > 0 && (tok_offset < 0 || tok_offset + S > t_max)) return VLA_K_ERR_SHAPE;
    const int D = head_dim;
    // every segment is a whole number of 64-column tiles, 8-column groups stay inside a head
    if ((n_q_heads * D) % BN || (nk * D) % BN || (nv * D) % BN || D % 8) return VLA_K_ERR_SHAPE;
    if (cos_tab && D % BN) return VLA_K_ERR_SHAPE;  // rotation pairs both halves of a head inside one tile
    GemmArgs a = {};
    a.A = x; a.W = W; a.bias = bias; a.M = M; a.K = K;
    a.N = (n_q_heads + nk + nv) * D;
    a.S = S; a.Hq = n_q_heads; a.nk = nk; a.nv = nv; a.D = D; a.Hkv = n_kv_heads;
    a.cos_t = cos_tab; a.sin_t = sin_tab; a.q_out = q_out; a.k_cache = k_cache; a.vt_cache = vt_cache;
    a.t_max = t_max; a.tok_offset = tok_offset;
    const int nt = a.N / BN;
    if (dtype == VLA_DT_BF16) {
        if (K % 8) return VLA_K_ERR_SHAPE;
        return launch<bf16_t, EPI_QKV>(a, nt, stream);
    }
    if (dtype == VLA_DT_F32) {
        if (K % 4) return VLA_K_ERR_SHAPE;
        return launch<float, EPI_QKV>(a, nt, stream);
    }
    return VLA_K_ERR_ARG;
}

int vla_ternary_gemm(const int8_t* A, const uint32_t* W_packed, uint16_t* out, int32_t* acc_out, const float* s,
                     const int32_t* rowsum, const float* ws, int ws_num, int M, int N, int K, vla_stream_t stream) {
    if (!A || !W_packed || !rowsum || (!out && !acc_out) || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out && (!s || !ws || ws_num <= 0)) return VLA_K_ERR_ARG;
    if (K % 128 || (out && N % ws_num)) return VLA_K_ERR_SHAPE;
    GemmArgs a = {};
    a.A = A; a.W = W_packed; a.M = M; a.N = N; a.K = K;
    a.Y = out; a.acc_out = acc_out; a.s = s; a.rowsum = rowsum; a.ws = ws; a.ws_num = ws_num > 0 ? ws_num : 1;
    return launch<int8_t, EPI_TERNARY>(a, (N + BN - 1) / BN, stream);
}

static int bitvla_ws_num(int N, int K) {  // the reference's per-shape table, bitnet_kernels.cu:31-116
    if (N == 3840 && K == 2560) return 3;
    if (N == 13824 && K == 2560) return 2;
    if (N == 4800 && K == 3200) return 6;
    if (N == 20480 && K == 3200) return 2;
    return 1;
}

int bitlinear_int8xint2_m(int8_t* A, int8_t* B, uint16_t* out, float* s, float* ws, int M, int N, int K,
                          vla_stream_t stream) {
    if (!A || !B || !out || !s || !ws || M < 0) return VLA_K_ERR_ARG;
    if (M == 0) return VLA_K_OK;
    if (M > g_rowsum_cap) {
        if (g_rowsum) (void)hipFree(g_rowsum);
        g_rowsum = nullptr;
        g_rowsum_cap = 0;
        const int cap = M < 4096 ? 4096 : M;
        if (hipMalloc((void**)&g_rowsum, (size_t)cap * sizeof(int32_t)) != hipSuccess) return VLA_K_ERR_LAUNCH;
        g_rowsum_cap = cap;
    }
    rowsum_i8_kernel<<<M, 64, 0, (hipStream_t)stream>>>(A, g_rowsum, K);
    return vla_ternary_gemm(A, (const uint32_t*)B, out, nullptr, s, g_rowsum, ws, bitvla_ws_num(N, K), M, N, K, stream);
}

int bitlinear_int8xint2(int8_t* A, int8_t* B, uint16_t* out, float* s, float* ws, int M, int N, int K,
                        vla_stream_t stream) {
    return bitlinear_int8xint2_m(A, B, out, s, ws, M, N, K, stream);
}

int vla_ternary_quant_host(const float* W, int64_t n, int8_t* ternary, float* absmean) {
    if (!W || !ternary || !absmean || n < 0) return VLA_K_ERR_ARG;
    double sum = 0.0;
    for (int64_t i = 0; i < n; ++i) sum += fabs((double)W[i]);
    float mean = n > 0 ? (float)(sum / (double)n) : 0.0f;
    if (mean < 1e-5f) mean = 1e-5f;
    *absmean = mean;
    const float inv = 1.0f / mean;
    for (int64_t i = 0; i < n; ++i) {
        float q = nearbyintf(W[i] * inv);
        q = q > 1.0f ? 1.0f : (q < -1.0f ? -1.0f : q);
        ternary[i] = (int8_t)q;
    }
    return VLA_K_OK;
}

int vla_ternary_pack_host(const int8_t* ternary, int N, int K, uint32_t* packed) {
    if (!ternary || !packed || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (K % 16) return VLA_K_ERR_SHAPE;
    const int kw = K / 16;
    for (long n = 0; n < N; ++n)
        for (int w = 0; w < kw; ++w) {
            uint32_t word = 0;
            for (int v = 0; v < 16; ++v) {
                const int t = ternary[n * K + w * 16 + v];
                if (t < -2 || t > 1) return VLA_K_ERR_ARG;
                word |= (uint32_t)((t + 2) & 3) << (8 * (v & 3) + 2 * (v >> 2));
            }
            packed[n * kw + w] = word;
        }
    return VLA_K_OK;
}

// A ladder slot is the same 16-value word; only the word order differs
// (src/models/bitvla.cpp:453-483): inside each 16-row block the words run
// (k_0: 128 k) (major_k: 32 k) (y_half: 8 rows) (sub_k: 16 k) (row in half).
int vla_ternary_repack_ladder_host(const uint8_t* ladder, int N, int K, uint32_t* packed) {
    if (!ladder || !packed || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (N % 16 || K % 128) return VLA_K_ERR_SHAPE;
    const uint32_t* src = (const uint32_t*)ladder;
    const int kw = K / 16;
    for (long n = 0; n < N; ++n)
        for (int w = 0; w < kw; ++w) {
            const long n_block = n / 16;
            const int y = (int)(n % 16), y_half = y / 8, y_in_h = y % 8;
            const int k_0 = w / 8, tx = w % 8, major_k = tx / 2, sub_k = tx % 2;
            const long slot = n_block * K + (long)k_0 * 128 + major_k * 32 + y_half * 16 + sub_k * 8 + y_in_h;
            packed[n * kw + w] = src[slot];
        }
    return VLA_K_OK;
}

}  // extern "C"
