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

#include <stdlib.h>
#include <string.h>
#include <type_traits>

#include "common.h"
#include "vla_kernels.h"

namespace {

using namespace vk;

constexpr int BN = 64;                     // epilogue sub-tile; column-tile unit of the N mapping
constexpr int C_STRIDE = BN + 4;           // floats

enum { EPI_PLAIN = 0, EPI_QKV = 1, EPI_TERNARY = 2, EPI_GLU = 3 };
enum { NORM_NONE = 0, NORM_RMS = 1, NORM_LAYER = 2, NORM_LAYER_PRE = 3 };  // row statistics taken inside gemm_dl_kernel (PRE: LayerNorm from sums handed over by the producing launch)
constexpr int STAT_MAX_TILES = 24;  // 64-column tiles of a row whose sums a consumer adds up (four threads per row, six pairs each)

struct GemmArgs {
    // Field order: what the single-token decode projections read (a chain of short launches, each waiting for its
    // arguments' cache lines before anything else) sits in the first two 64-byte lines of the block, the rotation
    // tables in the third; the tiled kernels' walk constants and epilogue extras follow.
    const void* A;
    const void* W;
    const float* bias;
    int M, N, K, n_tiles;
    // TERNARY (part): weight scales; row statistics of A taken inside the launch (see norm_eps below)
    int ws_num;
    // Row statistics of A taken inside the GEMM (direct-to-LDS kernel, kNorm): RMS when
    // colsum is null, else LayerNorm with colsum[n] = sum_k W[n][k] (fp32 [N])
    float norm_eps;
    const float* ws;
    const void* norm_w;  // ternary GEMV with the RMSNorm and quantisation of its rows inside: A is bf16, this the norm weight
    // PLAIN, GLU
    const void* residual;
    void* Y;
    int out_bf16;
    int act;  // VLA_ACT_*: PLAIN applies it after the bias, GLU to the gate
    // QKV
    void* q_out;
    void* k_cache;
    void* vt_cache;
    int t_max, tok_offset, Hkv, D;
    const float* cos_t;
    const float* sin_t;
    int S, Hq, nk, nv;
    int xm, xn;
    int pn;  // N tiles per panel of an XCD's walk (see xcd_tile)
    const float* col_gate;  // PLAIN: fp32 [N] factor on the projection before the residual is added, or null
    // TERNARY
    int32_t* acc_out;
    const float* s;
    const int32_t* rowsum;
    const float* colsum;
    // Row statistics handed from the launch that writes a row to the launch that normalises it: a PLAIN
    // launch with bf16 output leaves (sum of squares, sum) of the 64 values it wrote per (row, 64-column
    // tile) in stats_out [M][N / 64][2]; a QKV launch with the LayerNorm inside adds up the n_stat pairs
    // of a row from stats_in instead of summing the row from its operand tiles.
    float* stats_out;
    const float* stats_in;
    int n_stat;
    // The tile walk's constants (see xcd_tile), formed once on the host (xcd_split) so that a workgroup finds its tile
    // with a few multiplications: every division by a run-time value costs a wavefront some thirty dependent scalar
    // instructions in front of its first load.  cn, cm: tiles per XCD column / row; per_panel = pn cm; full = cn / pn
    // whole panels; w_last = cn - full pn; mg_*: 2^32 / d + 1 for d = cn, per_panel, pn, w_last (x / d = mulhi(x, mg)
    // for x < 2^16); xn_shift = log2 xn.
    int cn, cm, per_panel, full, w_last, xn_shift;
    unsigned mg_cn, mg_pp, mg_pn, mg_wl;
};

// Workgroup -> tile.  Workgroup i runs on XCD i % 8; the XCDs form an xm x xn grid over the
// tile grid and XCD (xr, xc) owns the tiles (m, n) with m % xm == xr, n % xn == xc.  Its
// workgroups walk them panel by panel: pn of its N tiles at a time, every M tile of the XCD
// against that panel before the next panel starts, so that the panel's rows of W stay in the
// XCD's L2 while the rows of A stream past them once per panel.  (With all of W in one
// panel and W larger than the L2, W would stream again for every few M tiles instead.)
__device__ __forceinline__ unsigned div_magic(unsigned x, unsigned d, unsigned mg) { return d == 1 ? x : __umulhi(x, mg); }
__device__ __forceinline__ bool xcd_tile(const GemmArgs& a, int n_wg_tiles, int m_wg_tiles, int& mtw, int& ntw) {
    const unsigned xcd = blockIdx.x & 7, local = blockIdx.x >> 3;  // local < 2^16 (checked where the grid is sized)
    unsigned ml, nl;
    if (a.pn >= a.cn) {
        ml = div_magic(local, a.cn, a.mg_cn);
        nl = local - ml * a.cn;
    } else {
        unsigned p = div_magic(local, a.per_panel, a.mg_pp), rem = local - p * a.per_panel, w = a.pn, mg = a.mg_pn;
        if (p >= (unsigned)a.full) {  // the last, narrower panel
            p = a.full;
            rem = local - a.full * a.per_panel;
            w = a.w_last;
            mg = a.mg_wl;
        }
        ml = div_magic(rem, w, mg);
        nl = p * a.pn + rem - ml * w;
    }
    ntw = (int)(nl * a.xn + (xcd & (a.xn - 1)));
    mtw = (int)(ml * a.xm + (xcd >> a.xn_shift));
    return ntw < n_wg_tiles && mtw < m_wg_tiles;
}

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

// Packed ternary weights are stored "MFMA-fragment-major": for each block of 32 output
// columns and each group of 32 k, 64 consecutive words [g][r] hold the 16 codes
// k = 32*kk + 16*g .. +15 of column 32*nb + r -- exactly what lane (g, r) of a wavefront
// feeds to v_mfma_i32_32x32x32_i8, so a fragment is one coalesced 256-byte load.
__host__ __device__ __forceinline__ long tern_word_index(long n, int w, int K) {
    return (((n >> 5) * (K / 32) + (w >> 1)) * 2 + (w & 1)) * 32 + (n & 31);
}

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
    if (kEpi == EPI_GLU) {  // W = [gate rows; up rows]: the tile pairs 32 gate columns with their up columns
        t.base0 = nt * 32;
        t.base1 = a.N / 2 + nt * 32;
        t.seg = 0;
        t.col0 = t.base0;
        t.col1 = t.base1;
        t.rope = false;
        return t;
    }
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

// acc + lo^2 + hi^2 of the two bf16 values packed in u (taken by value: a bit_cast applied
// directly to a vector element expression reads element 0).
__device__ __forceinline__ float add_squares_bf16x2(uint32_t u, float acc) {
    const bf16x2_t v = __builtin_bit_cast(bf16x2_t, u);
    return __builtin_amdgcn_fdot2_f32_bf16(v, v, acc, false);
}
// acc + lo + hi
__device__ __forceinline__ float add_pair_bf16x2(uint32_t u, float acc) {
    const bf16x2_t v = __builtin_bit_cast(bf16x2_t, u);
    const bf16x2_t ones = __builtin_bit_cast(bf16x2_t, 0x3f803f80u);
    return __builtin_amdgcn_fdot2_f32_bf16(v, ones, acc, false);
}

// Epilogue of one 64x64 sub-tile held in the LDS C tile: thread t owns row t/4 and
// columns jg..jg+7 and 32+jg..32+jg+7 of the sub-tile.
__device__ const float kNoBiasRegs[16] = {};
template <typename T, int kEpi, bool BIAS_REGS = false>
__device__ __forceinline__ void epilogue_64x64(const GemmArgs& a, const uint32_t* C, int m0, int nt, const TileCols& tc,
                                               int tid, bool have_res = false, u32x4_t res_lo = u32x4_t{0u, 0u, 0u, 0u},
                                               u32x4_t res_hi = u32x4_t{0u, 0u, 0u, 0u}, int norm_mode = 0,
                                               const float* row_stat = nullptr, int stat_stride = 0,
                                               const float (&bias_regs)[16] = kNoBiasRegs) {
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
                if (a.Y) {
                    bf16_t o = f2bf((float)v / sm * a.ws[n / group]);
                    if (a.residual) o = f2bf(bf2f(o) + bf2f(((const bf16_t*)a.residual)[(long)m * a.N + n]));
                    ((bf16_t*)a.Y)[(long)m * a.N + n] = o;
                }
            }
        return;
    }

    float lo[8], hi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        lo[e] = __uint_as_float(crow[jg + e]);
        hi[e] = __uint_as_float(crow[32 + jg + e]);
    }
    if (norm_mode) {
        // row_stat: per row of the sub-tile (sum of squares, sum) of the A row, as two partial
        // pairs stat_stride floats apart (one from each of the two wavefronts sharing the row)
        const float inv_k = 1.0f / (float)a.K;
        const float sq = row_stat[2 * erow] + row_stat[stat_stride + 2 * erow];
        if (norm_mode == NORM_LAYER && kEpi == EPI_QKV) {
            // sum_k (x - mean) rstd W[n][k] = rstd acc - (mean rstd) colsum[n]
            const float mean = (row_stat[2 * erow + 1] + row_stat[stat_stride + 2 * erow + 1]) * inv_k;
            const float f = rsqrtf(fmaxf(sq * inv_k - mean * mean, 0.f) + a.norm_eps);
            const float ms = mean * f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                lo[e] = lo[e] * f - ms * a.colsum[tc.base0 + jg + e];
                hi[e] = hi[e] * f - ms * a.colsum[tc.base1 + jg + e];
            }
        } else {
            const float f = rsqrtf(sq * inv_k + a.norm_eps);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                lo[e] *= f;
                hi[e] *= f;
            }
        }
    }

    if (kEpi == EPI_GLU) {
        // lo = gate columns nt*32 + jg .. +7, hi = the up columns of the same outputs
        const int I = a.N / 2, n0 = nt * 32 + jg;  // I is a multiple of 32: the 8 outputs are inside the row
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float gt = lo[e], up = hi[e];
            if (a.bias) {
                gt += a.bias[n0 + e];
                up += a.bias[I + n0 + e];
            }
            v[e] = apply_act(gt, a.act) * up;
        }
        const long o = (long)m * I + n0;
        if (a.out_bf16) {
            const u32x4_t pk = {pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
            *reinterpret_cast<u32x4_t*>((bf16_t*)a.Y + o) = pk;
        } else {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const f32x4_t pk = {v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
                *reinterpret_cast<f32x4_t*>((float*)a.Y + o + 4 * q) = pk;
            }
        }
        return;
    }

    if (kEpi == EPI_PLAIN) {
        float st1 = 0.f, st2 = 0.f;  // sum and sum of squares of the 16 values this thread writes (as written: rounded to bf16)
#pragma unroll
        for (int hlf = 0; hlf < 2; ++hlf) {
            const int n0 = nt * BN + hlf * 32 + jg;
            if (n0 >= a.N) continue;
            float* v = hlf ? hi : lo;
            const long o = (long)m * a.N + n0;
            const bool full = (n0 + 8 <= a.N) && (a.N % 8 == 0);
            // per-column operands: indices clamped into the row instead of a branch per element
            // (columns past N are never stored), so the eight loads are in flight together
            if (a.bias) {
                // BIAS_REGS: this thread's 2 x 8 values, fetched by the caller ahead of the epilogue
                float bv[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) bv[e] = BIAS_REGS ? bias_regs[hlf * 8 + e] : a.bias[min(n0 + e, a.N - 1)];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += bv[e];
            }
            if (a.act != VLA_ACT_NONE) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = apply_act(v[e], a.act);
            }
            if (a.col_gate) {
                float gv[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) gv[e] = a.col_gate[min(n0 + e, a.N - 1)];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] *= gv[e];
            }
            if (full && a.out_bf16) {  // 8 consecutive bf16 = one 16-byte access each way
                if (a.residual) {
                    // res_lo / res_hi: this thread's two residual vectors when fetched before the k loop
                    u32x4_t rr = hlf ? res_hi : res_lo;
                    if (!have_res) rr = *reinterpret_cast<const u32x4_t*>((const bf16_t*)a.residual + o);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[2 * e] += __uint_as_float(rr[e] << 16);
                        v[2 * e + 1] += __uint_as_float(rr[e] & 0xffff0000u);
                    }
                }
                const u32x4_t pk = {pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
                *reinterpret_cast<u32x4_t*>((bf16_t*)a.Y + o) = pk;
                if (a.stats_out) {  // two bf16 values per instruction, exact products, fp32 sums
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        st1 = add_pair_bf16x2(pk[e], st1);
                        st2 = add_squares_bf16x2(pk[e], st2);
                    }
                }
            } else if (full) {
                if (a.residual) {
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const f32x4_t rr = *reinterpret_cast<const f32x4_t*>((const float*)a.residual + o + 4 * q);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[4 * q + e] += rr[e];
                    }
                }
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const f32x4_t pk = {v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
                    *reinterpret_cast<f32x4_t*>((float*)a.Y + o + 4 * q) = pk;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (n0 + e >= a.N) continue;
                    float x = v[e];
                    if (a.out_bf16) {
                        if (a.residual) x += bf2f(((const bf16_t*)a.residual)[o + e]);
                        ((bf16_t*)a.Y)[o + e] = f2bf(x);
                    } else {
                        if (a.residual) x += ((const float*)a.residual)[o + e];
                        ((float*)a.Y)[o + e] = x;
                    }
                }
            }
        }
        if (a.stats_out) {
            // the four threads of a row (tid % 4) are neighbouring lanes: the row's 64 values of this tile
            st1 += __uint_as_float(dpp_u32<DPP_XOR1>(__float_as_uint(st1)));
            st2 += __uint_as_float(dpp_u32<DPP_XOR1>(__float_as_uint(st2)));
            st1 += __uint_as_float(dpp_u32<DPP_XOR2>(__float_as_uint(st1)));
            st2 += __uint_as_float(dpp_u32<DPP_XOR2>(__float_as_uint(st2)));
            if ((tid & 3) == 0) *reinterpret_cast<f32x2_t*>(a.stats_out + ((long)m * (a.N / BN) + nt) * 2) = f32x2_t{st2, st1};
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

// Workgroup tile (64*TM) x (64*TN), 2 x 2 wavefronts; wavefront (wm, wn) owns the 32x32
// MFMA blocks in block rows wm + 2i (i < TM) and block columns wn + 2j (j < TN), so every
// 64x64 sub-tile is made of one block from each wavefront.  KB = bytes of K per staged row.
template <typename T, int kEpi, int TM, int TN, int KB, int DEPTH>
__global__ void __launch_bounds__(256) gemm_kernel(GemmArgs a) {
    typedef Traits<T> TR;
    constexpr int EB = TR::kElemBytes;
    constexpr int BK = KB / EB;        // k elements per tile
    constexpr int EPV = 16 / EB;       // elements per 16-byte vector
    constexpr int STRIDE = KB + 16;    // padded LDS row
    constexpr int ROWS_A = 64 * TM, ROWS_W = 64 * TN;
    constexpr int VPR = KB / 16;       // 16-byte vectors per staged row
    constexpr int VA = ROWS_A * VPR / 256, VW = ROWS_W * VPR / 256;  // vectors per thread
    static_assert(kEpi != EPI_TERNARY || (TM == 1 && TN == 1 && KB == 128), "ternary staging assumes 64x64x128 tiles");

    // two operand buffers: tile kt is multiplied out of buffer kt & 1 while tile kt + 1 is
    // being stored into the other one, so a k-tile costs one barrier
    constexpr int BUF = (ROWS_A + ROWS_W) * STRIDE;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * BUF];
    static_assert(sizeof(float) * 64 * C_STRIDE <= sizeof(lds), "C sub-tile must fit in the operand buffers");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int g = lane >> 5, r = lane & 31;
    // Linear workgroup id -> (M tile, N tile).  id % 8 is the XCD a workgroup is dispatched
    // to; the 8 XCDs form an xm x xn grid and XCD (i, j) owns the M tiles = i (mod xm) and
    // the N tiles = j (mod xn), so each L2 fetches 1/xm of A and 1/xn of W instead of the
    // whole of either (the host picks the split that minimises the total).
    const int n_wg_tiles = (a.n_tiles + TN - 1) / TN, m_wg_tiles = (a.M + ROWS_A - 1) / ROWS_A;
    int mtw, ntw;
    if (!xcd_tile(a, n_wg_tiles, m_wg_tiles, mtw, ntw)) return;
    const int m0 = mtw * ROWS_A;
    TileCols tc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) tc[j] = tile_cols<kEpi>(a, ntw * TN + j);

    typename TR::Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int nkt = (a.K + BK - 1) / BK;

    // Operand staging: global -> registers -> LDS, with DEPTH k-tiles of loads in flight
    // (a ring of register stages with compile-time indices).  The loads are unconditional:
    // rows past M or N and k past K are redirected to valid addresses (their products land
    // in outputs that are dropped, or are zeroed when the one partial k-tile is stored), and
    // the ring keeps re-reading the last tile once the real ones are exhausted, so the loop
    // body has no load under a branch and the wait counts stay exact.
    const unsigned char* ap[VA];
    int a_koff[VA];
#pragma unroll
    for (int v = 0; v < VA; ++v) {
        const int idx = tid + v * 256;
        const int m = min(m0 + idx / VPR, a.M - 1);
        a_koff[v] = (idx % VPR) * EPV;
        ap[v] = (const unsigned char*)a.A + (long)m * a.K * EB;
    }
    const unsigned char* wp[VW];
    if (kEpi != EPI_TERNARY) {
#pragma unroll
        for (int v = 0; v < VW; ++v) {
            const int idx = tid + v * 256;
            constexpr int RPV = 256 / VPR;                     // rows covered by one vector index step
            const int sub = (v * RPV) / 64, wr = (idx / VPR) & 63;  // sub is compile-time per unrolled v
            int n = (wr < 32) ? tc[sub].base0 + wr : tc[sub].base1 + wr - 32;
            n = min(max(n, 0), a.N - 1);
            wp[v] = (const unsigned char*)a.W + (long)n * a.K * EB;
        }
    } else {
        // 64 rows x 128 k of 2-bit codes = 64 x 8 words; two words per thread: the two
        // 16-k halves (g = 0, 1) of 32-k group q of the tile.
        const int n = min(ntw * BN + (tid >> 2), a.N - 1);
        wp[0] = (const unsigned char*)((const uint32_t*)a.W + tern_word_index(n, (tid & 3) * 2, a.K));
    }
    u32x4_t ra[DEPTH][VA], rw[DEPTH][VW];
    // Load vector i of tile kt into ring stage st; i runs over the VA vectors of A and then
    // the VW vectors of W (the ternary staging has a single W entry of two words).
    constexpr int NLOAD = VA + ((kEpi != EPI_TERNARY) ? VW : 1);
    auto load_vec = [&](int st, int kt, int i) __attribute__((always_inline)) {
        const int k0 = kt * BK;
        if (i < VA) {
            const int k = min(k0 + a_koff[i], a.K - EPV);
            ra[st][i] = *reinterpret_cast<const u32x4_t*>(ap[i] + (long)k * EB);
        } else if (kEpi != EPI_TERNARY) {
            const int v = i - VA;
            const int k = min(k0 + a_koff[v % VA], a.K - EPV);  // same column pattern as A (VPR | 256)
            rw[st][v] = *reinterpret_cast<const u32x4_t*>(wp[v] + (long)k * EB);
        } else {
            const uint32_t* w = (const uint32_t*)wp[0] + (long)(k0 / 32) * 64;
            rw[st][0][0] = w[0];
            rw[st][0][1] = w[32];
        }
    };
    auto load_tile = [&](int st, int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) load_vec(st, kt, i);
    };
    auto mask_partial = [&](int st, int kt) __attribute__((always_inline)) {  // zero what lies past K
#pragma unroll
        for (int v = 0; v < VA; ++v)
            if (kt * BK + a_koff[v] >= a.K) {
                const u32x4_t z = {0u, 0u, 0u, 0u};
                ra[st][v] = z;
            }
        if (kEpi != EPI_TERNARY) {
#pragma unroll
            for (int v = 0; v < VW; ++v)
                if (kt * BK + a_koff[v % VA] >= a.K) {
                    const u32x4_t z = {0u, 0u, 0u, 0u};
                    rw[st][v] = z;
                }
        }
    };
    auto store_tile = [&](int st, int buf) __attribute__((always_inline)) {
        unsigned char* ldsA = lds + buf * BUF;
        unsigned char* ldsW = ldsA + ROWS_A * STRIDE;
#pragma unroll
        for (int v = 0; v < VA; ++v) {
            const int idx = tid + v * 256;
            *reinterpret_cast<u32x4_t*>(ldsA + (idx / VPR) * STRIDE + (idx % VPR) * 16) = ra[st][v];
        }
        if (kEpi != EPI_TERNARY) {
#pragma unroll
            for (int v = 0; v < VW; ++v) {
                const int idx = tid + v * 256;
                *reinterpret_cast<u32x4_t*>(ldsW + (idx / VPR) * STRIDE + (idx % VPR) * 16) = rw[st][v];
            }
        } else {
            // Decode 2 words -> 32 codes (unsigned 0..3; the -2 offset is folded
            // into the epilogue as -2*rowsum).  Word layout: value b+4j sits at
            // bits 8b+2j, so (w >> 2j) & 0x03030303 is values 4j..4j+3.
            const int row = tid >> 2, q = tid & 3;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t w = rw[st][0][h];
                u32x4_t d;
                d[0] = w & 0x03030303u;
                d[1] = (w >> 2) & 0x03030303u;
                d[2] = (w >> 4) & 0x03030303u;
                d[3] = (w >> 6) & 0x03030303u;
                *reinterpret_cast<u32x4_t*>(ldsW + row * STRIDE + q * 32 + h * 16) = d;
            }
        }
    };
    // Multiplies the tile in LDS buffer buf.  With LOAD set, the loads of tile kt_load into
    // ring stage st_load are issued a few per k-chunk between the MFMA groups instead of in
    // one burst: a burst keeps every wavefront of the workgroup waiting at the texture
    // unit's queue before any of them starts on the LDS reads, so load issue and multiply
    // would run one after the other instead of side by side.
    auto multiply = [&](int buf, auto do_load, int st_load, int kt_load) __attribute__((always_inline)) {
        constexpr bool LOAD = decltype(do_load)::value;
        constexpr int NCH = KB / TR::kChunkBytes;
        const unsigned char* ldsA = lds + buf * BUF;
        const unsigned char* ldsW = ldsA + ROWS_A * STRIDE;
        // operand fragments are read one k-chunk ahead of the MFMAs that use them, so the
        // LDS latency of chunk ch + 1 passes under the MFMAs of chunk ch
        u32x4_t fa[2][TM], fw[2][TN];
        auto read_frags = [&](int slot, int ch) __attribute__((always_inline)) {
            const int off = ch * TR::kChunkBytes + g * 16;
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[slot][i] = *reinterpret_cast<const u32x4_t*>(ldsA + ((wm + 2 * i) * 32 + r) * STRIDE + off);
#pragma unroll
            for (int j = 0; j < TN; ++j) fw[slot][j] = *reinterpret_cast<const u32x4_t*>(ldsW + ((wn + 2 * j) * 32 + r) * STRIDE + off);
        };
        read_frags(0, 0);
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            if (ch + 1 < NCH) read_frags((ch + 1) & 1, ch + 1);
            if (LOAD) {
#pragma unroll
                for (int i = ch * NLOAD / NCH; i < (ch + 1) * NLOAD / NCH; ++i) load_vec(st_load, kt_load, i);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) TR::mma(acc[i][j], fa[ch & 1][i], fw[ch & 1][j]);
            __builtin_amdgcn_sched_barrier(0);  // keeps the reads and loads where they were placed
        }
    };

    // Stage st of the ring holds tile kt with kt % DEPTH == st.  Main loop: whole groups
    // of DEPTH full tiles, no branch around a load.  The remaining tiles (fewer than DEPTH
    // full ones and at most one partial) are already in flight when the main loop ends
    // and are drained without further loads.  The LDS store of tile kt + 1 follows the
    // multiply of tile kt in program order, so it runs under the MFMAs still in flight.
#pragma unroll
    for (int st = 0; st < DEPTH; ++st) load_tile(st, min(st, nkt - 1));
    if (BK > a.K) mask_partial(0, 0);
    store_tile(0, 0);
    __syncthreads();
    const int n_main = (a.K / BK) / DEPTH;
    for (int gi = 0; gi < n_main; ++gi) {
#pragma unroll
        for (int st = 0; st < DEPTH; ++st) {
            const int kt = gi * DEPTH + st;
            // stage st held tile kt, already in LDS: refill it with tile kt + DEPTH
            multiply(kt & 1, std::true_type{}, st, min(kt + DEPTH, nkt - 1));
            if ((kt + 2) * BK > a.K) mask_partial((st + 1) % DEPTH, kt + 1);  // uniform; only the last tile can be partial
            store_tile((st + 1) % DEPTH, (kt + 1) & 1);  // past the last tile: a repeat of it, never read
            __syncthreads();
        }
    }
#pragma unroll
    for (int st = 0; st < DEPTH; ++st) {
        const int kt = n_main * DEPTH + st;
        if (kt < nkt) {  // uniform
            multiply(kt & 1, std::false_type{}, 0, 0);
            if (kt + 1 < nkt) {
                if ((kt + 2) * BK > a.K) mask_partial((st + 1) % DEPTH, kt + 1);
                store_tile((st + 1) % DEPTH, (kt + 1) & 1);
            }
            __syncthreads();
        }
    }

    // Epilogue, one 64x64 sub-tile at a time through an LDS copy of the accumulators.
    uint32_t* C = reinterpret_cast<uint32_t*>(lds);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if (i + j > 0) __syncthreads();
#pragma unroll
            for (int jj = 0; jj < 4; ++jj)
#pragma unroll
                for (int ii = 0; ii < 4; ++ii)
                    C[(wm * 32 + 8 * jj + 4 * g + ii) * C_STRIDE + wn * 32 + r] = acc_bits(acc[i][j][4 * jj + ii]);
            __syncthreads();
            const int nt_sub = ntw * TN + j;
            if (nt_sub < a.n_tiles) epilogue_64x64<T, kEpi>(a, C, m0 + i * 64, nt_sub, tc[j], tid);
        }
}

// ---- bf16 GEMM with operand tiles loaded straight into LDS --------------------------
// Same tiling, wavefront layout, XCD mapping and epilogues as gemm_kernel, for bf16
// operands with K a multiple of 16.  A stage of the LDS ring holds one k-tile of A and W
// rows, KB bytes per row and no padding: a load instruction of a wavefront fills 1 KiB of
// consecutive LDS (1024 / KB rows).  Bank conflicts of the fragment reads are avoided by a
// swizzle instead of padding: the 16-byte piece c of row `row` is kept at piece position
// c ^ swz(row), swz = (row >> 1) & 7 for 128-byte rows and row & 15 for 256-byte rows (16
// consecutive fragment rows then cover all 64 banks exactly once); the loading lane picks
// the global piece that belongs in its LDS slot.  NS - 1 tiles of loads are in flight; a
// k-tile costs one barrier, and no wavefront spends issue slots on LDS stores.
template <int kEpi, int TM, int TN, int KB, int NS, int kNorm>
__global__ void __launch_bounds__(256) gemm_dl_kernel(GemmArgs a) {
    typedef bf16_t T;
    typedef Traits<bf16_t> TR;
    constexpr int EB = 2, BK = KB / EB, EPV = 8;
    constexpr int ROWS_A = 64 * TM, ROWS_W = 64 * TN;
    constexpr int VPR = KB / 16;        // 16-byte pieces per row
    constexpr int RPS = 256 / VPR;      // rows filled by one load per thread of the workgroup
    constexpr int VA = ROWS_A / RPS, VW = ROWS_W / RPS, NLOAD = VA + VW;
    constexpr int NCH = KB / 32;        // 16-k MFMA chunks per tile
    constexpr int STAGE = (ROWS_A + ROWS_W) * KB;
    constexpr int C_BYTES = 4 * 64 * C_STRIDE;
    constexpr int EPI_BYTES = 2 * C_BYTES + ROWS_A * 16;  // two C sub-tiles, then two (sum of squares, sum) pairs per tile row (kNorm)
    constexpr int LDS_BYTES = NS * STAGE > EPI_BYTES ? NS * STAGE : EPI_BYTES;
    constexpr int IN_FLIGHT = (NS - 2) * NLOAD;  // loads younger than the tile about to be multiplied
    static_assert(KB == 128 || KB == 256, "swizzle is defined for 128- and 256-byte rows");
    static_assert(NS >= 2 && IN_FLIGHT <= 63, "ring depth exceeds the vector-memory counter");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int g = lane >> 5, r = lane & 31;
    const int n_wg_tiles = (a.n_tiles + TN - 1) / TN, m_wg_tiles = (a.M + ROWS_A - 1) / ROWS_A;
    int mtw, ntw;
    if (!xcd_tile(a, n_wg_tiles, m_wg_tiles, mtw, ntw)) return;
    const int m0 = mtw * ROWS_A;
    TileCols tc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) tc[j] = tile_cols<kEpi>(a, ntw * TN + j);

    typename TR::Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int nkt = (a.K + BK - 1) / BK, nkt_full = a.K / BK;
    // kNorm: the GEMM multiplies raw rows of A and scales row m of the result by
    // rsqrt(mean_k A[m][k]^2 + eps); the squares are summed from the same LDS fragments
    // the MFMAs read (lane (g, r) sees 8 of every 16 k of its rows; the two halves meet
    // after the loop), two bf16 products per instruction.  NORM_LAYER also sums the values:
    // row m of the result becomes rstd (acc - mean colsum[n]), the projection of the
    // centred and scaled row.  The two wavefronts that read the same A rows (wn = 0, 1)
    // take alternate k-chunks, and each of a fragment's four words has its own
    // accumulator, so a chunk adds one dependent operation per accumulator.
    float ssq[TM][4], ssum[TM][4];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) ssq[i][e] = ssum[i][e] = 0.f;

    // A bf16 residual is fetched now, ahead of every operand load, instead of in the
    // epilogue where nothing is left to hide its latency (the epilogue thread layout:
    // row tid / 4, columns 8 (tid % 4) .. +7 of each 32-column half of a 64x64 sub-tile).
    u32x4_t res_pf[TM][TN][2] = {};
    const bool pf = kEpi == EPI_PLAIN && a.residual != nullptr && a.out_bf16 && a.N % 8 == 0;
    if (pf) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int hlf = 0; hlf < 2; ++hlf) {
                    const int m = min(m0 + i * 64 + (tid >> 2), a.M - 1);
                    const int n0 = min((ntw * TN + j) * BN + hlf * 32 + (tid & 3) * 8, a.N - 8);
                    res_pf[i][j][hlf] = *reinterpret_cast<const u32x4_t*>((const bf16_t*)a.residual + (long)m * a.N + n0);
                }
    }

    // NORM_LAYER_PRE: the row sums handed over by the producing launch, six (sum of squares, sum) pairs per thread
    // and tile row (the four threads of a row take the tiles t % 4), requested ahead of the operand loads as well.
    f32x2_t st_pf[TM][STAT_MAX_TILES / 4] = {};
    if (kNorm == NORM_LAYER_PRE) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const float* sp = a.stats_in + (long)min(m0 + i * 64 + (tid >> 2), a.M - 1) * a.n_stat * 2;
#pragma unroll
            for (int t = 0; t < STAT_MAX_TILES / 4; ++t) st_pf[i][t] = *reinterpret_cast<const f32x2_t*>(sp + min((tid & 3) + 4 * t, a.n_stat - 1) * 2);
        }
    }

    // Loader side.  Thread tid fills LDS slot tid of each 256-slot slab; slab v of A holds
    // rows v*RPS .. v*RPS+RPS-1.  The slot is piece position tid % VPR of row tid / VPR, so
    // the lane fetches the logical piece (tid % VPR) ^ swz(row); swz only involves the low
    // row bits, which do not depend on the slab.  Rows past M or N and k past K are
    // redirected to valid addresses: their products land in outputs that are dropped, and
    // k-chunks past K are never multiplied.
    const int lrow = tid / VPR;
    const int lsw = (KB == 128) ? ((lrow >> 1) & 7) : (lrow & 15);
    const int koff = ((tid % VPR) ^ lsw) * EPV;
    const unsigned char* ap[VA];
#pragma unroll
    for (int v = 0; v < VA; ++v) ap[v] = (const unsigned char*)a.A + (long)min(m0 + v * RPS + lrow, a.M - 1) * a.K * EB;
    const unsigned char* wp[VW];
#pragma unroll
    for (int v = 0; v < VW; ++v) {
        const int sub = (v * RPS) / 64, wr = (v * RPS + lrow) & 63;  // sub is compile-time per unrolled v
        int n = (wr < 32) ? tc[sub].base0 + wr : tc[sub].base1 + wr - 32;
        n = min(max(n, 0), a.N - 1);
        wp[v] = (const unsigned char*)a.W + (long)n * a.K * EB;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds + wave * 1024;  // low 32 bits of a shared-aperture address = LDS offset
    auto issue = [&](int i, int kt, int stage) __attribute__((always_inline)) {
        const long kb = (long)min(kt * BK + koff, a.K - EPV) * EB;
        if (i < VA) load_to_lds16(ap[i] + kb, lds0 + stage * STAGE + i * 4096);
        else load_to_lds16(wp[i - VA] + kb, lds0 + stage * STAGE + ROWS_A * KB + (i - VA) * 4096);
    };

    // Consumer side.  Fragment row r of any 32-row block has swz = (r >> 1) & 7 (or r & 15);
    // the lane wants logical piece 2 ch + g, i.e. position (2 ch) ^ (g ^ swz).
    const int fsw = (KB == 128) ? ((r >> 1) & 7) : (r & 15);
    const int xo = (g ^ fsw) * 16;
    const int fragA = (wm * 32 + r) * KB, fragW = ROWS_A * KB + (wn * 32 + r) * KB;
    auto multiply = [&](int stage, auto do_load, int st_load, int kt_load, int n_chunks) __attribute__((always_inline)) {
        constexpr bool LOAD = decltype(do_load)::value;
        // fragments are read PF k-chunks ahead of the MFMAs that use them: one chunk of MFMAs
        // is shorter than the LDS latency, so a single chunk of lookahead leaves every chunk
        // waiting on its reads
        constexpr int PF = NCH >= 4 ? 2 : 1, SLOTS = PF + 1;
        const unsigned char* base = lds + stage * STAGE;
        u32x4_t fa[SLOTS][TM], fw[SLOTS][TN];
        auto read_frags = [&](int slot, int ch) __attribute__((always_inline)) {
            const int off = (ch * 32) ^ xo;
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[slot][i] = *reinterpret_cast<const u32x4_t*>(base + fragA + i * 64 * KB + off);
#pragma unroll
            for (int j = 0; j < TN; ++j) fw[slot][j] = *reinterpret_cast<const u32x4_t*>(base + fragW + j * 64 * KB + off);
        };
#pragma unroll
        for (int ch = 0; ch < PF; ++ch) read_frags(ch % SLOTS, ch);
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            if (ch + PF < NCH) read_frags((ch + PF) % SLOTS, ch + PF);
            if (LOAD) {
#pragma unroll
                for (int i = ch * NLOAD / NCH; i < (ch + 1) * NLOAD / NCH; ++i) issue(i, kt_load, st_load);
            }
            if (LOAD || ch < n_chunks) {  // uniform; only the partial last tile has fewer chunks
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) TR::mma(acc[i][j], fa[ch % SLOTS][i], fw[ch % SLOTS][j]);
                if ((kNorm == NORM_RMS || kNorm == NORM_LAYER) && (ch & 1) == wn) {
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            ssq[i][e] = add_squares_bf16x2(fa[ch % SLOTS][i][e], ssq[i][e]);
                            if (kNorm == NORM_LAYER) ssum[i][e] = add_pair_bf16x2(fa[ch % SLOTS][i][e], ssum[i][e]);
                        }
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // keeps the reads and loads where they were placed
        }
    };

    // Stage kt % NS holds tile kt.  Before tile kt is multiplied every wavefront waits for
    // its own loads of that tile (the IN_FLIGHT younger ones may still be pending) and all
    // meet at the barrier, which also tells that stage (kt - 1) % NS has been read by
    // everyone: the loads of tile kt + NS - 1 go there.  Past the last tile the ring keeps
    // re-fetching it into free stages, so the counts stay the same to the end.
#pragma unroll
    for (int t = 0; t < NS - 1; ++t)
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) issue(i, min(t, nkt - 1), t);
    int cs = 0, ls = NS - 1;
    for (int kt = 0; kt < nkt_full; ++kt) {
        wait_vmcnt<IN_FLIGHT>();
        __syncthreads();
        multiply(cs, std::true_type{}, ls, min(kt + NS - 1, nkt - 1), NCH);
        cs = (cs + 1 == NS) ? 0 : cs + 1;
        ls = (ls + 1 == NS) ? 0 : ls + 1;
    }
    if (nkt > nkt_full) {
        wait_vmcnt<IN_FLIGHT>();
        __syncthreads();
        multiply(cs, std::false_type{}, 0, 0, (a.K - nkt_full * BK) / 16);
    }
    // The bias columns of every sub-tile's epilogue (thread layout as for the residual) are
    // requested here, while the ring's last loads drain, and not behind each sub-tile's barrier.
    float bias_pf[TN][16] = {};
    if (kEpi == EPI_PLAIN && a.bias != nullptr) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                bias_pf[j][e] = a.bias[min((ntw * TN + j) * BN + (e >> 3) * 32 + (tid & 3) * 8 + (e & 7), a.N - 1)];
    }
    wait_vmcnt<0>();  // the re-fetches must have landed before the ring is reused for C
    __syncthreads();

    // The accumulators leave through LDS one 64x64 sub-tile at a time (the epilogue wants whole
    // rows of a sub-tile per thread: rotation partners, 16-byte stores).  Two staging buffers in
    // turn: sub-tile n + 1 is written between the same pair of barriers in which sub-tile n is
    // read, so a sub-tile costs one barrier, and its LDS writes overlap the previous epilogue's
    // memory traffic.
    uint32_t* Cb[2] = {reinterpret_cast<uint32_t*>(lds), reinterpret_cast<uint32_t*>(lds + C_BYTES)};
    float* row_stat = reinterpret_cast<float*>(lds + 2 * C_BYTES);  // [wn][ROWS_A][2]
    if (kNorm == NORM_LAYER_PRE) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            float q = 0.f, u = 0.f;
#pragma unroll
            for (int t = 0; t < STAT_MAX_TILES / 4; ++t) {
                const bool on = (tid & 3) + 4 * t < a.n_stat;  // the clamped repeats of the last tile do not count
                q += on ? st_pf[i][t][0] : 0.f;
                u += on ? st_pf[i][t][1] : 0.f;
            }
            q += __uint_as_float(dpp_u32<DPP_XOR1>(__float_as_uint(q)));
            u += __uint_as_float(dpp_u32<DPP_XOR1>(__float_as_uint(u)));
            q += __uint_as_float(dpp_u32<DPP_XOR2>(__float_as_uint(q)));
            u += __uint_as_float(dpp_u32<DPP_XOR2>(__float_as_uint(u)));
            if ((tid & 3) == 0) {  // the epilogue adds two partial pairs per row: the totals and zeros
                float* dst = row_stat + (i * 64 + (tid >> 2)) * 2;
                dst[0] = q;
                dst[1] = u;
                dst[ROWS_A * 2] = 0.f;
                dst[ROWS_A * 2 + 1] = 0.f;
            }
        }
    } else if (kNorm) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            float q = (ssq[i][0] + ssq[i][1]) + (ssq[i][2] + ssq[i][3]);
            float u = (ssum[i][0] + ssum[i][1]) + (ssum[i][2] + ssum[i][3]);
            q += __shfl_xor(q, 32, 64);
            u += __shfl_xor(u, 32, 64);
            if (g == 0) {
                float* dst = row_stat + (wn * ROWS_A + (wm + 2 * i) * 32 + r) * 2;
                dst[0] = q;
                dst[1] = u;
            }
        }
    }
    constexpr int NSUB = TM * TN;
    auto stage_c = [&](int n) __attribute__((always_inline)) {
        const int i = n / TN, j = n % TN;
        uint32_t* C = Cb[n & 1];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
            for (int ii = 0; ii < 4; ++ii)
                C[(wm * 32 + 8 * jj + 4 * g + ii) * C_STRIDE + wn * 32 + r] = acc_bits(acc[i][j][4 * jj + ii]);
    };
    stage_c(0);
#pragma unroll
    for (int n = 0; n < NSUB; ++n) {
        const int i = n / TN, j = n % TN;
        __syncthreads();  // sub-tile n is staged, and the buffer of sub-tile n - 1 has been read by everyone
        if (n + 1 < NSUB) stage_c(n + 1);
        const int nt_sub = ntw * TN + j;
        if (nt_sub < a.n_tiles)
            epilogue_64x64<T, kEpi, kEpi == EPI_PLAIN>(a, Cb[n & 1], m0 + i * 64, nt_sub, tc[j], tid, pf, res_pf[i][j][0],
                                                       res_pf[i][j][1], kNorm == NORM_LAYER_PRE ? NORM_LAYER : kNorm, row_stat + i * 128, ROWS_A * 2, bias_pf[j]);
    }
}

// ---- A few rows (M <= 64) of a bf16 projection: 16 columns per workgroup, K split over its wavefronts ----
// One observation's suffix rows through a projection.  The weights are read once and from
// memory (a step touches every layer's weights once, more than the caches hold), and what a
// CU gets out of memory is bounded by its own requests in flight, not by the chip: the tiled
// kernels' 64-column tiles put such a launch on N / 64 CUs, a tenth of the chip, each walking
// all of K tile by tile.  Here a workgroup owns 16 columns -- N / 16 workgroups -- and its
// eight wavefronts each take an eighth of K and request all of it at once, straight into
// MFMA operand registers: v_mfma_f32_16x16x32_bf16 with the weight rows as the left operand
// (16 columns x 32 k) and 16 activation rows as the right one, so that lane (c, q) =
// (lane % 16, lane / 16) reads 16 bytes (8 k) of weight row c and of activation row c, and
// four lanes cover 64 consecutive bytes of a row.  The partial tiles meet in LDS and are
// added in wavefront order; the epilogues (bias, fused-norm scaling, rotation, scatter into
// the caches, residual) are the tiled kernels' arithmetic on a (row, column pair) per thread.
// The 16 columns are 8 + 8: for rotated segments the columns d .. d + 7 of a head and their
// partners d + D / 2, else 16 consecutive columns.  The sums are formed in another order than
// by the tiled kernels: the two agree to fp32 rounding, not bit for bit.
constexpr int SR_WAVES = 8, SR_MAX_ROWS = 64, SR_PSTR = 20, SR_MAX_K = 2048;
struct RowCols {
    int base_lo, base_hi;  // rows of W of tile columns [0, 8) and [8, 16)
    int seg;               // 0 Q, 1 K, 2 V (QKV mode)
    int col_lo, col_hi;    // segment-local column of tile column 0 and of tile column 8
    bool rope;
};
template <int kEpi>
__device__ __forceinline__ RowCols row_cols(const GemmArgs& a, int t) {
    RowCols rc;
    rc.seg = 0;
    rc.rope = false;
    if (kEpi != EPI_QKV) {
        rc.base_lo = rc.col_lo = t * 16;
        rc.base_hi = rc.col_hi = t * 16 + 8;
        return rc;
    }
    const int tq = a.Hq * a.D / 16, tk = a.nk * a.D / 16;
    int lt = t, seg_base = 0;
    if (t >= tq + tk) {
        rc.seg = 2;
        lt = t - tq - tk;
        seg_base = (a.Hq + a.nk) * a.D;
    } else if (t >= tq) {
        rc.seg = 1;
        lt = t - tq;
        seg_base = a.Hq * a.D;
    }
    rc.rope = (a.cos_t != nullptr) && rc.seg != 2;
    if (rc.rope) {
        const int tph = a.D / 16;  // tiles per head
        const int head = lt / tph, chunk = lt % tph;
        rc.col_lo = head * a.D + chunk * 8;
        rc.col_hi = rc.col_lo + a.D / 2;
    } else {
        rc.col_lo = lt * 16;
        rc.col_hi = rc.col_lo + 8;
    }
    rc.base_lo = seg_base + rc.col_lo;
    rc.base_hi = seg_base + rc.col_hi;
    return rc;
}

template <int kEpi, int kNorm, int RB, int MAXC, int NB>  // RB: 16-row blocks; MAXC: 32-k chunks per wavefront held in registers, K <= 256 MAXC; NB: 16-column tiles per workgroup
__global__ void __launch_bounds__(SR_WAVES * 64) gemm_rows_bf16_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(16))) float part[SR_WAVES][NB][RB * 16][SR_PSTR];
    __shared__ float stat_part[SR_WAVES][RB * 16][2];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int n_t16 = (a.N + 15) / 16;
    RowCols rc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) rc[nb] = row_cols<kEpi>(a, min((int)blockIdx.x * NB + nb, n_t16 - 1));
    const int nch = (a.K + 31) / 32, per = (nch + SR_WAVES - 1) / SR_WAVES, ch0 = wave * per;

    // rows past N or M and pieces past K are read from valid addresses; their products are dropped or zeroed
    const unsigned char* wrow[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
        wrow[nb] = (const unsigned char*)a.W + (long)min(max(c < 8 ? rc[nb].base_lo + c : rc[nb].base_hi + c - 8, 0), a.N - 1) * a.K * 2;
    const unsigned char* xrow[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) xrow[rb] = (const unsigned char*)a.A + (long)min(rb * 16 + c, a.M - 1) * a.K * 2;
    u32x4_t wf[MAXC][NB], xf[MAXC][RB];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int ch = min(ch0 + i, nch - 1);
        const long off = (long)min(ch * 32 + 8 * q, a.K - 8) * 2;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) wf[i][nb] = *reinterpret_cast<const u32x4_t*>(wrow[nb] + off);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) xf[i][rb] = *reinterpret_cast<const u32x4_t*>(xrow[rb] + off);
    }
    // What the epilogue reads from memory is requested now, behind the operand loads.  Epilogue
    // thread -> row tid / 8, tile columns i = tid % 8 and 8 + i.  No branch around the loads:
    // addresses are clamped into the arrays and values that are not needed are dropped.
    const int erow = tid >> 3, ei = tid & 7;
    const int em = min(erow, a.M - 1);
    int n_lo[NB], n_hi[NB];
    float b_lo[NB], b_hi[NB], cs_lo[NB], cs_hi[NB], g_lo[NB], g_hi[NB], rot_c[NB], rot_s[NB], r_lo[NB], r_hi[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        n_lo[nb] = min(rc[nb].base_lo + ei, a.N - 1);
        n_hi[nb] = min(rc[nb].base_hi + ei, a.N - 1);
        b_lo[nb] = b_hi[nb] = cs_lo[nb] = cs_hi[nb] = r_lo[nb] = r_hi[nb] = rot_s[nb] = 0.f;
        g_lo[nb] = g_hi[nb] = rot_c[nb] = 1.f;
        if (a.bias) {
            b_lo[nb] = a.bias[n_lo[nb]];
            b_hi[nb] = a.bias[n_hi[nb]];
        }
        if (kNorm == NORM_LAYER) {
            cs_lo[nb] = a.colsum[n_lo[nb]];
            cs_hi[nb] = a.colsum[n_hi[nb]];
        }
        if (kEpi == EPI_PLAIN) {
            if (a.col_gate) {
                g_lo[nb] = a.col_gate[n_lo[nb]];
                g_hi[nb] = a.col_gate[n_hi[nb]];
            }
            if (a.residual) {
                if (a.out_bf16) {
                    r_lo[nb] = bf2f(((const bf16_t*)a.residual)[(long)em * a.N + n_lo[nb]]);
                    r_hi[nb] = bf2f(((const bf16_t*)a.residual)[(long)em * a.N + n_hi[nb]]);
                } else {
                    r_lo[nb] = ((const float*)a.residual)[(long)em * a.N + n_lo[nb]];
                    r_hi[nb] = ((const float*)a.residual)[(long)em * a.N + n_hi[nb]];
                }
            }
        }
        if (kEpi == EPI_QKV && rc[nb].rope) {
            const int half = a.D >> 1;
            const long ri = (long)(em % a.S) * half + (rc[nb].col_lo % a.D) + ei;
            rot_c[nb] = a.cos_t[ri];
            rot_s[nb] = a.sin_t[ri];
        }
    }

    f32x4_t acc[NB][RB];
    float ssq[RB], ssum[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb][rb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        ssq[rb] = ssum[rb] = 0.f;
    }
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        if (i < per && ch0 + i < nch) {  // uniform
            const bool inside = (ch0 + i) * 32 + 8 * q < a.K;  // K is a multiple of 8: a piece is inside or outside as a whole
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                u32x4_t xv = xf[i][rb];
                if (!inside) xv = u32x4_t{0u, 0u, 0u, 0u};
                if (kNorm) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        ssq[rb] = add_squares_bf16x2(xv[e], ssq[rb]);
                        if (kNorm == NORM_LAYER) ssum[rb] = add_pair_bf16x2(xv[e], ssum[rb]);
                    }
                }
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[nb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, wf[i][nb]), __builtin_bit_cast(bf16x8_t, xv),
                                                                          acc[nb][rb], 0, 0, 0);
            }
        }
    }
    // acc[nb][rb][e]: column 4 q + e of tile nb, row 16 rb + c
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) *reinterpret_cast<f32x4_t*>(&part[wave][nb][rb * 16 + c][4 * q]) = acc[nb][rb];
        if (kNorm) {
            const float s2 = rows_sum(ssq[rb]), s1 = rows_sum(ssum[rb]);
            if (q == 0) {
                stat_part[wave][rb * 16 + c][0] = s2;
                stat_part[wave][rb * 16 + c][1] = s1;
            }
        }
    }
    __syncthreads();
    if (erow >= RB * 16 || erow >= a.M) return;
    const int m = erow;
    float sq = 0.f, sm = 0.f;
    if (kNorm) {
#pragma unroll
        for (int w = 0; w < SR_WAVES; ++w) {
            sq += stat_part[w][erow][0];
            sm += stat_part[w][erow][1];
        }
    }
    const int b = kEpi == EPI_QKV ? m / a.S : 0, s = kEpi == EPI_QKV ? m % a.S : 0;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        if ((int)blockIdx.x * NB + nb >= n_t16) break;  // uniform
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int w = 0; w < SR_WAVES; ++w) {
            lo += part[w][nb][erow][ei];
            hi += part[w][nb][erow][8 + ei];
        }
        if (kNorm) {
            const float inv_k = 1.0f / (float)a.K;
            if (kNorm == NORM_LAYER) {
                // sum_k (x - mean) rstd W[n][k] = rstd acc - (mean rstd) colsum[n]
                const float mean = sm * inv_k;
                const float f = rsqrtf(fmaxf(sq * inv_k - mean * mean, 0.f) + a.norm_eps);
                const float ms = mean * f;
                lo = lo * f - ms * cs_lo[nb];
                hi = hi * f - ms * cs_hi[nb];
            } else {
                const float f = rsqrtf(sq * inv_k + a.norm_eps);
                lo *= f;
                hi *= f;
            }
        }
        lo += b_lo[nb];
        hi += b_hi[nb];
        const bool ok_lo = rc[nb].base_lo + ei < a.N, ok_hi = rc[nb].base_hi + ei < a.N;
        if (kEpi == EPI_PLAIN) {
            if (a.act != VLA_ACT_NONE) {
                lo = apply_act(lo, a.act);
                hi = apply_act(hi, a.act);
            }
            lo = lo * g_lo[nb] + r_lo[nb];
            hi = hi * g_hi[nb] + r_hi[nb];
            const long o = (long)m * a.N;
            if (a.out_bf16) {
                if (ok_lo) ((bf16_t*)a.Y)[o + n_lo[nb]] = f2bf(lo);
                if (ok_hi) ((bf16_t*)a.Y)[o + n_hi[nb]] = f2bf(hi);
            } else {
                if (ok_lo) ((float*)a.Y)[o + n_lo[nb]] = lo;
                if (ok_hi) ((float*)a.Y)[o + n_hi[nb]] = hi;
            }
            continue;
        }
        // QKV: rotation, scatter
        if (rc[nb].rope) {
            const float x0 = lo, x1 = hi;
            lo = x0 * rot_c[nb] - x1 * rot_s[nb];
            hi = x1 * rot_c[nb] + x0 * rot_s[nb];
        }
#pragma unroll
        for (int hlf = 0; hlf < 2; ++hlf) {
            const float v = hlf ? hi : lo;
            const int col = (hlf ? rc[nb].col_hi : rc[nb].col_lo) + ei;
            if (rc[nb].seg == 0) {
                ((bf16_t*)a.q_out)[(long)m * (a.Hq * a.D) + col] = f2bf(v);
            } else {
                const int head = col / a.D, d = col % a.D;
                if (rc[nb].seg == 1) ((bf16_t*)a.k_cache)[(((long)b * a.Hkv + head) * a.t_max + a.tok_offset + s) * a.D + d] = f2bf(v);
                else ((bf16_t*)a.vt_cache)[(((long)b * a.Hkv + head) * a.D + d) * (long)a.t_max + a.tok_offset + s] = f2bf(v);
            }
        }
    }
}

// Large-M ternary GEMM (BitVLA prefill: M = batch x prefix tokens).  Workgroup tile
// (64*WM) x 256 with WM x 2 wavefronts, each owning 64 x 128 = 2 x 4 MFMA blocks (128
// accumulator registers), so one 16-byte A fragment feeds four MFMAs and one weight
// fragment two.  int8 activations go global -> registers -> double-buffered LDS (one
// barrier per 128-k tile).  The 2-bit weights never touch LDS: the fragment-major layout
// makes each (32 columns x 32 k) fragment one coalesced 256-byte load per wavefront; a
// word is expanded to bytes with shift/mask right before use and its register is
// refilled at once with the word of the next k-tile, a full tile of MFMAs ahead of need.
template <int WM>
__global__ void __launch_bounds__(WM * 128, 2) ternary_gemm_big_kernel(GemmArgs a) {
    constexpr int NT = WM * 128, ROWS = WM * 64, STRIDE = 144, VA = ROWS * 8 / NT;
    constexpr int T_STRIDE = 272;  // bf16 transpose staging: 128 columns + 16 bytes of padding
    __shared__ __attribute__((aligned(16))) unsigned char lds[2][ROWS * STRIDE];
    static_assert(sizeof(lds) >= (size_t)(WM * 2) * 32 * T_STRIDE, "epilogue staging must fit in the A buffers");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int g = lane >> 5, r = lane & 31;
    // id % 8 (the XCD) = M tile % 8: workgroups sharing an L2 share their activation rows,
    // the larger operand, and stream the whole (4x smaller) packed weight matrix.
    const int m_tiles = (a.M + ROWS - 1) / ROWS, mt_pad = (m_tiles + 7) & ~7;
    const int mt = blockIdx.x % mt_pad;
    if (mt >= m_tiles) return;
    const int m0 = mt * ROWS, n0 = (blockIdx.x / mt_pad) * 256 + wn * 128;

    const int kgroups = a.K / 32, nblocks = (a.N + 31) / 32;
    const uint32_t* wp[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int nb = n0 / 32 + j;
        nb = nb < nblocks ? nb : nblocks - 1;  // columns past N: any valid block, result dropped
        wp[j] = (const uint32_t*)a.W + (long)nb * kgroups * 64 + lane;
    }
    const unsigned char* ap[VA];
#pragma unroll
    for (int v = 0; v < VA; ++v) {
        const int idx = tid + v * NT;
        const int m = min(m0 + idx / 8, a.M - 1);  // rows past M: a valid row, result dropped
        ap[v] = (const unsigned char*)a.A + (long)m * a.K + (idx % 8) * 16;
    }

    i32x16_t acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    u32x4_t ra[VA];
    uint32_t bw[4][4];  // [k group of the tile][column block]
    const int nkt = a.K / 128;

#pragma unroll
    for (int ch = 0; ch < 4; ++ch)
#pragma unroll
        for (int j = 0; j < 4; ++j) bw[ch][j] = wp[j][ch * 64];
#pragma unroll
    for (int v = 0; v < VA; ++v) ra[v] = *reinterpret_cast<const u32x4_t*>(ap[v]);
#pragma unroll
    for (int v = 0; v < VA; ++v) {
        const int idx = tid + v * NT;
        *reinterpret_cast<u32x4_t*>(&lds[0][(idx / 8) * STRIDE + (idx % 8) * 16]) = ra[v];
    }
    __syncthreads();

    for (int kt = 0; kt < nkt; ++kt) {
        const unsigned char* cur = lds[kt & 1];
        const int kn = kt + 1 < nkt ? kt + 1 : kt;  // the last tile re-reads itself; copy unused
#pragma unroll
        for (int v = 0; v < VA; ++v) ra[v] = *reinterpret_cast<const u32x4_t*>(ap[v] + (long)kn * 128);
        u32x4_t fa[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
            fa[0][i] = *reinterpret_cast<const u32x4_t*>(cur + (wm * 64 + i * 32 + r) * STRIDE + g * 16);
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) {
            u32x4_t fw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w = bw[ch][j];
                fw[j][0] = w & 0x03030303u;
                fw[j][1] = (w >> 2) & 0x03030303u;
                fw[j][2] = (w >> 4) & 0x03030303u;
                fw[j][3] = (w >> 6) & 0x03030303u;
                bw[ch][j] = wp[j][(kn * 4 + ch) * 64];
            }
            if (ch < 3) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    fa[(ch + 1) & 1][i] =
                        *reinterpret_cast<const u32x4_t*>(cur + (wm * 64 + i * 32 + r) * STRIDE + (ch + 1) * 32 + g * 16);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) Traits<int8_t>::mma(acc[i][j], fa[ch & 1][i], fw[j]);
        }
        unsigned char* nxt = lds[(kt + 1) & 1];
#pragma unroll
        for (int v = 0; v < VA; ++v) {
            const int idx = tid + v * NT;
            *reinterpret_cast<u32x4_t*>(nxt + (idx / 8) * STRIDE + (idx % 8) * 16) = ra[v];
        }
        __syncthreads();
    }

    // Accumulator element 4jj+ii of block (i, j) is row 8jj + 4g + ii, column r.
    if (a.acc_out) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * g + (e & 3);
                if (m >= a.M) continue;
                const int rs2 = 2 * a.rowsum[m];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = n0 + j * 32 + r;
                    if (n < a.N) a.acc_out[(long)m * a.N + n] = acc[i][j][e] - rs2;
                }
            }
    }
    if (!a.Y) return;

    // bf16 output: out = float(acc - 2*rowsum) / s[m] * ws[group], staged per wavefront as
    // 32 rows x 128 columns in LDS and written with 16-byte stores (16 lanes per row).
    const int group = a.N / a.ws_num;
    float wsc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + j * 32 + r;
        wsc[j] = n < a.N ? a.ws[n / group] : 0.f;
    }
    // The division is the correctly rounded IEEE quotient.  When every scale of the
    // wavefront's 64 rows is far from the exponent limits it is computed as the refinement
    // sequence of the full-range expansion without its operand scaling (identical bits):
    // y ~ 1/s by one Newton step on v_rcp_f32, then q0 = a*y, two residual corrections.
    // Lane l holds the activation scale and the row sum of the wavefront's row l: one coalesced
    // load each.  The loops below pick a row's pair out of these with v_readlane (the row of an
    // accumulator element is a compile-time constant apart from the lane's half g) instead of
    // fetching it from memory where it is needed, which cost a round trip per pair of rows.
    const int lane_row = min(m0 + wm * 64 + lane, a.M - 1);
    const float s_lane = a.s[lane_row];
    const int rs_lane = a.rowsum[lane_row];
    const float sabs = fabsf(s_lane);
    const bool fast = __builtin_amdgcn_ballot_w64(sabs > 0x1p-60f && sabs < 0x1p60f) == ~0ull;
    unsigned char* tp = &lds[0][0] + wave * (32 * T_STRIDE);
    const bool vec_ok = (a.N % 8) == 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        // the residual vectors of this half of the rows, requested ahead of the staging arithmetic
        u32x4_t res_v[8] = {};
        const bool res_vec = a.residual != nullptr && vec_ok;
        if (res_vec) {
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const int m = min(m0 + wm * 64 + i * 32 + p * 4 + (lane >> 4), a.M - 1), n = min(n0 + (lane & 15) * 8, a.N - 8);
                res_v[p] = *reinterpret_cast<const u32x4_t*>((const bf16_t*)a.residual + (long)m * a.N + n);
            }
        }
        if (fast) {
#pragma unroll
            for (int jj = 0; jj < 4; ++jj)
#pragma unroll
                for (int ip = 0; ip < 4; ip += 2) {
                    const int row = 8 * jj + 4 * g + ip;
                    float sm[2], y[2];
                    int rs2[2];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        // row of the wavefront's tile: i * 32 + 8 jj + 4 g + ip + t (rows past M repeat row M - 1, as lane_row does)
                        const int r0 = i * 32 + 8 * jj + ip + t;
                        const int rs_g0 = __builtin_amdgcn_readlane(rs_lane, r0), rs_g1 = __builtin_amdgcn_readlane(rs_lane, r0 + 4);
                        const int sb_g0 = __builtin_amdgcn_readlane(__float_as_int(s_lane), r0);
                        const int sb_g1 = __builtin_amdgcn_readlane(__float_as_int(s_lane), r0 + 4);
                        rs2[t] = 2 * (g ? rs_g1 : rs_g0);
                        sm[t] = __int_as_float(g ? sb_g1 : sb_g0);
                        const float y0 = __builtin_amdgcn_rcpf(sm[t]);
                        y[t] = __builtin_fmaf(__builtin_fmaf(-sm[t], y0, 1.0f), y0, y0);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float o[2];
#pragma unroll
                        for (int t = 0; t < 2; ++t) {
                            const float av = (float)(acc[i][j][4 * jj + ip + t] - rs2[t]);
                            const float q0 = av * y[t];
                            const float q1 = __builtin_fmaf(__builtin_fmaf(-sm[t], q0, av), y[t], q0);
                            o[t] = __builtin_fmaf(__builtin_fmaf(-sm[t], q1, av), y[t], q1) * wsc[j];
                        }
                        const uint32_t pk = pack_bf2(o[0], o[1]);
                        *reinterpret_cast<bf16_t*>(tp + row * T_STRIDE + (j * 32 + r) * 2) = (bf16_t)(pk & 0xffff);
                        *reinterpret_cast<bf16_t*>(tp + (row + 1) * T_STRIDE + (j * 32 + r) * 2) = (bf16_t)(pk >> 16);
                    }
                }
        } else {
#pragma unroll 1
            for (int e = 0; e < 16; ++e) {
                const int row = 8 * (e >> 2) + 4 * g + (e & 3);
                const int mm = min(m0 + wm * 64 + i * 32 + row, a.M - 1);
                const int rs2 = 2 * a.rowsum[mm];
                const float sm = a.s[mm];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    int v = 0;
#pragma unroll
                    for (int e2 = 0; e2 < 16; ++e2) v = (e2 == e) ? acc[i][j][e2] : v;
                    *reinterpret_cast<bf16_t*>(tp + row * T_STRIDE + (j * 32 + r) * 2) =
                        f2bf((float)(v - rs2) / sm * wsc[j]);
                }
            }
        }
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int row = p * 4 + (lane >> 4), c16 = lane & 15;
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(tp + row * T_STRIDE + c16 * 16);
            const int m = m0 + wm * 64 + i * 32 + row, n = n0 + c16 * 8;
            if (m >= a.M) continue;
            bf16_t* dst = (bf16_t*)a.Y + (long)m * a.N + n;
            const bf16_t* res = a.residual ? (const bf16_t*)a.residual + (long)m * a.N + n : nullptr;
            if (vec_ok && n + 8 <= a.N) {
                u32x4_t o = v;
                if (res) {  // out = bf16(out + residual), both already bf16
                    const u32x4_t rr = res_v[p];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        o[e] = pack_bf2(__uint_as_float(v[e] << 16) + __uint_as_float(rr[e] << 16),
                                        __uint_as_float(v[e] & 0xffff0000u) + __uint_as_float(rr[e] & 0xffff0000u));
                }
                *reinterpret_cast<u32x4_t*>(dst) = o;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < a.N) {
                        const bf16_t o = (bf16_t)(v[e >> 1] >> (16 * (e & 1)));
                        dst[e] = res ? f2bf(bf2f(o) + bf2f(res[e])) : o;
                    }
            }
        }
    }
}

// ---- Large-M ternary GEMM on v_mfma_i32_16x16x64_i8 (BitVLA prefill) ------------------
// The 16x16x64 form moves a quarter of the accumulator registers per multiply-add that the
// 32x32x32 form does, and on this part that is what the matrix pipe's clock follows: the
// same product streams about a fifth faster.  Everything around the MFMAs is built so that
// nothing the compiler schedules can sit between a load and its first use:
//
//  - int8 activation tiles (128 rows x 128 k) go from global memory straight into a
//    three-stage LDS ring (global_load_lds_dwordx4, rows unpadded, 16-byte pieces
//    XOR-swizzled by (row >> 1) & 7 so that a fragment read touches every bank once);
//  - a wavefront's packed weight words (one dword = 16 codes of one column) go from the
//    fragment-major layout into registers with inline-assembly loads, refilled in place
//    right after they are expanded, a full k-tile ahead of their next use;
//  - both kinds are counted by hand: every pass issues the same loads in the same order,
//    so "the words of this chunk have landed" is always s_waitcnt vmcnt(NB / 2 + 4), and the
//    activation tile of a pass is older than that.  One barrier per k-tile.
//
// The product is formed as D = W . A^T: a lane ends up with four consecutive output
// columns of one row, so the row's scale and row sum are per-lane constants (no lane
// exchange), the accumulators start at -2 * rowsum (the code offset), and the bf16 results
// go to the LDS staging area as 16-byte pieces (a 16-lane group takes the even columns of
// a 32-column block in one MFMA and the odd ones in the next, so that its two weight words
// are one 8-byte load and its eight outputs per row are consecutive).
//
// Registers written by the inline-assembly loads are "in flight" until the matching wait.
// Each of them is an in/out operand of that wait, which keeps the compiler from reading it
// early and from giving the register to anything else in between.  The kernel must not
// spill (a spilled in-flight register is stored before its data arrives and its register
// reused while the load is still due): vla_cpp_amd/build.py checks the scratch size.
template <int IMM>
__device__ __forceinline__ void tern_wload_i(u32x2_t& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
}
__device__ __forceinline__ void tern_aload_lds(uint32_t voff, const void* sbase, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void tern_gload(uint32_t& dst, const void* p) {
    asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
template <int CNT>
__device__ __forceinline__ void tern_wait_words(u32x2_t (&w)[4]) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]) : "n"(CNT));
}

// 2 x 2 wavefronts, each 64 rows x 128 columns (4 x 8 blocks of 16 x 16); workgroup tile 128 x 256.
__global__ void __launch_bounds__(256, 2) ternary_gemm_x16_kernel(GemmArgs a) {
    constexpr int NB = 8, MB = 4, NS = 3, ROWS = 128, CW = 16 * NB, COLS = 2 * CW, STAGE = ROWS * 128;
    constexpr int CNT = NB / 2 + 4;    // loads younger than a chunk's words when they are waited for
    constexpr int T_STRIDE = 272;      // staging row: 128 bf16 + 16 bytes
    __shared__ __attribute__((aligned(1024))) unsigned char lds[NS * STAGE];
    static_assert(NS * STAGE >= 4 * 16 * T_STRIDE, "epilogue staging must fit in the ring");

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int q = lane >> 4, c = lane & 15;
    // id % 8 (the XCD) = M tile % 8: workgroups sharing an L2 share their activation rows,
    // the larger operand, and stream the whole (4x smaller) packed weight matrix.
    const int m_tiles = (a.M + ROWS - 1) / ROWS, mt_pad = (m_tiles + 7) & ~7;
    const int mt = blockIdx.x % mt_pad;
    if (mt >= m_tiles) return;
    const int m0 = mt * ROWS, n0 = (blockIdx.x / mt_pad) * COLS + wn * CW;

    // Row constants of the lane's four output rows m = m0 + 64 wm + 16 mb + c: requested
    // before everything else, valid after the first wait of the ring.
    uint32_t rs_raw[MB], sc_raw[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = min(m0 + wm * 64 + mb * 16 + c, a.M - 1);
        tern_gload(rs_raw[mb], a.rowsum + m);
        tern_gload(sc_raw[mb], a.s ? a.s + m : (const float*)(a.rowsum + m));
    }
    // The 16 lanes c of a k quarter q take the columns 2 c (block 2 p) and 2 c + 1 (block 2 p + 1) of the 32-column
    // block n0 / 32 + p: the two words sit side by side in the fragment-major layout (k group 2 chunk + q / 2, half
    // q % 2), one 8-byte load.  Byte offsets; both operands fit 32 bits (checked by the launcher).
    const int kgroups = a.K / 32, nblocks = (a.N + 31) / 32;
    uint32_t woff[NB / 2];
#pragma unroll
    for (int p = 0; p < NB / 2; ++p) {
        const int nb32 = min(n0 / 32 + p, nblocks - 1);  // columns past N: any valid block, result dropped
        woff[p] = ((uint32_t)nb32 * (uint32_t)kgroups * 64u + (uint32_t)((q >> 1) * 64 + (q & 1) * 32 + 2 * c)) * 4u;
    }
    // Activation loader: wavefront w fills the 1 KiB slabs 4 w + v of a stage (8 rows each);
    // the lane's slot is piece position lane % 8 of row lane / 8 and holds logical piece (lane % 8) ^ ((row >> 1) & 7).
    uint32_t aoff[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row = (wave * 4 + v) * 8 + (lane >> 3);
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        aoff[v] = (uint32_t)min(m0 + row, a.M - 1) * (uint32_t)a.K + (uint32_t)(piece * 16);  // rows past M: a valid row, result dropped
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds + wave * 4096;  // low 32 bits of a shared-aperture address = LDS offset

    u32x2_t bw[2][NB / 2] = {};  // [chunk][32-column block]: the words of blocks 2 p and 2 p + 1
    const int nkt = a.K / 128;
    const unsigned char* Ab = (const unsigned char*)a.A;
    const unsigned char* Wb = (const unsigned char*)a.W;
#define TERN_WLOAD(ch, base) \
    _Pragma("unroll") for (int p = 0; p < NB / 2; ++p) tern_wload_i<(ch) * 512>(bw[ch][p], woff[p], base);
#define TERN_ALOAD(ch, abase, lbase)                                   \
    tern_aload_lds(aoff[(ch) * 2], abase, (lbase) + ((ch) * 2) * 1024); \
    tern_aload_lds(aoff[(ch) * 2 + 1], abase, (lbase) + ((ch) * 2 + 1) * 1024);

    // Prologue = the issue order of two passes before the first: activation tile 0, then
    // (words of tile 0, activation tile 1) chunk by chunk.  Past the last tile the ring
    // keeps re-fetching it, so the counts stay the same to the end.
#pragma unroll
    for (int v = 0; v < 4; ++v) tern_aload_lds(aoff[v], Ab, lds0 + v * 1024);
    {
        const unsigned char* a1 = Ab + (long)min(1, nkt - 1) * 128;
        TERN_WLOAD(0, Wb) TERN_ALOAD(0, a1, lds0 + STAGE)
        TERN_WLOAD(1, Wb) TERN_ALOAD(1, a1, lds0 + STAGE)
    }
    // Fragment reads: row 64 wm + 16 mb + c, logical piece 4 ch + q at position (4 ch + q) ^ ((c >> 1) & 7).
    const int fsw = (c >> 1) & 7;
    const int fragA = (wm * 64 + c) * 128;

    // Words of (tile 0, chunk 0) have landed, and with them everything older: activation tile 0 and the row constants.
    tern_wait_words<CNT>(bw[0]);
    asm volatile("" : "+v"(rs_raw[0]), "+v"(rs_raw[1]), "+v"(rs_raw[2]), "+v"(rs_raw[3]), "+v"(sc_raw[0]), "+v"(sc_raw[1]), "+v"(sc_raw[2]), "+v"(sc_raw[3]));
    i32x4_t acc[NB][MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int init = -2 * (int)rs_raw[mb];  // 2-bit codes are t + 2: sum_k q (t + 2) - 2 rowsum
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb][mb] = i32x4_t{init, init, init, init};
    }
    int cs = 0, ls = 2;
    for (int kt = 0; kt < nkt; ++kt) {
        const unsigned char* cur = lds + cs * STAGE;
        const unsigned char* wn_base = Wb + (long)min(kt + 1, nkt - 1) * 1024;
        const unsigned char* an_base = Ab + (long)min(kt + 2, nkt - 1) * 128;
        const uint32_t lds_ld = lds0 + ls * STAGE;
        u32x4_t fa[2][MB];
        __syncthreads();  // every wavefront's loads of this tile have landed; stage ls has been read by everyone
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            fa[0][mb] = *reinterpret_cast<const u32x4_t*>(cur + fragA + mb * 16 * 128 + ((q ^ fsw) * 16));
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            if (ch > 0) tern_wait_words<CNT>(bw[ch]);
            u32x4_t fw[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const uint32_t w = bw[ch][nb >> 1][nb & 1];
                fw[nb][0] = w & 0x03030303u;
                fw[nb][1] = (w >> 2) & 0x03030303u;
                fw[nb][2] = (w >> 4) & 0x03030303u;
                fw[nb][3] = (w >> 6) & 0x03030303u;
            }
            // refill the words just expanded with the next k-tile's, then two activation slabs of the tile after that
            if (ch == 0) { TERN_WLOAD(0, wn_base) TERN_ALOAD(0, an_base, lds_ld) }
            if (ch == 1) { TERN_WLOAD(1, wn_base) TERN_ALOAD(1, an_base, lds_ld) }
            if (ch == 0) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    fa[1][mb] = *reinterpret_cast<const u32x4_t*>(cur + fragA + mb * 16 * 128 + (((4 + q) ^ fsw) * 16));
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[nb][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4_t, fw[nb]),
                                                                        __builtin_bit_cast(i32x4_t, fa[ch][mb]), acc[nb][mb], 0, 0, 0);
        }
        tern_wait_words<CNT>(bw[0]);  // the next tile's first chunk (and, older than it, the next activation tile)
        cs = (cs + 1 == NS) ? 0 : cs + 1;
        ls = (ls + 1 == NS) ? 0 : ls + 1;
    }
#undef TERN_WLOAD
#undef TERN_ALOAD
    // the ring's trailing loads (repeats of the last tile) still target the word registers and the LDS stages
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(bw[0][0]), "+v"(bw[0][1]), "+v"(bw[0][2]), "+v"(bw[0][3]), "+v"(bw[1][0]), "+v"(bw[1][1]), "+v"(bw[1][2]), "+v"(bw[1][3]));
    __syncthreads();

    // acc[nb][mb][i]: column n = n0 + 32 (nb / 2) + 2 (4 q + i) + nb % 2, row m = m0 + 64 wm + 16 mb + c
    if (a.acc_out) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int m = m0 + wm * 64 + mb * 16 + c;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + (nb >> 1) * 32 + 2 * (4 * q + i) + (nb & 1);
                    if (m < a.M && n < a.N) a.acc_out[(long)m * a.N + n] = acc[nb][mb][i];
                }
        }
    }
    if (!a.Y) return;

    // bf16 output: out = float(acc) / s[m] * ws[group], staged per wavefront as 16 rows x 128
    // columns and written with 16-byte stores (16 lanes per row), the residual added on the way.
    // The quotient is the correctly rounded one.  For a positive scale away from the exponent
    // limits it is computed with the scale's exponent taken out: y ~ 1 / mantissa by one Newton
    // step on v_rcp_f32, q0 = a y, one residual correction; for |a| < 2^20 that sequence gives
    // the IEEE quotient for every mantissa (checked exhaustively on the device), and the power
    // of two goes back in exactly.  Larger accumulators take a second correction (the compiler's
    // own sequence without its operand scaling); other scales take the division operator.
    const int group = a.N / a.ws_num;
    float wsc[NB / 2];  // one weight scale per 32-column block (the launcher checks that a scale group is a multiple of 32 columns)
    bool ok = true;
#pragma unroll
    for (int p = 0; p < NB / 2; ++p) {
        wsc[p] = a.ws[min(n0 + p * 32, a.N - 1) / group];
        const float wa = fabsf(wsc[p]);
        ok = ok && (wa == 0.f || (wa > 0x1p-60f && wa < 0x1p60f));  // 2^-e ws below is then exact
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const float sm = __uint_as_float(sc_raw[mb]);
        ok = ok && sm > 0x1p-60f && sm < 0x1p60f;
    }
    const bool fast = __builtin_amdgcn_ballot_w64(ok) == ~0ull;
    const bool one_step = a.K < 8192;  // |acc| <= 128 K < 2^20
    unsigned char* tp = &lds[0] + wave * (16 * T_STRIDE);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        u32x4_t res_v[4] = {};
        if (a.residual) {  // this row block's residual vectors, requested ahead of the staging arithmetic
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int m = min(m0 + wm * 64 + mb * 16 + p * 4 + (lane >> 4), a.M - 1), n = min(n0 + (lane & 15) * 8, a.N - 8);
                res_v[p] = *reinterpret_cast<const u32x4_t*>((const bf16_t*)a.residual + (long)m * a.N + n);
            }
        }
        const float sm = __uint_as_float(sc_raw[mb]);
        if (fast) {
            const uint32_t sb = sc_raw[mb];
            const float mant = __uint_as_float((sb & 0x007fffffu) | 0x3f800000u);      // in [1, 2)
            const float pw = __uint_as_float(0x7f000000u - (sb & 0x7f800000u));         // 2^-(exponent of sm), exact
            const float y0 = __builtin_amdgcn_rcpf(mant);
            const float y = __builtin_fmaf(__builtin_fmaf(-mant, y0, 1.0f), y0, y0);
#pragma unroll
            for (int p = 0; p < NB / 2; ++p) {
                const float pws = pw * wsc[p];  // exact: (q 2^-e) ws and q (2^-e ws) round the same product once
                u32x4_t o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float r2[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const float av = (float)acc[2 * p + h][mb][i];
                        const float q0 = av * y;
                        float q1 = __builtin_fmaf(__builtin_fmaf(-mant, q0, av), y, q0);
                        if (!one_step) q1 = __builtin_fmaf(__builtin_fmaf(-mant, q1, av), y, q1);
                        r2[h] = q1 * pws;
                    }
                    o[i] = pack_bf2(r2[0], r2[1]);
                }
                *reinterpret_cast<u32x4_t*>(tp + c * T_STRIDE + (p * 32 + 8 * q) * 2) = o;
            }
        } else {
#pragma unroll
            for (int p = 0; p < NB / 2; ++p) {
                u32x4_t o;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    o[i] = pack_bf2((float)acc[2 * p][mb][i] / sm * wsc[p], (float)acc[2 * p + 1][mb][i] / sm * wsc[p]);
                *reinterpret_cast<u32x4_t*>(tp + c * T_STRIDE + (p * 32 + 8 * q) * 2) = o;
            }
        }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int row = p * 4 + (lane >> 4), c16 = lane & 15;
            u32x4_t v = *reinterpret_cast<const u32x4_t*>(tp + row * T_STRIDE + c16 * 16);
            const int m = m0 + wm * 64 + mb * 16 + row, n = n0 + c16 * 8;
            if (m >= a.M || n + 8 > a.N) continue;
            if (a.residual) {  // out = bf16(out + residual), both already bf16
                const u32x4_t rr = res_v[p];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    v[e] = pack_bf2(__uint_as_float(v[e] << 16) + __uint_as_float(rr[e] << 16),
                                    __uint_as_float(v[e] & 0xffff0000u) + __uint_as_float(rr[e] & 0xffff0000u));
            }
            // streaming store: the 2 M N bytes leave the L2 as they are produced instead of waiting, dirty, for the
            // write-back at the end of the kernel (each XCD's L2 would hold its whole share until then)
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>((bf16_t*)a.Y + (long)m * a.N + n));
        }
    }
}

// fp32 projection of a few rows (M <= 64: the suffix of one observation in the reference's
// own fp32 case).  The fp32 MFMA gives a CU 256 flop per clock, no more than its plain FMA
// rate, and the MFMA kernel's 64 x 64 tiles leave a 50 x 720 x 960 problem on 12 CUs that walk
// K one after the other (22 us).  Here a wavefront owns 4 rows and 8 output columns and its
// lanes share K: lane l sums k = 256 j + 4 l + (0..3), so a load instruction reads 1 KiB of
// consecutive bytes of a row of x or W, K = 960 is four rounds of loads (two in flight at a
// time), and a 50 x 720 problem is 1170 wavefronts.  The 64 partial sums of an output meet
// through six xor-shuffles, in that order whatever the launch.  The 8 columns are two runs
// of 4: next to each other for a plain projection, half a head apart where the QKV epilogue
// rotates, so that lane ks < 16 ends up with both members of a rotation pair (row ks / 4 of
// the four, columns ks % 4 of either run).
constexpr int SKINNY_MAX_M = 64;
template <int kEpi>
__global__ void __launch_bounds__(256) linear_f32_skinny_kernel(GemmArgs a) {
    const int tid = threadIdx.x, ks = tid & 63, rg = (tid >> 6) + 4 * blockIdx.y;
    const int K = a.K;
    // W rows of the two runs, and for QKV the segment and the segment-local columns
    int base0 = blockIdx.x * 8, base1 = base0 + 4, seg = 0, col0 = base0, col1 = base1;
    bool rope = false;
    if (kEpi == EPI_QKV) {
        const int gq = a.Hq * a.D / 8, gk = a.nk * a.D / 8;
        int lt = blockIdx.x, seg_base = 0;
        if (lt >= gq + gk) {
            seg = 2;
            lt -= gq + gk;
            seg_base = (a.Hq + a.nk) * a.D;
        } else if (lt >= gq) {
            seg = 1;
            lt -= gq;
            seg_base = a.Hq * a.D;
        }
        rope = a.cos_t != nullptr && seg != 2;
        if (rope) {
            const int gph = a.D / 8;  // groups per head
            col0 = (lt / gph) * a.D + (lt % gph) * 4;
            col1 = col0 + a.D / 2;
        } else {
            col0 = lt * 8;
            col1 = col0 + 4;
        }
        base0 = seg_base + col0;
        base1 = seg_base + col1;
    }
    const float* xr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) xr[i] = (const float*)a.A + (long)min(4 * rg + i, a.M - 1) * K;
    const float* wr[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) wr[c] = (const float*)a.W + (long)min((c < 4 ? base0 : base1 - 4) + c, a.N - 1) * K;
    float acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0.f;
    if (4 * rg < a.M) {  // whole wavefronts
#pragma unroll 2
        for (int k = 4 * ks; k < K; k += 256) {
            f32x4_t xv[4], wv[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[i] = *reinterpret_cast<const f32x4_t*>(xr[i] + k);
#pragma unroll
            for (int c = 0; c < 8; ++c) wv[c] = *reinterpret_cast<const f32x4_t*>(wr[c] + k);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int c = 0; c < 8; ++c)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][c] = fmaf(xv[i][e], wv[c][e], acc[i][c]);
        }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[i][c] += __shfl_xor(acc[i][c], off, 64);
    if (ks >= 16) return;
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int cp = 0; cp < 4; ++cp)
            if (ks == i * 4 + cp) {
                lo = acc[i][cp];
                hi = acc[i][cp + 4];
            }
    const int m = 4 * rg + (ks >> 2), cp = ks & 3;
    if (m >= a.M) return;
    if (kEpi == EPI_PLAIN) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int n = (e ? base1 : base0) + cp;
            if (n >= a.N) continue;
            float y = e ? hi : lo;
            if (a.bias) y += a.bias[n];
            if (a.act != VLA_ACT_NONE) y = apply_act(y, a.act);
            if (a.col_gate) y *= a.col_gate[n];
            const long o = (long)m * a.N + n;
            if (a.out_bf16) {
                if (a.residual) y += bf2f(((const bf16_t*)a.residual)[o]);
                ((bf16_t*)a.Y)[o] = f2bf(y);
            } else {
                if (a.residual) y += ((const float*)a.residual)[o];
                ((float*)a.Y)[o] = y;
            }
        }
        return;
    }
    // QKV: bias, rotation, scatter (the MFMA kernel's epilogue, two columns per lane)
    const int b = m / a.S, sq = m % a.S;
    if (a.bias) {
        lo += a.bias[base0 + cp];
        hi += a.bias[base1 + cp];
    }
    if (rope) {
        const int half = a.D >> 1, p0 = (col0 % a.D) + cp;
        const float c = a.cos_t[(long)sq * half + p0], sn = a.sin_t[(long)sq * half + p0];
        const float x0 = lo, x1 = hi;
        lo = x0 * c - x1 * sn;
        hi = x1 * c + x0 * sn;
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const float v = e ? hi : lo;
        const int col = (e ? col1 : col0) + cp;
        if (seg == 0) {
            ((float*)a.q_out)[(long)m * (a.Hq * a.D) + col] = v;
        } else {
            const int head = col / a.D, d = col % a.D;
            if (seg == 1) ((float*)a.k_cache)[(((long)b * a.Hkv + head) * a.t_max + a.tok_offset + sq) * a.D + d] = v;
            else ((float*)a.vt_cache)[(((long)b * a.Hkv + head) * a.D + d) * a.t_max + a.tok_offset + sq] = v;
        }
    }
}

// Ternary GEMV for a handful of rows (single-token decode, M <= 32).  A workgroup owns 32
// output columns; its 8 wavefronts each take one eighth of K and multiply it with
// v_mfma_i32_32x32x32_i8 as C[n][m] = sum_k W[n][k] * A[m][k] (weight fragment as the A
// operand: one coalesced 256-byte load per 32 k; activation rows as the B operand, lanes
// past M feed zeros).  Every load of a wavefront's slice is issued before the first is
// used; the eight partial 32 x 32 int32 tiles are summed through LDS (exact) and the
// epilogue of the tiled kernels follows, with an optional bf16 residual add.
constexpr int GEMV_WAVES = 8;
template <int MAXG>  // k groups of 32 per wavefront held in registers: K <= 256 * MAXG
__global__ void __launch_bounds__(GEMV_WAVES * 64) ternary_gemv_kernel(GemmArgs a) {
    __shared__ int part[GEMV_WAVES][32][33];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 5, r = lane & 31;
    const int nb = blockIdx.x;                       // 32-column block
    const int kgroups = a.K / 32;
    const int per_wave = (kgroups + GEMV_WAVES - 1) / GEMV_WAVES;
    const int kg0 = wave * per_wave, kg1 = min(kgroups, kg0 + per_wave);
    const uint32_t* wp = (const uint32_t*)a.W + (long)nb * kgroups * 64 + lane;
    const bool row_ok = r < a.M;
    const unsigned char* ap = (const unsigned char*)a.A + (long)(row_ok ? r : 0) * a.K + g * 16;

    uint32_t wv[MAXG];
    u32x4_t av[MAXG];
#pragma unroll
    for (int i = 0; i < MAXG; ++i) {
        const int kg = min(kg0 + i, kgroups - 1);    // past the slice: a valid group, not multiplied
        wv[i] = wp[(long)kg * 64];
        av[i] = *reinterpret_cast<const u32x4_t*>(ap + kg * 32);
    }
    i32x16_t acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0;
#pragma unroll
    for (int i = 0; i < MAXG; ++i) {
        if (kg0 + i < kg1) {                         // uniform
            const uint32_t w = wv[i];
            const u32x4_t fw = {w & 0x03030303u, (w >> 2) & 0x03030303u, (w >> 4) & 0x03030303u, (w >> 6) & 0x03030303u};
            const u32x4_t z = {0u, 0u, 0u, 0u};
            Traits<int8_t>::mma(acc, fw, row_ok ? av[i] : z);
        }
    }
    // element 4j+i of lane (g, r) is C[n = 8j + 4g + i][m = r]
#pragma unroll
    for (int e = 0; e < 16; ++e) part[wave][8 * (e >> 2) + 4 * g + (e & 3)][r] = acc[e];
    __syncthreads();
    // thread -> (m, n): 512 threads cover 16 rows x 32 columns per pass, n fastest
    const int group = a.N / a.ws_num;
    for (int m = tid >> 5; m < a.M; m += GEMV_WAVES * 2) {
        const int nl = tid & 31, n = nb * 32 + nl;
        if (n >= a.N) continue;
        int v = 0;
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; ++w) v += part[w][nl][m];
        v -= 2 * a.rowsum[m];
        if (a.acc_out) a.acc_out[(long)m * a.N + n] = v;
        if (a.Y) {
            bf16_t o = f2bf((float)v / (a.s ? a.s[m] : 1.f) * a.ws[n / group]);
            if (a.residual) o = f2bf(bf2f(o) + bf2f(((const bf16_t*)a.residual)[(long)m * a.N + n]));
            ((bf16_t*)a.Y)[(long)m * a.N + n] = o;
        }
    }
}

// The same GEMV with the producer of its activations inside: A holds the bf16 rows before
// RMSNorm, and wavefront w of every workgroup normalises and quantises row w (the code of
// the stand-alone kernel, so the bits are the same) into LDS while the weight loads are in
// flight.  Saves the separate norm + quantise launch in front of each decode projection
// (bitvla.cpp's attn_norm -> QKV and sub_norm -> O pairs).  M <= GEMV_WAVES, K <= 512 NV.
//
// ROPE: the fused Q | K | V projection of one appended token per batch row, with the split,
// the NeoX rotation and the cache append of qkv_split_rope_append_kernel in the epilogue.  The
// weight rows are in "paired" order (vla_ternary_pair_rope_rows_host): inside the Q and K
// columns every 32-row block holds 16 rotation pairs, d in lanes 0-15 and d + D/2 in lanes
// 16-31, so a pair meets through one shuffle.  The projection is rounded to bf16 before the
// rotation, as the stand-alone chain stores it.
//
// GLU: A is a fused [gate | up] projection of 2 K columns and the rows are relu(gate)^2 * up
// (the FFN's sub-norm -> down projection step, bitvla_lm_cuda.cu:505-517).
constexpr int GEMV_FUSED_MAX_K = 7168;
template <int MAXG, int NV, bool ROPE, bool GLU = false>
__global__ void __launch_bounds__(GEMV_WAVES * 64) ternary_gemv_norm_kernel(GemmArgs a) {
    // int8 rows (stride K + 32 bytes: eight rows' 16-byte fragments fall on distinct banks),
    // later the partial accumulator tiles
    constexpr int KMAX = NV * 512 < GEMV_FUSED_MAX_K ? NV * 512 : GEMV_FUSED_MAX_K;
    constexpr int kPartBytes = GEMV_WAVES * 32 * 33 * 4, kRowBytes = GEMV_WAVES * (KMAX + 32);
    __shared__ __align__(16) unsigned char smem[kPartBytes > kRowBytes ? kPartBytes : kRowBytes];
    __shared__ float s_sh[GEMV_WAVES];
    __shared__ int rs_sh[GEMV_WAVES];
    int (*part)[32][33] = reinterpret_cast<int (*)[32][33]>(smem);
    // Every kernel argument the launch will need, fetched in one batch at its start: left to the compiler the ones of
    // the epilogue are requested where they are first used, a second wait for the scalar cache in the middle of a
    // launch that is one chain of dependent steps.
    asm volatile("" ::"s"(a.A), "s"(a.W), "s"(a.norm_w), "s"(a.ws), "s"(a.q_out), "s"(a.k_cache), "s"(a.vt_cache), "s"(a.cos_t),
                 "s"(a.sin_t), "s"(a.residual), "s"(a.Y), "s"(a.t_max), "s"(a.tok_offset), "s"(a.Hkv), "s"(a.D), "s"(a.K), "s"(a.N),
                 "s"(a.M));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 5, r = lane & 31;
    const int nb = blockIdx.x;
    const int kgroups = a.K / 32;
    const int per_wave = (kgroups + GEMV_WAVES - 1) / GEMV_WAVES;
    const int kg0 = wave * per_wave, kg1 = min(kgroups, kg0 + per_wave);
    const uint32_t* wp = (const uint32_t*)a.W + (long)nb * kgroups * 64 + lane;
    const int stride = a.K + 32;

    uint32_t wv[MAXG];
#pragma unroll
    for (int i = 0; i < MAXG; ++i) wv[i] = wp[(long)min(kg0 + i, kgroups - 1) * 64];
    // What the epilogue reads from memory is fetched now, behind the weight loads, instead of
    // after the last barrier where nothing is left to hide a round trip to memory.  Epilogue
    // thread -> (row em = tid / 32, column en): M <= GEMV_WAVES, so one pass covers every row.
    const int group = a.N / a.ws_num;
    const int em = tid >> 5, enl = tid & 31, en = nb * 32 + enl;
    // (no branch around any of these loads: addresses are clamped into the arrays instead, and
    // a value that is not needed is dropped -- a load under a branch is waited for at the join,
    // together with every load issued before it)
    const bool e_ok = em < a.M && en < a.N;
    const int ec = min(en, a.N - 1), emc = min(em, a.M - 1);
    const float ws_pf = a.ws[ec / group];
    bf16_t res_pf = 0;
    float cos_pf = 0.f, sin_pf = 0.f;
    if constexpr (ROPE) {
        const int pi = 16 * ((ec % a.D) >> 5) + (enl & 15);  // < D / 2 for every column
        cos_pf = a.cos_t[pi];
        sin_pf = a.sin_t[pi];
    } else {
        // without a residual: the first element of the activations, dropped in the epilogue
        const bf16_t* rp = a.residual ? (const bf16_t*)a.residual + (long)emc * a.N + ec : (const bf16_t*)a.A;
        res_pf = *rp;
    }
    if (wave < a.M) {  // uniform per wavefront
        float scale;
        int sum;
        rms_act_quant_row<NV, GLU>((const bf16_t*)a.A + (long)wave * a.K * (GLU ? 2 : 1), (const bf16_t*)a.norm_w, a.K,
                                   a.norm_eps, lane, (int8_t*)smem + wave * stride, scale, sum);
        if (lane == 0) {
            s_sh[wave] = scale;
            rs_sh[wave] = sum;
        }
    }
    __syncthreads();
    const bool row_ok = r < a.M;
    const unsigned char* ap = smem + (row_ok ? r : 0) * stride + g * 16;
    u32x4_t av[MAXG];
#pragma unroll
    for (int i = 0; i < MAXG; ++i) av[i] = *reinterpret_cast<const u32x4_t*>(ap + min(kg0 + i, kgroups - 1) * 32);
    __syncthreads();  // the rows are in registers: the partial tiles may overwrite them
    i32x16_t acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0;
#pragma unroll
    for (int i = 0; i < MAXG; ++i) {
        if (kg0 + i < kg1) {
            const uint32_t w = wv[i];
            const u32x4_t fw = {w & 0x03030303u, (w >> 2) & 0x03030303u, (w >> 4) & 0x03030303u, (w >> 6) & 0x03030303u};
            const u32x4_t z = {0u, 0u, 0u, 0u};
            Traits<int8_t>::mma(acc, fw, row_ok ? av[i] : z);
        }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) part[wave][8 * (e >> 2) + 4 * g + (e & 3)][r] = acc[e];
    __syncthreads();
    if (e_ok) {
        const int m = em, nl = enl, n = en;
        int v = 0;
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; ++w) v += part[w][nl][m];
        v -= 2 * rs_sh[m];
        bf16_t o = f2bf((float)v / s_sh[m] * ws_pf);
        if constexpr (ROPE) {  // N is a multiple of 32 here: no lane of a half-wavefront is missing
            const float own = bf2f(o);
            const float other = __shfl_xor(own, 16, 64);
            const int hh = n / a.D, r = n % a.D, half = a.D >> 1;
            if (hh < a.Hq + a.Hkv) {
                const bool lower = nl < 16;
                const int pi = 16 * (r >> 5) + (nl & 15);
                const float c = cos_pf, sn = sin_pf;
                const float x0 = lower ? own : other, x1 = lower ? other : own;
                const float lo = x0 * c - x1 * sn, hi = x1 * c + x0 * sn;
                const int d = lower ? pi : pi + half;
                const bf16_t rot = f2bf(lower ? lo : hi);
                if (hh < a.Hq) ((bf16_t*)a.q_out)[((long)m * a.Hq + hh) * a.D + d] = rot;
                else ((bf16_t*)a.k_cache)[(((long)m * a.Hkv + (hh - a.Hq)) * a.t_max + a.tok_offset) * a.D + d] = rot;
            } else {
                ((bf16_t*)a.vt_cache)[(((long)m * a.Hkv + (hh - a.Hq - a.Hkv)) * a.D + r) * (long)a.t_max + a.tok_offset] = o;
            }
        } else {
            if (a.residual) o = f2bf(bf2f(o) + bf2f(res_pf));
            ((bf16_t*)a.Y)[(long)m * a.N + n] = o;
        }
    }
}

// XCD grid xm x xn = 8 for a tile grid of m_wg x n_wg workgroup tiles of tile_cols columns:
// every L2 reads its N tiles' rows of W once and its M tiles' rows of A once per panel of N
// tiles (xcd_tile).  One panel while an XCD's rows of W fit in half of its 4 MiB L2 beside
// the streaming A and C; else panels of about 2 MiB of W.  The split with the least total,
// counting the padding of the tile grid.  Returns the grid size.
unsigned xcd_split(GemmArgs& a, int m_wg, int n_wg, double w_bytes_per_elem, int tile_cols, double a_bytes_per_elem) {
    const double bytes_a = (double)a.M * a.K * a_bytes_per_elem, bytes_w = (double)a.N * a.K * w_bytes_per_elem;
    const double tile_w = (double)tile_cols * a.K * w_bytes_per_elem, l2_panel = 2.0 * 1024 * 1024;
    const int forced = tuning().gemm_panel;  // 0 = by size, > 0 = that many tiles per panel
    double best = -1;
    for (int xm = 1; xm <= 8; xm *= 2) {
        const int xn = 8 / xm;
        const int cn = (n_wg + xn - 1) / xn, cm = (m_wg + xm - 1) / xm;
        int pn = cn;
        if (forced > 0) pn = forced < cn ? forced : cn;
        else if (cn * tile_w > l2_panel && cm >= 4) pn = tile_w >= l2_panel ? 1 : (int)(l2_panel / tile_w);
        const int panels = (cn + pn - 1) / pn;
        const long wgs = (long)cm * cn * 8;
        const double cost = (bytes_a * xn * panels + bytes_w * xm) * (double)wgs / ((double)m_wg * n_wg);
        if (best < 0 || cost < best) {
            best = cost;
            a.xm = xm;
            a.xn = xn;
            a.pn = pn;
        }
    }
    auto magic = [](int d) { return d > 1 ? (unsigned)((1ull << 32) / (unsigned)d) + 1u : 0u; };
    a.cn = (n_wg + a.xn - 1) / a.xn;
    a.cm = (m_wg + a.xm - 1) / a.xm;
    a.per_panel = a.pn * a.cm;
    a.full = a.cn / a.pn;
    a.w_last = a.cn - a.full * a.pn;
    a.xn_shift = a.xn == 1 ? 0 : a.xn == 2 ? 1 : a.xn == 4 ? 2 : 3;
    a.mg_cn = magic(a.cn);
    a.mg_pp = magic(a.per_panel);
    a.mg_pn = magic(a.pn);
    a.mg_wl = magic(a.w_last);
    const long wgs = (long)a.cm * a.cn;
    if (wgs >= 65536) return 0;  // the tile walk's divisions are exact below 2^16 workgroups per XCD
    return (unsigned)(wgs * 8);
}

template <typename T, int kEpi, int TM, int TN, int KB, int DEPTH>
void launch_cfg(GemmArgs a, hipStream_t st) {
    const unsigned grid = xcd_split(a, (a.M + 64 * TM - 1) / (64 * TM), (a.n_tiles + TN - 1) / TN, kEpi == EPI_TERNARY ? 0.25 : sizeof(T), 64 * TN,
                                    kEpi == EPI_TERNARY ? 1.0 : sizeof(T));
    gemm_kernel<T, kEpi, TM, TN, KB, DEPTH><<<grid, 256, 0, st>>>(a);
}

template <int kEpi, int TM, int TN, int KB, int NS>
void launch_dl(GemmArgs a, hipStream_t st) {
    const unsigned grid = xcd_split(a, (a.M + 64 * TM - 1) / (64 * TM), (a.n_tiles + TN - 1) / TN, 2.0, 64 * TN, 2.0);
    if constexpr (kEpi == EPI_QKV) {
        if (a.norm_eps >= 0.f && a.colsum) {
            if (a.stats_in) gemm_dl_kernel<kEpi, TM, TN, KB, NS, NORM_LAYER_PRE><<<grid, 256, 0, st>>>(a);
            else gemm_dl_kernel<kEpi, TM, TN, KB, NS, NORM_LAYER><<<grid, 256, 0, st>>>(a);
            return;
        }
    }
    if constexpr (kEpi == EPI_QKV || kEpi == EPI_GLU) {
        if (a.norm_eps >= 0.f) {
            gemm_dl_kernel<kEpi, TM, TN, KB, NS, NORM_RMS><<<grid, 256, 0, st>>>(a);
            return;
        }
    }
    gemm_dl_kernel<kEpi, TM, TN, KB, NS, NORM_NONE><<<grid, 256, 0, st>>>(a);
}

template <typename T, int kEpi>
int launch(GemmArgs a, int n_tiles, vla_stream_t stream) {
    if (a.M == 0 || n_tiles == 0) return VLA_K_OK;
    a.n_tiles = n_tiles;
    hipStream_t st = (hipStream_t)stream;
    if constexpr (std::is_same<T, float>::value && (kEpi == EPI_PLAIN || kEpi == EPI_QKV)) {
        // a few fp32 rows: the FMA kernel (VLA_GEMM_TILE pins the MFMA kernel's tiles instead)
        if (a.M <= SKINNY_MAX_M && a.K % 4 == 0 && a.norm_eps < 0.f && tuning().gemm_tile < 0 && (uintptr_t)a.A % 16 == 0 &&
            (uintptr_t)a.W % 16 == 0 && (kEpi == EPI_PLAIN || a.D % 8 == 0)) {
            linear_f32_skinny_kernel<kEpi><<<dim3((unsigned)((a.N + 7) / 8), (unsigned)((a.M + 15) / 16)), 256, 0, st>>>(a);
            return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
        }
    }
    if constexpr (std::is_same<T, bf16_t>::value && (kEpi == EPI_PLAIN || kEpi == EPI_QKV)) {
        // a few bf16 rows (one observation's suffix through a projection): 16 columns per workgroup, K split over its wavefronts
        bool rows_ok = a.M <= tuning().gemm_rows_max && a.M <= SR_MAX_ROWS && a.K % 8 == 0 && a.K >= 64 && a.K <= SR_MAX_K &&
                       tuning().gemm_tile < 0 && (uintptr_t)a.A % 16 == 0 && (uintptr_t)a.W % 16 == 0 && !(a.colsum && a.norm_eps < 0.f) &&
                       !a.stats_out && !a.stats_in;
        if (kEpi == EPI_QKV) rows_ok = rows_ok && a.D % 16 == 0 && a.N % 16 == 0;
        if (rows_ok) {
            // more 16-column tiles than CUs: two per workgroup, so that no CU gets two workgroups' worth of requests while
            // its neighbours get one (GR00T's fused Q | K | V: 288 tiles).  Up to 32 rows only (registers).
            const int n_t16 = (a.N + 15) / 16, per = ((a.K + 31) / 32 + SR_WAVES - 1) / SR_WAVES, rb = (a.M + 15) / 16;
            const bool two = n_t16 > 256 && rb <= 2 && per <= 6;
            const unsigned grid = (unsigned)(two ? (n_t16 + 1) / 2 : n_t16);
#define VLA_ROWS_K(NORM, RB, NB)                                                                                   \
    do {                                                                                                           \
        if (per <= 2) gemm_rows_bf16_kernel<kEpi, NORM, RB, 2, NB><<<grid, SR_WAVES * 64, 0, st>>>(a);              \
        else if (per <= 4) gemm_rows_bf16_kernel<kEpi, NORM, RB, 4, NB><<<grid, SR_WAVES * 64, 0, st>>>(a);         \
        else if (per <= 6) gemm_rows_bf16_kernel<kEpi, NORM, RB, 6, NB><<<grid, SR_WAVES * 64, 0, st>>>(a);         \
        else if (NB == 1) gemm_rows_bf16_kernel<kEpi, NORM, RB, 8, 1><<<grid, SR_WAVES * 64, 0, st>>>(a);           \
    } while (0)
#define VLA_ROWS(NORM)                                \
    do {                                              \
        if (two && rb <= 1) VLA_ROWS_K(NORM, 1, 2);   \
        else if (two) VLA_ROWS_K(NORM, 2, 2);         \
        else if (rb <= 1) VLA_ROWS_K(NORM, 1, 1);     \
        else if (rb == 2) VLA_ROWS_K(NORM, 2, 1);     \
        else VLA_ROWS_K(NORM, 4, 1);                  \
    } while (0)
            if (a.norm_eps < 0.f) {
                VLA_ROWS(NORM_NONE);
            } else if constexpr (kEpi == EPI_QKV) {
                if (a.colsum) VLA_ROWS(NORM_LAYER);
                else VLA_ROWS(NORM_RMS);
            } else {
                return VLA_K_ERR_SHAPE;  // the row statistics belong to the fused QKV projections
            }
#undef VLA_ROWS
#undef VLA_ROWS_K
            return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
        }
    }
    if constexpr (kEpi != EPI_TERNARY) {
        // VLA_GEMM_TILE = 0..5 pins the tile configuration and VLA_GEMM_STAGES the ring depth
        // of the direct-to-LDS kernel (tests and tuning); unset = by shape.
        int cfg = tuning().gemm_tile;
        const long m128 = (a.M + 127) / 128, m64 = (a.M + 63) / 64;
        const long wgs0 = m128 * ((n_tiles + 1) / 2), wgs2 = m128 * n_tiles, wgs4 = m64 * n_tiles;
        if (cfg < 0) {
            // Enough 128x128 tiles to occupy the chip: use them (half the LDS and L2 traffic
            // per multiply); else 128x64 tiles if those fill it; else 64x64 tiles, with
            // 256-byte K rows (half the barriers per K) while one workgroup per CU covers them.
            cfg = wgs0 >= 128 ? 0 : (wgs2 >= 150 ? 2 : (wgs4 <= 256 ? 1 : 4));
            // 128x128 tiles that leave more than a third of the CUs idle lose to 128x64 tiles
            // that cover the chip in little more than one round (pi0's fused QKV: 140 -> 280)
            if (cfg == 0 && wgs0 < 160 && wgs2 <= 288) cfg = 2;
            // Between one and one and a half rounds of 128x128 tiles, some CUs would run two
            // workgroups while the rest run one; 128x192 tiles cover the same grid in a single
            // round of 1.5x workgroups (GR00T's fused QKV: 324 -> 216 workgroups).
            const long wgs5 = m128 * ((n_tiles + 2) / 3);
            if (cfg == 0 && wgs0 > 256 && wgs0 <= 384 && wgs5 <= 256) cfg = 5;
        }
        // bf16 operands with 16-byte aligned rows and K a multiple of the MFMA depth take the
        // direct-to-LDS kernel (VLA_GEMM_DL=0 pins the register-staged one).  Its ring depth
        // trades loads in flight against LDS per workgroup: a workgroup is short-lived, so
        // what matters first is that the whole grid is resident at once (160 KiB of LDS per
        // CU, 256 CUs), and only then how far ahead each workgroup fetches.
        bool dl = false;
        if constexpr (std::is_same<T, bf16_t>::value) {
            dl = tuning().gemm_dl != 0 && a.K % 16 == 0 && ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.W % 16 == 0);
        }
        if (a.norm_eps >= 0.f && !(dl && (kEpi == EPI_QKV || kEpi == EPI_GLU))) return VLA_K_ERR_SHAPE;  // only that kernel takes the row statistics
        if (a.colsum && kEpi != EPI_QKV) return VLA_K_ERR_SHAPE;
        if (dl) {
            int ns = tuning().gemm_stages;
            const long wgs = cfg == 0 ? wgs0 : (cfg == 2 || cfg == 3 ? wgs2 : wgs4);
            switch (cfg) {
                case 5:  // 40 KiB per stage, one workgroup per CU
                    launch_dl<kEpi, 2, 3, 128, 3>(a, st);
                    break;
                case 0:  // 32 KiB per stage
                    if (ns == 0) ns = wgs <= 256 ? 3 : 2;
                    if (ns <= 2) launch_dl<kEpi, 2, 2, 128, 2>(a, st);
                    else launch_dl<kEpi, 2, 2, 128, 3>(a, st);
                    break;
                case 1:  // 32 KiB per stage
                    if (ns == 0) ns = 4;
                    if (ns <= 3) launch_dl<kEpi, 1, 1, 256, 3>(a, st);
                    else launch_dl<kEpi, 1, 1, 256, 4>(a, st);
                    break;
                case 2:  // 24 KiB per stage
                    if (ns == 0) ns = wgs <= 256 ? 4 : (wgs <= 512 ? 3 : 2);
                    if (ns <= 2) launch_dl<kEpi, 2, 1, 128, 2>(a, st);
                    else if (ns == 3) launch_dl<kEpi, 2, 1, 128, 3>(a, st);
                    else launch_dl<kEpi, 2, 1, 128, 4>(a, st);
                    break;
                case 3:  // 24 KiB per stage
                    if (ns == 0) ns = wgs <= 256 ? 4 : 3;
                    if (ns <= 3) launch_dl<kEpi, 1, 2, 128, 3>(a, st);
                    else launch_dl<kEpi, 1, 2, 128, 4>(a, st);
                    break;
                default:  // 16 KiB per stage
                    if (ns == 0) ns = wgs <= 512 ? 4 : 3;
                    if (ns <= 3) launch_dl<kEpi, 1, 1, 128, 3>(a, st);
                    else launch_dl<kEpi, 1, 1, 128, 4>(a, st);
                    break;
            }
            return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
        }
        switch (cfg) {
            case 0: launch_cfg<T, kEpi, 2, 2, 128, 3>(a, st); break;
            case 1: launch_cfg<T, kEpi, 1, 1, 256, 4>(a, st); break;
            case 2: launch_cfg<T, kEpi, 2, 1, 128, 4>(a, st); break;
            case 3: launch_cfg<T, kEpi, 1, 2, 128, 4>(a, st); break;
            case 5: launch_cfg<T, kEpi, 2, 2, 128, 3>(a, st); break;  // the register-staged kernel has no 192-column tile
            default: launch_cfg<T, kEpi, 1, 1, 128, 6>(a, st); break;
        }
    } else {
        // VLA_TERNARY_TILE = 64 | 128 | 256 pins a tile of the 32x32x32 kernels, 16 the 16x16x64 kernel (tests and tuning); unset = by shape.
        const int force = tuning().ternary_tile;
        // Enough 128 x 256 tiles for half the chip: the large-M kernel, two workgroups per
        // CU (measured faster than one 256 x 256 workgroup: fewer wavefronts per barrier).
        const int n256 = (a.N + 255) / 256;
        const long wg128 = (long)((a.M + 127) / 128) * n256;
        const int gemv_groups = (a.K / 32 + GEMV_WAVES - 1) / GEMV_WAVES;  // k groups per wavefront
        // The 16x16x64 kernel addresses both operands with 32-bit byte offsets, writes 8-column vectors and keeps one
        // weight scale per 32-column block; anything else stays with the 32x32x32 kernels.
        const int ws_group = a.N / (a.ws_num > 0 ? a.ws_num : 1);
        const bool x16_ok = a.N % 8 == 0 && (a.Y == nullptr || ws_group % 32 == 0) && (long)a.M * a.K < (1l << 32) &&
                            (long)((a.N + 31) / 32) * a.K * 8 < (1l << 32) && ((uintptr_t)a.A % 16 == 0) && a.K % 16 == 0;
        if (force == 0 && a.M <= 32 && gemv_groups <= 28) {
            const unsigned grid = (unsigned)((a.N + 31) / 32);
            if (gemv_groups <= 10) ternary_gemv_kernel<10><<<grid, GEMV_WAVES * 64, 0, st>>>(a);
            else ternary_gemv_kernel<28><<<grid, GEMV_WAVES * 64, 0, st>>>(a);
        } else if (force == 256) {
            const unsigned grid = (unsigned)(((((a.M + 255) / 256) + 7) & ~7) * n256);
            ternary_gemm_big_kernel<4><<<grid, 512, 0, st>>>(a);
        } else if (x16_ok && (force == 16 || (force == 0 && wg128 >= 128))) {
            // the 16x16x64 kernel: 128 x 256 tiles, two workgroups per CU
            const unsigned grid = (unsigned)(((((a.M + 127) / 128) + 7) & ~7) * n256);
            ternary_gemm_x16_kernel<<<grid, 256, 0, st>>>(a);
        } else if (force == 128 || (force == 0 && wg128 >= 128)) {
            const unsigned grid = (unsigned)(((((a.M + 127) / 128) + 7) & ~7) * n256);
            ternary_gemm_big_kernel<2><<<grid, 256, 0, st>>>(a);
        } else {
            launch_cfg<T, EPI_TERNARY, 1, 1, 128, 4>(a, st);
        }
    }
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

template <bool ROPE, bool GLU = false>
int launch_gemv_norm(const GemmArgs& a, vla_stream_t stream) {
    const unsigned grid = (unsigned)((a.N + 31) / 32);
    const int groups = (a.K / 32 + GEMV_WAVES - 1) / GEMV_WAVES, nvec = a.K / 8;
    hipStream_t st = (hipStream_t)stream;
#define VLA_GEMV_NORM(G, NV) ternary_gemv_norm_kernel<G, NV, ROPE, GLU><<<grid, GEMV_WAVES * 64, 0, st>>>(a)
    if (groups <= 10) {
        if (nvec <= 128) VLA_GEMV_NORM(10, 2);
        else if (nvec <= 256) VLA_GEMV_NORM(10, 4);
        else VLA_GEMV_NORM(10, 8);
    } else if (groups <= 16) {
        VLA_GEMV_NORM(16, 8);
    } else {
        if constexpr (ROPE) return VLA_K_ERR_SHAPE;  // the QKV projection's K is the model width, never that long
        else VLA_GEMV_NORM(28, 16);
    }
#undef VLA_GEMV_NORM
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int vla_linear(const void* x, const void* W, const float* bias, const void* residual, void* y, int dtype,
               int out_dtype, int M, int N, int K, vla_stream_t stream) {
    if (!x || !W || !y || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out_dtype != VLA_DT_F32 && out_dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    GemmArgs a = {};
    a.norm_eps = -1.f;
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

static int qkv_rope_impl(const void* x, const void* W, const float* bias, int dtype, int M, int K, int S, int n_q_heads,
                         int n_kv_heads, int has_k, int has_v, int head_dim, const float* cos_tab, const float* sin_tab,
                         void* q_out, void* k_cache, void* vt_cache, int t_max, int tok_offset, float rms_eps,
                         vla_stream_t stream, const float* colsum = nullptr, const float* stats_in = nullptr, int n_stat = 0) {
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
    a.norm_eps = rms_eps;
    a.colsum = colsum;
    a.stats_in = stats_in;
    a.n_stat = n_stat;
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

int vla_attn_qkv_rope(const void* x, const void* W, const float* bias, int dtype, int M, int K, int S, int n_q_heads,
                      int n_kv_heads, int has_k, int has_v, int head_dim, const float* cos_tab, const float* sin_tab,
                      void* q_out, void* k_cache, void* vt_cache, int t_max, int tok_offset, vla_stream_t stream) {
    return qkv_rope_impl(x, W, bias, dtype, M, K, S, n_q_heads, n_kv_heads, has_k, has_v, head_dim, cos_tab, sin_tab, q_out,
                         k_cache, vt_cache, t_max, tok_offset, -1.f, stream);
}

int vla_linear_act(const void* x, const void* W, const float* bias, const void* residual, void* y, int dtype,
                   int out_dtype, int M, int N, int K, int act, vla_stream_t stream) {
    if (!x || !W || !y || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out_dtype != VLA_DT_F32 && out_dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    if (act < VLA_ACT_NONE || act > VLA_ACT_RELU) return VLA_K_ERR_ARG;
    GemmArgs a = {};
    a.norm_eps = -1.f;
    a.A = x; a.W = W; a.bias = bias; a.M = M; a.N = N; a.K = K;
    a.residual = residual; a.Y = y; a.out_bf16 = (out_dtype == VLA_DT_BF16); a.act = act;
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

int vla_linear_gated(const void* x, const void* W, const float* bias, const float* col_gate, const void* residual, void* y,
                     int dtype, int out_dtype, int M, int N, int K, vla_stream_t stream) {
    if (!x || !W || !y || !col_gate || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out_dtype != VLA_DT_F32 && out_dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    GemmArgs a = {};
    a.norm_eps = -1.f;
    a.A = x; a.W = W; a.bias = bias; a.M = M; a.N = N; a.K = K;
    a.residual = residual; a.Y = y; a.out_bf16 = (out_dtype == VLA_DT_BF16); a.col_gate = col_gate;
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

int vla_glu_linear(const void* x, const void* W_gate_up, const float* bias, void* y, int dtype, int out_dtype, int M, int I,
                   int K, int act, float rms_eps, vla_stream_t stream) {
    if (!x || !W_gate_up || !y || M < 0 || I <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out_dtype != VLA_DT_F32 && out_dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    if (act < VLA_ACT_NONE || act > VLA_ACT_RELU) return VLA_K_ERR_ARG;
    if (I % 32) return VLA_K_ERR_SHAPE;  // a tile pairs 32 gate columns with their 32 up columns
    GemmArgs a = {};
    a.norm_eps = rms_eps >= 0.f ? rms_eps : -1.f;
    a.A = x; a.W = W_gate_up; a.bias = bias; a.M = M; a.N = 2 * I; a.K = K;
    a.Y = y; a.out_bf16 = (out_dtype == VLA_DT_BF16); a.act = act;
    const int nt = I / 32;
    if (dtype == VLA_DT_BF16) {
        if (K % 8) return VLA_K_ERR_SHAPE;
        return launch<bf16_t, EPI_GLU>(a, nt, stream);
    }
    if (dtype == VLA_DT_F32) {
        if (K % 4) return VLA_K_ERR_SHAPE;
        return launch<float, EPI_GLU>(a, nt, stream);
    }
    return VLA_K_ERR_ARG;
}

int vla_rmsnorm_attn_qkv_rope(const void* x, const void* W_folded, const float* bias, int dtype, int M, int K, int S,
                              int n_q_heads, int n_kv_heads, int has_k, int has_v, int head_dim, const float* cos_tab,
                              const float* sin_tab, void* q_out, void* k_cache, void* vt_cache, int t_max, int tok_offset,
                              float rms_eps, vla_stream_t stream) {
    if (rms_eps < 0.f) return VLA_K_ERR_ARG;
    if (dtype != VLA_DT_BF16) return VLA_K_ERR_SHAPE;
    return qkv_rope_impl(x, W_folded, bias, dtype, M, K, S, n_q_heads, n_kv_heads, has_k, has_v, head_dim, cos_tab, sin_tab,
                         q_out, k_cache, vt_cache, t_max, tok_offset, rms_eps, stream);
}

int vla_layernorm_attn_qkv_rope(const void* x, const void* W_folded, const float* colsum, const float* bias, int dtype, int M,
                                int K, int S, int n_q_heads, int n_kv_heads, int has_k, int has_v, int head_dim,
                                const float* cos_tab, const float* sin_tab, void* q_out, void* k_cache, void* vt_cache,
                                int t_max, int tok_offset, float ln_eps, vla_stream_t stream) {
    if (ln_eps < 0.f || !colsum) return VLA_K_ERR_ARG;
    if (dtype != VLA_DT_BF16) return VLA_K_ERR_SHAPE;
    return qkv_rope_impl(x, W_folded, bias, dtype, M, K, S, n_q_heads, n_kv_heads, has_k, has_v, head_dim, cos_tab, sin_tab,
                         q_out, k_cache, vt_cache, t_max, tok_offset, ln_eps, stream, colsum);
}

int vla_layernorm_attn_qkv_rope_stats(const void* x, const void* W_folded, const float* colsum, const float* bias,
                                      const float* row_stats, int n_stat_tiles, int dtype, int M, int K, int S, int n_q_heads,
                                      int n_kv_heads, int has_k, int has_v, int head_dim, const float* cos_tab,
                                      const float* sin_tab, void* q_out, void* k_cache, void* vt_cache, int t_max,
                                      int tok_offset, float ln_eps, vla_stream_t stream) {
    if (ln_eps < 0.f || !colsum || !row_stats) return VLA_K_ERR_ARG;
    if (dtype != VLA_DT_BF16 || n_stat_tiles < 1 || n_stat_tiles > STAT_MAX_TILES || K != n_stat_tiles * BN) return VLA_K_ERR_SHAPE;
    return qkv_rope_impl(x, W_folded, bias, dtype, M, K, S, n_q_heads, n_kv_heads, has_k, has_v, head_dim, cos_tab, sin_tab,
                         q_out, k_cache, vt_cache, t_max, tok_offset, ln_eps, stream, colsum, row_stats, n_stat_tiles);
}

int vla_linear_row_stats(const void* x, const void* W, const float* bias, const void* residual, void* y, float* row_stats,
                         int dtype, int M, int N, int K, vla_stream_t stream) {
    if (!x || !W || !y || !row_stats || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (dtype != VLA_DT_BF16 || N % BN || K % 8) return VLA_K_ERR_SHAPE;
    GemmArgs a = {};
    a.norm_eps = -1.f;
    a.A = x; a.W = W; a.bias = bias; a.M = M; a.N = N; a.K = K;
    a.residual = residual; a.Y = y; a.out_bf16 = 1;
    a.stats_out = row_stats;
    return launch<bf16_t, EPI_PLAIN>(a, N / BN, stream);
}

int vla_fold_norm_weight_host(const void* W, const void* g, int dtype, int N, int K, void* W_out) {
    if (!W || !g || !W_out || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (dtype == VLA_DT_F32) {
        for (long n = 0; n < N; ++n)
            for (int k = 0; k < K; ++k) ((float*)W_out)[n * K + k] = ((const float*)W)[n * K + k] * ((const float*)g)[k];
        return VLA_K_OK;
    }
    if (dtype == VLA_DT_BF16) {
        const uint16_t* w = (const uint16_t*)W;
        const uint16_t* gg = (const uint16_t*)g;
        for (long n = 0; n < N; ++n)
            for (int k = 0; k < K; ++k) {
                uint32_t wb = (uint32_t)w[n * K + k] << 16, gb = (uint32_t)gg[k] << 16;
                float wf, gf;
                memcpy(&wf, &wb, 4);
                memcpy(&gf, &gb, 4);
                const float p = wf * gf;
                uint32_t pb;
                memcpy(&pb, &p, 4);
                if ((pb & 0x7fffffffu) > 0x7f800000u) pb |= 0x00400000u;                // NaN stays NaN
                else pb += 0x7fffu + ((pb >> 16) & 1u);                                  // round to nearest even
                ((uint16_t*)W_out)[n * K + k] = (uint16_t)(pb >> 16);
            }
        return VLA_K_OK;
    }
    return VLA_K_ERR_ARG;
}

int vla_fold_adaln_weight_host(const void* W, const float* bias, const float* scale, const float* shift, int N, int K,
                               void* W_out, float* colsum_out, float* bias_out) {
    if (!W || !scale || !shift || !W_out || !colsum_out || !bias_out || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    const uint16_t* w = (const uint16_t*)W;
    for (long n = 0; n < N; ++n) {
        double cs = 0.0, bs = bias ? (double)bias[n] : 0.0;
        for (int k = 0; k < K; ++k) {
            const uint32_t wb = (uint32_t)w[n * K + k] << 16;
            float wf;
            memcpy(&wf, &wb, 4);
            bs += (double)wf * (double)shift[k];
            const float p = wf * (1.0f + scale[k]);
            uint32_t pb;
            memcpy(&pb, &p, 4);
            if ((pb & 0x7fffffffu) > 0x7f800000u) pb |= 0x00400000u;  // NaN stays NaN
            else pb += 0x7fffu + ((pb >> 16) & 1u);                    // round to nearest even
            pb &= 0xffff0000u;
            ((uint16_t*)W_out)[n * K + k] = (uint16_t)(pb >> 16);
            float rf;
            memcpy(&rf, &pb, 4);
            cs += (double)rf;
        }
        colsum_out[n] = (float)cs;
        bias_out[n] = (float)bs;
    }
    return VLA_K_OK;
}

int vla_ternary_gemm(const int8_t* A, const uint32_t* W_packed, uint16_t* out, int32_t* acc_out, const float* s,
                     const int32_t* rowsum, const float* ws, int ws_num, int M, int N, int K, vla_stream_t stream) {
    if (!A || !W_packed || !rowsum || (!out && !acc_out) || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (out && (!s || !ws || ws_num <= 0)) return VLA_K_ERR_ARG;
    if (K % 128 || (out && N % ws_num)) return VLA_K_ERR_SHAPE;
    GemmArgs a = {};
    a.norm_eps = -1.f;
    a.A = A; a.W = W_packed; a.M = M; a.N = N; a.K = K;
    a.Y = out; a.acc_out = acc_out; a.s = s; a.rowsum = rowsum; a.ws = ws; a.ws_num = ws_num > 0 ? ws_num : 1;
    return launch<int8_t, EPI_TERNARY>(a, (N + BN - 1) / BN, stream);
}

int vla_ternary_gemm_add(const int8_t* A, const uint32_t* W_packed, uint16_t* out, const uint16_t* residual, const float* s,
                         const int32_t* rowsum, const float* ws, int ws_num, int M, int N, int K, vla_stream_t stream) {
    if (!A || !W_packed || !rowsum || !out || !s || !ws || ws_num <= 0 || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (K % 128 || N % ws_num) return VLA_K_ERR_SHAPE;
    GemmArgs a = {};
    a.norm_eps = -1.f;
    a.A = A; a.W = W_packed; a.M = M; a.N = N; a.K = K;
    a.Y = out; a.residual = residual; a.s = s; a.rowsum = rowsum; a.ws = ws; a.ws_num = ws_num;
    return launch<int8_t, EPI_TERNARY>(a, (N + BN - 1) / BN, stream);
}

int vla_rmsnorm_ternary_gemv(const uint16_t* x, const uint16_t* norm_w, float eps, const uint32_t* W_packed, uint16_t* out,
                             const uint16_t* residual, const float* ws, int ws_num, int M, int N, int K,
                             vla_stream_t stream) {
    if (!x || !W_packed || !out || !ws || ws_num <= 0 || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M > GEMV_WAVES || K > GEMV_FUSED_MAX_K || K % 128 || N % ws_num || (((uintptr_t)x) & 15)) return VLA_K_ERR_SHAPE;
    if (M == 0) return VLA_K_OK;
    GemmArgs a = {};
    a.A = x; a.norm_w = norm_w; a.norm_eps = eps; a.W = W_packed; a.M = M; a.N = N; a.K = K;
    a.Y = out; a.residual = residual; a.ws = ws; a.ws_num = ws_num;
    return launch_gemv_norm<false>(a, stream);
}

int vla_sqrelu_rmsnorm_ternary_gemv(const uint16_t* gate_up, const uint16_t* norm_w, float eps, const uint32_t* W_packed,
                                    uint16_t* out, const uint16_t* residual, const float* ws, int ws_num, int M, int N, int K,
                                    vla_stream_t stream) {
    if (!gate_up || !W_packed || !out || !ws || ws_num <= 0 || M < 0 || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M > GEMV_WAVES || K > GEMV_FUSED_MAX_K || K % 128 || N % ws_num || (((uintptr_t)gate_up) & 15)) return VLA_K_ERR_SHAPE;
    if (M == 0) return VLA_K_OK;
    GemmArgs a = {};
    a.A = gate_up; a.norm_w = norm_w; a.norm_eps = eps; a.W = W_packed; a.M = M; a.N = N; a.K = K;
    a.Y = out; a.residual = residual; a.ws = ws; a.ws_num = ws_num;
    return launch_gemv_norm<false, true>(a, stream);
}

int vla_rmsnorm_ternary_gemv_rope_append(const uint16_t* x, const uint16_t* norm_w, float eps, const uint32_t* W_paired,
                                         const float* ws, int ws_num, const float* cos_row, const float* sin_row,
                                         uint16_t* q_out, uint16_t* k_cache, uint16_t* vt_cache, int batch, int n_q_heads,
                                         int n_kv_heads, int head_dim, int K, int t_max, int tok_offset,
                                         vla_stream_t stream) {
    if (!x || !W_paired || !ws || !cos_row || !sin_row || !q_out || !k_cache || !vt_cache || ws_num <= 0 || batch < 0 ||
        n_q_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || K <= 0)
        return VLA_K_ERR_ARG;
    const int N = (n_q_heads + 2 * n_kv_heads) * head_dim;
    if (batch > GEMV_WAVES || K > 4096 || K % 128 || head_dim % 32 || N % ws_num || (N / ws_num) % head_dim ||
        tok_offset < 0 || tok_offset >= t_max || (((uintptr_t)x) & 15))
        return VLA_K_ERR_SHAPE;
    if (batch == 0) return VLA_K_OK;
    GemmArgs a = {};
    a.A = x; a.norm_w = norm_w; a.norm_eps = eps; a.W = W_paired; a.M = batch; a.N = N; a.K = K;
    a.ws = ws; a.ws_num = ws_num; a.cos_t = cos_row; a.sin_t = sin_row;
    a.q_out = q_out; a.k_cache = k_cache; a.vt_cache = vt_cache;
    a.Hq = n_q_heads; a.Hkv = n_kv_heads; a.D = head_dim; a.t_max = t_max; a.tok_offset = tok_offset; a.S = 1;
    return launch_gemv_norm<true>(a, stream);
}

int vla_ternary_pair_rope_rows_host(const uint32_t* packed, int n_q_heads, int n_kv_heads, int head_dim, int K,
                                    uint32_t* paired) {
    if (!packed || !paired || packed == paired || n_q_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || K <= 0)
        return VLA_K_ERR_ARG;
    if (head_dim % 32 || K % 32) return VLA_K_ERR_SHAPE;
    const int half = head_dim / 2, kw = K / 16;
    const long rope_rows = (long)(n_q_heads + n_kv_heads) * head_dim, N = rope_rows + (long)n_kv_heads * head_dim;
    for (long n = 0; n < N; ++n) {
        long src = n;
        if (n < rope_rows) {
            const int r = (int)(n % head_dim), nl = r % 32;
            src = n - r + (nl < 16 ? 16 * (r / 32) + nl : half + 16 * (r / 32) + (nl - 16));
        }
        for (int w = 0; w < kw; ++w) paired[tern_word_index(n, w, K)] = packed[tern_word_index(src, w, K)];
    }
    return VLA_K_OK;
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
    // the reference's signature carries no row sums: they go into a block the library keeps
    // for this stream (calls on one stream are ordered, other streams have their own block)
    int32_t* rowsum = (int32_t*)stream_scratch(SCRATCH_ROWSUM, (hipStream_t)stream, (size_t)M * sizeof(int32_t));
    if (!rowsum) return VLA_K_ERR_LAUNCH;
    rowsum_i8_kernel<<<M, 64, 0, (hipStream_t)stream>>>(A, rowsum, K);
    return vla_ternary_gemm(A, (const uint32_t*)B, out, nullptr, s, rowsum, ws, bitvla_ws_num(N, K), M, N, K, stream);
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

long vla_ternary_packed_words(int N, int K) { return (long)((N + 31) / 32 * 32) * (K / 16); }

static void tern_fill_pad_rows(int N, int K, uint32_t* packed) {
    for (long n = N; n < (N + 31) / 32 * 32; ++n)
        for (int w = 0; w < K / 16; ++w) packed[tern_word_index(n, w, K)] = 0xAAAAAAAAu;  // code 2 = weight 0
}

int vla_ternary_pack_host(const int8_t* ternary, int N, int K, uint32_t* packed) {
    if (!ternary || !packed || N <= 0 || K <= 0) return VLA_K_ERR_ARG;
    if (K % 32) return VLA_K_ERR_SHAPE;
    const int kw = K / 16;
    for (long n = 0; n < N; ++n)
        for (int w = 0; w < kw; ++w) {
            uint32_t word = 0;
            for (int v = 0; v < 16; ++v) {
                const int t = ternary[n * K + w * 16 + v];
                if (t < -2 || t > 1) return VLA_K_ERR_ARG;
                word |= (uint32_t)((t + 2) & 3) << (8 * (v & 3) + 2 * (v >> 2));
            }
            packed[tern_word_index(n, w, K)] = word;
        }
    tern_fill_pad_rows(N, K, packed);
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
            packed[tern_word_index(n, w, K)] = src[slot];
        }
    tern_fill_pad_rows(N, K, packed);
    return VLA_K_OK;
}

}  // extern "C"
