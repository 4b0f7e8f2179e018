// Masked prefix+suffix attention over the resident KV cache (gfx950).
//
// out = softmax(scale * Q K^T + mask) V, one pass over the keys with an online
// softmax, fp32 scores / statistics / accumulation in every mode (the
// reference's precision split, src/act_dtype.h:29-35).
//
// Work decomposition.  A workgroup owns one (batch, kv head) pair, a group of
// 32-row tiles of that head's query rows and (optionally) a slice of the keys.
// The rows of all g = Hq/Hkv query heads sharing the kv head are flattened
// (row = head_in_group * S + s), so a K/V tile staged in LDS is read once per
// query-head group (GQA / MQA sharing) instead of being copied per query head
// as bitvla_repeat_kv_bf16 does (src/kernels/bitvla/bitvla_lm_cuda.cu:181-190).
// Each 64-lane wavefront owns one row tile.
//
// Memory.  The cache layout makes both tiles plain block copies: K [t][D] of one
// head is contiguous, V^T [D][t] has the keys innermost.  A tile's 16-byte
// global loads are all issued before any is consumed, and the next tile's loads
// are in flight while the current tile is multiplied.  Workgroups that share a
// (batch, kv head) get linear ids equal modulo 8, so they land on the same XCD
// and share its L2.
//
// MFMA formulation (transposed, so softmax statistics are per lane):
//   S^T[key][row] = K . Q^T     A = K tile rows (lane r <-> key), B = Q rows
//   O^T[d][row]  += V^T . P^T   A = V^T rows (lane r <-> d),      B = P^T
// The 32x32 accumulator gives lane (g, r) the 16 score rows 8j+4g+i of query row r,
// so row max / sum are 15 in-lane ops plus one exchange with lane r+32, and the
// probabilities are already in B-operand position for the second product.  Which key
// sits in score row x is free (it is just the K row a lane fetches): row 8j+4g+i holds
// key 16(j/2) + 8g + 4(j%2) + i of the 32-key block, so that the 8 probabilities a lane
// feeds to one output MFMA belong to 8 consecutive keys and its V^T fragment is a single
// 16-byte run.  No score matrix is ever written
// (the reference's explicit path writes and re-reads Hq*S*T scores).
//
// Few query rows (single-token decode, batch 1): the keys are split across
// workgroups, each writes an unnormalised partial (max, sum, O) and a second
// kernel merges them.

#include <math.h>
#include <stdlib.h>

#include <mutex>
#include <type_traits>

#include "common.h"
#include "vla_kernels.h"

namespace {

using namespace vk;

constexpr float RESCALE_LOG2 = 8.0f;  // see the online softmax
constexpr int SPLIT_KEYS = 64;  // granularity of key slices; keys per LDS tile of narrow heads

struct AttnArgs {
    const void* q;
    const void* k_cache;
    const void* vt_cache;
    void* out;
    int batch, S, Hq, Hkv, t_max, n_keys;
    float scale;
    int mask_kind, n_prefix, pad_start, pad_end;
    const float* mask;
    int n_groups, n_split, tiles_per_split, r_pad, p2;
    int n_rblocks;  // direct kernel: 32-row blocks per (batch, kv head)
    int n_slices;   // LDS kernel, direct-to-LDS variant: key slices (wavefronts) per row tile
    float* part_o;   // [pair][split][r_pad][D] fp32 unnormalised, or fp16 normalised (part_half); merged in the launch: [pair][r_pad][split][D]
    float* part_ml;  // [pair][split][r_pad][2]; merged in the launch: [pair][r_pad][split][2]
    int part_half;   // partial outputs stored as o / l in fp16 (half the bytes; wide heads)
    int* arrive;     // decode kernel: one counter per pair; the slice that arrives last merges (zero between launches)
    // divisors of the kernels' index arithmetic (set_divisors, at the launch): S, Hkv, n_split, n_groups n_split and
    // eight times that; grp = Hq / Hkv
    DivC dS, dHkv, dns, dGS, d8GS;
    int grp;
};
// Called once the slicing of a launch is fixed.  max_id: the largest workgroup index of the launch.
inline void set_divisors(AttnArgs& a, long max_id) {
    a.grp = a.Hq / a.Hkv;
    const long R = (long)a.grp * a.S, GS = (long)a.n_groups * a.n_split;
    const long mx = max_id > R ? max_id : R;
    a.dS = make_divc(a.S, mx);
    a.dHkv = make_divc(a.Hkv, mx);
    a.dns = make_divc(a.n_split, mx);
    a.dGS = make_divc(GS, mx);
    a.d8GS = make_divc(8 * GS, mx);
}

// Key (within a 32-key block) held by score row x = 8j + 4h + i: 16(j/2) + 8h + 4(j%2) + i.
__device__ __forceinline__ int key_of_score_row(int x) {
    return 16 * (x >> 4) + 8 * ((x >> 2) & 1) + 4 * ((x >> 3) & 1) + (x & 3);
}
// Key of accumulator element e (= 4j + i) of a lane in half g.
__device__ __forceinline__ int key_of_element(int e, int g) { return 16 * (e >> 3) + 8 * g + 4 * ((e >> 2) & 1) + (e & 3); }

// One output row from its key slices' partials, by one wavefront: the slices' (max, sum) pairs
// are read by every lane (one address per slice: a broadcast), the weights 2^(m_slice - m) are
// formed once, and each lane combines four consecutive elements per 256-element stretch.
// prow0 = the row's index in slice 0; slice sp lies sp * r_pad rows further.  HALF: the
// partial outputs are fp16 and normalised by their slice's sum.
template <typename T, bool HALF>
__device__ __forceinline__ void merge_row(const float* __restrict__ part_o, const float* __restrict__ part_ml, T* __restrict__ orow,
                                          long prow0, int n_split, int r_pad, int D, int lane) {
    float m = -INFINITY;
    for (int sp = 0; sp < n_split; ++sp) m = fmaxf(m, part_ml[(prow0 + (long)sp * r_pad) * 2]);
    for (int d0 = lane * 4; d0 < D; d0 += 256) {
        float l = 0.f;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (m > -INFINITY) {
            for (int sp = 0; sp < n_split; ++sp) {
                const long prow = prow0 + (long)sp * r_pad;
                const float w = exp2f(part_ml[prow * 2] - m);
                if (HALF) {
                    typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
                    const float wl = part_ml[prow * 2 + 1] * w;
                    l += wl;
                    const h4_t po = *reinterpret_cast<const h4_t*>(reinterpret_cast<const _Float16*>(part_o) + prow * D + d0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] += (float)po[e] * wl;
                } else {
                    l += part_ml[prow * 2 + 1] * w;
                    const f32x4_t po = *reinterpret_cast<const f32x4_t*>(part_o + prow * D + d0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] += po[e] * w;
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) Elem<T>::store(orow + d0 + e, l > 0.f ? acc[e] / l : 0.f);
    }
}

// The same for a slice count known at compile time: every load of the row -- the slices' (max, sum) pairs and their
// partial outputs -- is requested before the first is used, one trip to memory instead of one per slice (the loop above
// waits for each slice's loads inside its iteration).  Same arithmetic in the same order.
template <typename T, bool HALF, int NS>
__device__ __forceinline__ void merge_row_static(const float* __restrict__ part_o, const float* __restrict__ part_ml, T* __restrict__ orow,
                                                 long prow0, int r_pad, int D, int lane) {
    typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
    f32x2_t ml[NS];
#pragma unroll
    for (int sp = 0; sp < NS; ++sp) ml[sp] = *reinterpret_cast<const f32x2_t*>(part_ml + (prow0 + (long)sp * r_pad) * 2);
    for (int d0 = lane * 4; d0 < D; d0 += 256) {
        h4_t ph[NS];
        f32x4_t pf[NS];
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) {
            const long prow = prow0 + (long)sp * r_pad;
            if (HALF) ph[sp] = *reinterpret_cast<const h4_t*>(reinterpret_cast<const _Float16*>(part_o) + prow * D + d0);
            else pf[sp] = *reinterpret_cast<const f32x4_t*>(part_o + prow * D + d0);
        }
        float m = -INFINITY;
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) m = fmaxf(m, ml[sp][0]);
        const float mm = m > -INFINITY ? m : 0.f;  // nothing visible in any slice: every weight 2^-inf = 0
        float l = 0.f;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) {
            const float w = exp2f(ml[sp][0] - mm);
            if (HALF) {
                const float wl = ml[sp][1] * w;
                l += wl;
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += (float)ph[sp][e] * wl;
            } else {
                l += ml[sp][1] * w;
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += pf[sp][e] * w;
            }
        }
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = l > 0.f ? acc[e] / l : 0.f;
        if constexpr (sizeof(T) == 2) *reinterpret_cast<u32x2_t*>(orow + d0) = u32x2_t{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3])};
        else *reinterpret_cast<f32x4_t*>(orow + d0) = f32x4_t{v[0], v[1], v[2], v[3]};
    }
}

template <typename T> struct AT;
template <> struct AT<bf16_t> {
    static constexpr int EB = 2;
    static constexpr int CE = 16;  // k elements per MFMA group
    __device__ static __forceinline__ void mma(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                      acc, 0, 0, 0);
    }
    __device__ static __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
};
template <> struct AT<float> {
    static constexpr int EB = 4;
    static constexpr int CE = 8;
    __device__ static __forceinline__ void mma(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
        const f32x4_t fa = __builtin_bit_cast(f32x4_t, a), fb = __builtin_bit_cast(f32x4_t, b);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[t], fb[t], acc, 0, 0, 0);
    }
    __device__ static __forceinline__ float fexp2(float x) { return exp2f(x); }
};

// NL > 0: producer / consumer wavefronts.  Wavefronts NW .. NW+NL-1 only move data: they
// keep LOAD_AHEAD key tiles of global loads in flight in their own registers (they need
// none for arithmetic) and store them into a double-buffered LDS tile pair; the NW compute
// wavefronts never touch global memory inside the loop.  One barrier per tile.  Used for
// wide heads, whose accumulators and query fragments leave the compute wavefronts no
// registers to prefetch with, so that memory latency would be exposed once per tile.
//
// NSL > 0 selects the direct-to-LDS variant (bf16, 128- or 256-byte K rows): tiles go from
// the cache straight into an unpadded, swizzled LDS ring (16-byte piece c of row `row` at
// piece position c ^ swz(row), swz = (row >> 1) & 7 for 128-byte rows, row & 15 for 256-byte
// rows), one barrier per step and no staging registers or LDS stores.  The workgroup then
// has NW x NSL wavefronts: NSL key slices per row tile, slice sl taking tiles sl, sl + NSL,
// ... of the workgroup's key range; a step multiplies NSL tiles at once and the slices'
// partial (max, sum, output) meet in LDS at the end.  RS step slots form the ring.
constexpr int WIDE_FB = 4;  // LDS fragments read ahead of their MFMAs, 256-wide heads (8 spills registers)

template <typename T, int D, int NW, bool P2, int NL, int NSL = 0, int RS = 1>
__global__ void __launch_bounds__((NW * (NSL > 0 ? NSL : 1) + NL) * 64, (D * sizeof(T) <= 128) ? 2 : 1) attn_kernel(AttnArgs a) {
    typedef AT<T> A;
    constexpr int EB = A::EB, CE = A::CE;
    constexpr bool DLOAD = NSL > 0;
    static_assert(!DLOAD || (NL == 0 && EB == 2 && (D == 64 || D == 128)), "direct-to-LDS tiles: bf16, 128/256-byte K rows");
    // Keys per staged tile: 64, or 32 for wide heads (rows of 512 bytes and more), whose
    // accumulators and query fragments leave too few registers to stage 64 keys.
    constexpr int TK = (D * EB >= 512) ? 32 : SPLIT_KEYS;
    constexpr int NKB = TK / 32;
    constexpr int DP = (D + 31) / 32 * 32;  // head_dim padded to whole 32-row output blocks
    constexpr int NQ = D / CE;              // MFMA groups along head_dim
    constexpr int NDB = DP / 32;            // 32-row blocks of O^T
    constexpr int KS = D * EB + 16;         // LDS stride of a K row (bytes)
    constexpr int VS = TK * EB + 16;        // LDS stride of a V^T row (bytes)
    constexpr int NT = NW * 64;
    constexpr int KV_PER_ROW = D * EB / 16;   // 16-byte vectors per K row
    constexpr int VV_PER_ROW = TK * EB / 16;  // 16-byte vectors per V^T row
    constexpr int EPV = 16 / EB;              // elements per vector
    constexpr int NVEC = TK * KV_PER_ROW;     // vectors in a K tile == vectors in a V^T tile
    constexpr int IT = (NVEC + NT - 1) / NT;  // vectors per thread per tile and operand
    constexpr bool PREFETCH = (2 * IT <= 16); // keep the next tile in registers across the multiply
    static_assert(D % CE == 0 && (D * EB) % 16 == 0, "head_dim must be whole MFMA groups and 16-byte rows");
    static_assert(NVEC == D * VV_PER_ROW, "K and V^T tiles hold the same number of vectors");

    constexpr int KROW = D * EB, VROW = TK * EB;          // unpadded row sizes of the direct-to-LDS ring
    constexpr int KTILE = TK * KROW, VTILE = DP * VROW, STAGE = KTILE + VTILE;
    constexpr int NWAVES = NW * (DLOAD ? NSL : 1);
    constexpr int XCH = (NSL > 1) ? (NSL - 1) * NW * (NDB * 16 + 2) * 64 * 4 : 0;  // slice merge buffer
    constexpr int RING = DLOAD ? (RS * NSL * STAGE > XCH ? RS * NSL * STAGE : XCH) : 16;
    __shared__ __attribute__((aligned(16))) unsigned char ldsK_buf[NL ? 2 : 1][DLOAD ? 16 : TK * KS];
    __shared__ __attribute__((aligned(16))) unsigned char ldsV_buf[NL ? 2 : 1][DLOAD ? 16 : DP * VS];
    __shared__ __attribute__((aligned(1024))) unsigned char ring[RING];
    unsigned char* ldsK = ldsK_buf[0];
    unsigned char* ldsV = ldsV_buf[0];

    // ---- XCD-aware decode of the linear workgroup id
    const int GS = a.n_groups * a.n_split;
    const int id = blockIdx.x;
    const int pair = (int)div_c(id, a.d8GS) * 8 + (id & 7);
    if (pair >= a.batch * a.Hkv) return;
    const int t_idx = (id >> 3) - (int)div_c(id >> 3, a.dGS) * GS;
    const int group = (int)div_c(t_idx, a.dns), split = t_idx - group * a.n_split;
    const int b = (int)div_c(pair, a.dHkv), hk = pair - b * a.Hkv;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 5, r = lane & 31;
    const int grp = a.grp;
    const int R = grp * a.S;
    const int rw = DLOAD ? wave % NW : wave;  // row tile of this wavefront
    const int sl = DLOAD ? wave / NW : 0;     // key slice of this wavefront
    const int row = (group * NW + rw) * 32 + r;
    const bool wave_active = rw < NW && (group * NW + rw) * 32 < R;
    const bool row_valid = rw < NW && row < R;
    const int hg = row_valid ? (int)div_c(row, a.dS) : 0;
    const int s = row_valid ? row - hg * a.S : 0;
    const int h = hk * grp + hg;

    const int k_begin = split * a.tiles_per_split * SPLIT_KEYS;
    const int k_end = min(a.n_keys, k_begin + a.tiles_per_split * SPLIT_KEYS);

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
    // Scores are kept in the base-2 exponent domain: s2 = score * scale * log2(e).
    float m_run = -INFINITY, l_run = 0.f;
    constexpr float LOG2E = 1.4426950408889634f;
    const float c2 = a.scale * LOG2E;

    const unsigned char* kbase = (const unsigned char*)a.k_cache + ((long)b * a.Hkv + hk) * a.t_max * D * EB;
    const unsigned char* vbase = (const unsigned char*)a.vt_cache + ((long)b * a.Hkv + hk) * D * (long)a.t_max * EB;

    // Per-row visibility of the generated masks, branch-free: a key is visible iff
    // key < hi and it is not inside the padded-language range of the prefix.
    int hi = a.n_keys;
    if (a.mask_kind == VLA_MASK_CAUSAL_SUFFIX) hi = min(a.n_keys, a.n_prefix + s + 1);
    else if (a.mask_kind == VLA_MASK_PI0_STATE && s == 0) hi = min(a.n_keys, a.n_prefix + 1);
    const int pad_lo = a.pad_start, pad_hi = min(a.pad_end, a.n_prefix);

    // Staging.  Full tiles are plain block copies with no bounds checks; only the last,
    // partial tile clamps K rows to a valid key and zeroes V^T elements past n_keys, so
    // that stale cache contents (possibly NaN) cannot reach the accumulators.
    constexpr bool EXACT = (NVEC % NT) == 0;
    u32x4_t kreg[IT], vreg[IT];
    auto load_k = [&](int k0) __attribute__((always_inline)) {
        if (k0 + TK <= a.n_keys) {  // uniform
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int v = tid + i * NT;
                if (EXACT || i < IT - 1 || v < NVEC) kreg[i] = *reinterpret_cast<const u32x4_t*>(kbase + (long)k0 * D * EB + v * 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int v = tid + i * NT;
                if (!(EXACT || i < IT - 1 || v < NVEC)) continue;
                const int key = min(k0 + v / KV_PER_ROW, a.n_keys - 1);
                kreg[i] = *reinterpret_cast<const u32x4_t*>(kbase + (long)key * D * EB + (v % KV_PER_ROW) * 16);
            }
        }
    };
    auto load_v = [&](int k0) __attribute__((always_inline)) {
        if (k0 + TK <= a.n_keys) {  // uniform
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int v = tid + i * NT;
                if (EXACT || i < IT - 1 || v < NVEC)
                    vreg[i] = *reinterpret_cast<const u32x4_t*>(vbase + ((long)(v / VV_PER_ROW) * a.t_max + k0 + (v % VV_PER_ROW) * EPV) * EB);
            }
        } else {
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int v = tid + i * NT;
                if (!(EXACT || i < IT - 1 || v < NVEC)) continue;
                const int d = v / VV_PER_ROW, key0 = k0 + (v % VV_PER_ROW) * EPV;
                u32x4_t val = {0u, 0u, 0u, 0u};
                if (key0 < a.n_keys) val = *reinterpret_cast<const u32x4_t*>(vbase + ((long)d * a.t_max + key0) * EB);
                const int nvalid = a.n_keys - key0;  // elements of this vector that are real keys
                if (EB == 2) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        val[e] &= (2 * e < nvalid ? 0xffffu : 0u) | (2 * e + 1 < nvalid ? 0xffff0000u : 0u);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) val[e] = e < nvalid ? val[e] : 0u;
                }
                vreg[i] = val;
            }
        }
    };
    auto store_k = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int v = tid + i * NT;
            if (!(EXACT || i < IT - 1 || v < NVEC)) continue;
            *reinterpret_cast<u32x4_t*>(ldsK + (v / KV_PER_ROW) * KS + (v % KV_PER_ROW) * 16) = kreg[i];
        }
    };
    auto store_v = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int v = tid + i * NT;
            if (!(EXACT || i < IT - 1 || v < NVEC)) continue;
            *reinterpret_cast<u32x4_t*>(ldsV + (v / VV_PER_ROW) * VS + (v % VV_PER_ROW) * 16) = vreg[i];
        }
    };

    // Direct-to-LDS ring: this lane's K fragment row and V^T fragment row inside a tile and
    // the swizzle terms of its 16-byte pieces (piece 2c + g of a K row, piece 4kb + 2hh + g of
    // a V^T row; the swizzle only involves the low row bits, which the 32-row block offsets
    // leave alone).
    const int krow_l = key_of_score_row(r);
    const int kfrag = krow_l * KROW;
    const int kx = g ^ (KROW == 128 ? ((krow_l >> 1) & 7) : (krow_l & 15));
    const int vfrag = r * VROW;
    const int vx = g ^ ((r >> 1) & 7);

    // Scores and online softmax of the staged K tile; leaves the probabilities in p.
    float p[NKB][16];
    auto scores_softmax = [&](int k0) __attribute__((always_inline)) {
        // Whether any key of this tile can be hidden from any row (uniform per tile).
        const bool tile_masked = a.mask != nullptr || k0 + TK > a.n_keys || (k0 < pad_hi && k0 + TK > pad_lo) ||
                                 (a.mask_kind != VLA_MASK_NONE && k0 + TK > a.n_prefix);
        float m_tile = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
            // the head_dim contraction runs as NA independent MFMA chains (a single chain of
            // NQ dependent MFMAs is latency-bound for wide heads), summed at the end
            // fragments are read FB at a time ahead of their MFMAs: a read per MFMA leaves every
            // MFMA waiting for the LDS latency, and for 256-wide heads the register allocator
            // otherwise keeps only two fragments in flight (the second accumulator chain is
            // given up for the fragment registers there)
            constexpr int FB = (NQ >= 16 && !DLOAD) ? WIDE_FB - 1 : 1;  // (one fewer than for V^T: the second accumulator chain takes the registers)
            constexpr int NA = (NQ >= 4 && NKB == 1) ? 2 : 1;
            f32x16_t sc[NA];
#pragma unroll
            for (int n = 0; n < NA; ++n)
#pragma unroll
                for (int i = 0; i < 16; ++i) sc[n][i] = 0.f;
            if constexpr (FB > 1) {
                // rolling read-ahead: FB fragments are on their way when the first product starts, and each
                // product is followed by the read of the fragment FB places further on
                u32x4_t kf[NQ];
#pragma unroll
                for (int c = 0; c < NQ; ++c)
                    kf[c] = *reinterpret_cast<const u32x4_t*>(ldsK + (kb * 32 + key_of_score_row(r)) * KS + (c * CE + g * (CE / 2)) * EB);
#pragma unroll
                for (int c = 0; c < NQ; ++c) A::mma(sc[c % NA], kf[c], qf[c]);
                __builtin_amdgcn_sched_group_barrier(0x100, FB, 0);
#pragma unroll
                for (int c = 0; c < NQ - FB; ++c) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, FB, 0);
            } else {
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(
                        DLOAD ? ldsK + kb * 32 * KROW + kfrag + (((2 * c) ^ kx) * 16)
                              : ldsK + (kb * 32 + key_of_score_row(r)) * KS + (c * CE + g * (CE / 2)) * EB);
                    A::mma(sc[c % NA], kf, qf[c]);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float v = sc[0][i];
#pragma unroll
                for (int n = 1; n < NA; ++n) v += sc[n][i];
                p[kb][i] = v * c2;
            }
        }
        if (tile_masked) {
            if (a.mask) {  // mask given as data: additive, one fp32 per (query, key)
#pragma unroll
                for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = k0 + kb * 32 + key_of_element(e, g);
                        p[kb][e] = key < a.n_keys ? p[kb][e] + a.mask[(long)s * a.n_keys + key] * LOG2E : -INFINITY;
                    }
            } else {
                const int kl = k0 + 8 * g;
#pragma unroll
                for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = kl + kb * 32 + key_of_element(e, 0);
                        const bool visible = (key < hi) & !((key >= pad_lo) & (key < pad_hi));
                        p[kb][e] = visible ? p[kb][e] : -INFINITY;
                    }
            }
        }
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) m_tile = fmaxf(m_tile, p[kb][i]);
        m_tile = halves_max(m_tile);
        // Online softmax with a lazily updated reference: m_run moves (and the accumulators
        // are rescaled) only when some row's maximum exceeds it by more than 2^RESCALE_LOG2;
        // until then the probabilities are taken against the older reference, at most
        // 2^RESCALE_LOG2 large, and the common factor cancels in o / l at the end.
        if (__builtin_amdgcn_ballot_w64(m_tile > m_run + RESCALE_LOG2) != 0) {
            const float m_new = fmaxf(m_run, m_tile);
            // m_new == -inf: nothing visible yet, keep everything at zero.
            const float alpha = A::fexp2(m_run - ((m_new == -INFINITY) ? 0.f : m_new));  // 2^-inf = 0 at the first visible tile
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = A::fexp2(p[kb][i] - m_use);
                p[kb][i] = e;
                psum += e;
            }
        psum = halves_sum(psum);
        l_run += psum;
    };
    // O^T += V^T . P^T from the staged V^T tile.
    auto output_product = [&](int k0) __attribute__((always_inline)) {
        // direct-to-LDS tiles arrive unfiltered: V^T elements past n_keys (stale cache
        // contents, possibly NaN) are zeroed in the fragment registers of the last tile
        const bool v_partial = DLOAD && k0 + TK > a.n_keys;  // uniform
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
            if constexpr (NL > 0 && EB == 2 && NDB >= 8 && NKB == 1) {
                // 256-wide heads: the 2 x NDB fragments of both key halves as one sequence with a rolling
                // read-ahead of WIDE_FB fragments, so that the LDS latency is paid once per tile
                // (with two-term probabilities the halves stay two sequences: both halves' terms at once do not fit the registers)
                constexpr int HPS = P2 ? 1 : 2, NF = HPS * NDB;  // key halves and fragments per sequence
#pragma unroll
                for (int h0 = 0; h0 < 2; h0 += HPS) {
                    u32x4_t pf[HPS], pl[HPS];
#pragma unroll
                    for (int hh = 0; hh < HPS; ++hh) {
                        const float* pp = &p[kb][(h0 + hh) * 8];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t hi16 = pack_bf2(pp[2 * e], pp[2 * e + 1]);
                            pf[hh][e] = hi16;
                            if (P2)
                                pl[hh][e] = pack_bf2(pp[2 * e] - __uint_as_float(hi16 << 16), pp[2 * e + 1] - __uint_as_float(hi16 & 0xffff0000u));
                        }
                    }
                    u32x4_t vf[NF];
#pragma unroll
                    for (int f = 0; f < NF; ++f)
                        vf[f] = *reinterpret_cast<const u32x4_t*>(ldsV + ((f % NDB) * 32 + r) * 64 + (((2 * (h0 + f / NDB) + g) ^ ((r >> 2) & 3)) * 16));  // (NKB == 1)
#pragma unroll
                    for (int f = 0; f < NF; ++f) {
                        A::mma(o[f % NDB], vf[f], pf[f / NDB]);
                        if (P2) A::mma(o[f % NDB], vf[f], pl[f / NDB]);
                    }
                    constexpr int MPF = P2 ? 2 : 1;  // products per fragment
                    __builtin_amdgcn_sched_group_barrier(0x100, WIDE_FB, 0);
#pragma unroll
                    for (int f = 0; f < NF - WIDE_FB; ++f) {
                        __builtin_amdgcn_sched_group_barrier(0x008, MPF, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x008, WIDE_FB * MPF, 0);
                }
            } else if (EB == 2) {
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    // P2: the probabilities enter the bf16 MFMA as hi + lo (two bf16 terms,
                    // ~16 mantissa bits), so the P.V product matches an fp32-probability
                    // reference instead of carrying a 2^-9 rounding per weight; otherwise
                    // one bf16 term (the rounding is of the size of the output's own).
                    const float* pp = &p[kb][hh * 8];
                    u32x4_t pf, pl;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t hi16 = pack_bf2(pp[2 * e], pp[2 * e + 1]);
                        pf[e] = hi16;
                        if (P2)
                            pl[e] = pack_bf2(pp[2 * e] - __uint_as_float(hi16 << 16), pp[2 * e + 1] - __uint_as_float(hi16 & 0xffff0000u));
                    }
                    const int key_off = (kb * 32 + hh * 16 + 8 * g) * EB;
                    const int nvalid = a.n_keys - (k0 + kb * 32 + hh * 16 + 8 * g);  // real keys among this lane's 8
                    {
#pragma unroll
                        for (int db = 0; db < NDB; ++db) {
                            u32x4_t vf = *reinterpret_cast<const u32x4_t*>(
                                DLOAD ? ldsV + db * 32 * VROW + vfrag + (((4 * kb + 2 * hh) ^ vx) * 16) : ldsV + (db * 32 + r) * VS + key_off);
                            if (v_partial) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) vf[e] &= (2 * e < nvalid ? 0xffffu : 0u) | (2 * e + 1 < nvalid ? 0xffff0000u : 0u);
                            }
                            A::mma(o[db], vf, pf);
                            if (P2) A::mma(o[db], vf, pl);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float* pp = &p[kb][4 * j];
                    const u32x4_t pf = {__float_as_uint(pp[0]), __float_as_uint(pp[1]), __float_as_uint(pp[2]),
                                        __float_as_uint(pp[3])};
                    const int key_off = (kb * 32 + key_of_element(4 * j, g)) * EB;
#pragma unroll
                    for (int db = 0; db < NDB; ++db) {
                        const u32x4_t vf = *reinterpret_cast<const u32x4_t*>(ldsV + (db * 32 + r) * VS + key_off);
                        A::mma(o[db], vf, pf);
                    }
                }
            }
        }
    };

    // The rows leave through LDS.  A lane holds 4 consecutive d of its query row per (block, j):
    // written from the registers that is 8-byte pieces of 32 different rows per instruction
    // (3.3 us of a 12.6 us launch for 256-wide heads at 83 keys).  The wavefront parks its
    // 32 x D tile (bf16 outputs, or fp16 partials of a key slice) in `park`, LDS nobody else
    // touches any more, and writes whole rows, 64 lanes x 16 bytes per instruction.
    auto flush_rows = [&](unsigned char* park) __attribute__((always_inline)) {
        constexpr int ROWB = D * 2 + 16;  // staged row: D 16-bit values + padding
        const bool as_partial = a.n_split > 1;
        const float inv_l = l_run > 0.f ? 1.0f / l_run : 0.f;
        const long prow = as_partial ? ((long)pair * a.n_split + split) * a.r_pad + row : 0;
        if (as_partial && row_valid && g == 0) {
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_run;
        }
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int d = db * 32 + 8 * j + 4 * g;
                if (d >= D) continue;
                const float v0 = o[db][4 * j] * inv_l, v1 = o[db][4 * j + 1] * inv_l, v2 = o[db][4 * j + 2] * inv_l,
                            v3 = o[db][4 * j + 3] * inv_l;
                u32x2_t pk;
                if (as_partial) {
                    typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
                    const h4_t hv = {(_Float16)v0, (_Float16)v1, (_Float16)v2, (_Float16)v3};
                    pk = __builtin_bit_cast(u32x2_t, hv);
                } else {
                    pk = u32x2_t{pack_bf2(v0, v1), pack_bf2(v2, v3)};
                }
                *reinterpret_cast<u32x2_t*>(park + r * ROWB + d * 2) = pk;
            }
        // destination of tile row rr, in 16-bit elements (-1: no such row), from the lane that owns it
        long dst = -1;
        if (row_valid && g == 0) dst = as_partial ? prow * D : (((long)b * a.S + s) * a.Hq + h) * D;
        const int dst_lo = (int)(dst & 0xffffffffl), dst_hi = (int)(dst >> 32);
        unsigned short* base16 = as_partial ? reinterpret_cast<unsigned short*>(a.part_o) : reinterpret_cast<unsigned short*>(a.out);
        constexpr int PIECES = D * 2 / 16, RPI = 64 / PIECES;  // 16-byte pieces per row, rows per instruction
#pragma unroll
        for (int i = 0; i < 32 / RPI; ++i) {
            const int rr = i * RPI + lane / PIECES, pc = lane % PIECES;
            const long d64 = ((long)__shfl(dst_hi, rr, 64) << 32) | (unsigned int)__shfl(dst_lo, rr, 64);
            const u32x4_t val = *reinterpret_cast<const u32x4_t*>(park + rr * ROWB + pc * 16);
            if (d64 >= 0) *reinterpret_cast<u32x4_t*>(base16 + d64 + pc * 8) = val;
        }
    };

    if constexpr (DLOAD) {
        constexpr int KI = KTILE / 1024, VI = VTILE / 1024;   // load instructions (1 KiB each) per K / V^T tile
        constexpr int PER_STEP = NSL * (KI + VI);
        constexpr int IPW = (PER_STEP + NWAVES - 1) / NWAVES;  // per wavefront and step, padded with repeats
        constexpr int KRPI = 1024 / KROW;                      // K rows per load instruction (8 or 4)
        static_assert(RS >= 2, "the ring needs a slot to load into while another is read");
        constexpr int W0 = (RS - 1) * IPW < 63 ? (RS - 1) * IPW : 63;  // a smaller count only waits longer
        constexpr int W1 = (RS - 2) * IPW < 63 ? (RS - 2) * IPW : 63;
        const int n_t = (k_end - k_begin + TK - 1) / TK;
        const int n_steps = (n_t + NSL - 1) / NSL;
        const uint32_t ring0 = (uint32_t)(uintptr_t)ring;  // low 32 bits of a shared-aperture address = LDS offset
        const int wv = __builtin_amdgcn_readfirstlane(wave);
        // Step `st` goes into ring slot `slot`.  Instruction j of a step: tile j / (KI + VI)
        // of the step, then K rows (j' < KI) or V^T rows.  Tiles past the last one repeat it
        // and K rows past n_keys repeat the last key (their scores are masked); V^T runs are
        // kept inside the cache row.  Repeats rewrite the same bytes, so the padding of the
        // per-wavefront count is harmless.
        auto issue_step = [&](int st, int slot) __attribute__((always_inline)) {
#pragma unroll
            for (int it = 0; it < IPW; ++it) {
                const int j = (wv + it * NWAVES) % PER_STEP;  // wavefront-uniform
                const int ts = j / (KI + VI), jj = j % (KI + VI);
                const int t = min(st * NSL + ts, n_t - 1);
                const int k0 = k_begin + t * TK;
                const uint32_t base = ring0 + (slot * NSL + ts) * STAGE;
                if (jj < KI) {
                    const int rowi = jj * KRPI + lane / (KROW / 16), pos = lane % (KROW / 16);
                    const int piece = pos ^ (KROW == 128 ? ((rowi >> 1) & 7) : (rowi & 15));
                    const int key = min(k0 + rowi, a.n_keys - 1);
                    load_to_lds16(kbase + (long)key * KROW + piece * 16, base + jj * 1024);
                } else {
                    const int rowi = (jj - KI) * 8 + lane / 8, pos = lane % 8;  // V^T rows are 128 bytes
                    const int piece = pos ^ ((rowi >> 1) & 7);
                    const int key0 = min(k0 + piece * 8, a.t_max - 8);
                    load_to_lds16(vbase + ((long)min(rowi, D - 1) * a.t_max + key0) * EB, base + KTILE + (jj - KI) * 1024);
                }
            }
        };
        // The whole ring is requested up front (for short key ranges that is every tile: the
        // kernel then pays the memory latency once); step st + RS - 1 follows at the start of
        // step st into the slot step st - 1 has just been read from.
#pragma unroll
        for (int st = 0; st < RS; ++st) issue_step(st, st);
        // The query fragments are ordinary loads, the ring's are inline assembly the compiler
        // does not count: left to itself it waits for the fragments at their first use, inside
        // the loop, with vmcnt(0) -- which also drains every ring load in flight, at every step.
        // Using them here puts that wait in front of the loop, once.
#pragma unroll
        for (int c = 0; c < NQ; ++c) asm volatile("" ::"v"(qf[c]));
        int slot = 0, lslot = RS - 1;
        for (int st = 0; st < n_steps; ++st) {
            // own loads of this step have landed (the younger ones may be pending) ...
            if (st == 0) wait_vmcnt<W0>();
            else wait_vmcnt<W1>();
            __syncthreads();  // ... everyone's have, and the slot read in the previous step is free
            if (st > 0) issue_step(st + RS - 1, lslot);
            const int t = st * NSL + sl;
            if (wave_active && t < n_t) {
                ldsK = ring + (slot * NSL + sl) * STAGE;
                ldsV = ldsK + KTILE;
                scores_softmax(k_begin + t * TK);
                output_product(k_begin + t * TK);
            }
            slot = (slot + 1 == RS) ? 0 : slot + 1;
            lslot = (lslot + 1 == RS) ? 0 : lslot + 1;
        }
        wait_vmcnt<0>();  // the repeats must have landed before the ring is reused
        __syncthreads();
        if constexpr (NSL > 1) {
            // slices 1.. leave their state in LDS, element-major with the lane innermost, so
            // the wavefront of slice 0 with the same row tile finds each value under its own lane
            constexpr int NE = NDB * 16 + 2;
            float* xch = reinterpret_cast<float*>(ring);
            if (sl > 0 && wave_active) {
                float* px = xch + ((long)((sl - 1) * NW + rw) * NE) * 64 + lane;
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int i = 0; i < 16; ++i) px[(db * 16 + i) * 64] = o[db][i];
                px[(NDB * 16) * 64] = m_run;
                px[(NDB * 16 + 1) * 64] = l_run;
            }
            __syncthreads();
            if (sl > 0) return;
            if (wave_active) {
#pragma unroll
                for (int s2 = 1; s2 < NSL; ++s2) {
                    const float* px = xch + ((long)((s2 - 1) * NW + rw) * NE) * 64 + lane;
                    const float m2 = px[(NDB * 16) * 64], l2 = px[(NDB * 16 + 1) * 64];
                    const float m_new = fmaxf(m_run, m2);
                    const float mm = (m_new == -INFINITY) ? 0.f : m_new;
                    const float w1 = A::fexp2(m_run - mm), w2 = A::fexp2(m2 - mm);  // 2^-inf = 0 for an empty side
                    l_run = l_run * w1 + l2 * w2;
                    m_run = m_new;
#pragma unroll
                    for (int db = 0; db < NDB; ++db)
#pragma unroll
                        for (int i = 0; i < 16; ++i) o[db][i] = o[db][i] * w1 + px[(db * 16 + i) * 64] * w2;
                }
            }
        }
    } else if constexpr (NL > 0) {
        constexpr int NTL = NL * 64, ITL = NVEC / NTL, LOAD_AHEAD = 3;
        static_assert(NVEC % NTL == 0 && EB == 2, "loader wavefronts split a tile evenly; bf16 only");
        const int n_t = (k_end - k_begin + TK - 1) / TK;
        const int n_pad = (n_t + LOAD_AHEAD - 1) / LOAD_AHEAD * LOAD_AHEAD;  // both roles run n_pad + 1 barriers
        if (wave >= NW) {
            const int lt = tid - NW * 64;
            u32x4_t kq[LOAD_AHEAD][ITL], vq[LOAD_AHEAD][ITL];
            // V^T rows lie unpadded (64 bytes) with their four 16-byte pieces XOR-swizzled by (row >> 2) & 3.  A
            // 16-byte LDS store is served eight lanes at a time and two of them collide when their addresses agree
            // in bits 4 .. 6: with 80-byte rows the first and the last of every eight lanes (two rows of four
            // pieces) do, and every store takes twice as long; the fragment reads (sixteen lanes at a time, rows
            // r, r + 12, r + 20, r + 24 together) are free of conflicts either way.
            static_assert(VV_PER_ROW == 4, "swizzle of four pieces per V^T row");
            auto v_at = [](int v) __attribute__((always_inline)) { return (v / 4) * 64 + (((v % 4) ^ ((v >> 4) & 3)) * 16); };
            // Unconditional loads with clamped addresses (K rows past n_keys repeat the last
            // key: their scores are masked; V^T runs are kept inside the row) so the loop body
            // has no load under a branch; tiles past the last repeat it and are never read.
            auto fetch = [&](int slot, int t) __attribute__((always_inline)) {
                const int k0 = k_begin + max(min(t, n_t - 1), 0) * TK;
#pragma unroll
                for (int i = 0; i < ITL; ++i) {
                    const int v = lt + i * NTL;
                    const int key = min(k0 + v / KV_PER_ROW, a.n_keys - 1);
                    kq[slot][i] = *reinterpret_cast<const u32x4_t*>(kbase + (long)key * D * EB + (v % KV_PER_ROW) * 16);
                    const int key0 = min(k0 + (v % VV_PER_ROW) * EPV, a.t_max - EPV);
                    vq[slot][i] = *reinterpret_cast<const u32x4_t*>(vbase + ((long)(v / VV_PER_ROW) * a.t_max + key0) * EB);
                }
            };
            // V^T elements past n_keys are zeroed so that stale cache contents (possibly NaN)
            // cannot reach the accumulators.
            // Only the tile that reaches past n_keys is masked, under a uniform branch: masking
            // every tile lets the compiler gather the mask arithmetic of all slots at the top of
            // the unrolled loop, in front of a wait for every load in flight -- the youngest
            // fetch included, which is the look-ahead gone.
            auto publish = [&](int slot, int t, int stage) __attribute__((always_inline)) {
                const int k0 = k_begin + max(min(t, n_t - 1), 0) * TK;
                if (k0 + TK <= a.n_keys) {
#pragma unroll
                    for (int i = 0; i < ITL; ++i) {
                        const int v = lt + i * NTL;
                        *reinterpret_cast<u32x4_t*>(ldsK_buf[stage] + (v / KV_PER_ROW) * KS + (v % KV_PER_ROW) * 16) = kq[slot][i];
                        *reinterpret_cast<u32x4_t*>(ldsV_buf[stage] + v_at(v)) = vq[slot][i];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < ITL; ++i) {
                        const int v = lt + i * NTL;
                        *reinterpret_cast<u32x4_t*>(ldsK_buf[stage] + (v / KV_PER_ROW) * KS + (v % KV_PER_ROW) * 16) = kq[slot][i];
                        const int nvalid = a.n_keys - (k0 + (v % VV_PER_ROW) * EPV);  // real keys among the 8, may be <= 0
                        u32x4_t val = vq[slot][i];
#pragma unroll
                        for (int e = 0; e < 4; ++e) val[e] &= (2 * e < nvalid ? 0xffffu : 0u) | (2 * e + 1 < nvalid ? 0xffff0000u : 0u);
                        *reinterpret_cast<u32x4_t*>(ldsV_buf[stage] + v_at(v)) = val;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            };
#pragma unroll
            for (int sl = 0; sl < LOAD_AHEAD; ++sl) fetch(sl, sl);
            publish(0, 0, 0);
            __syncthreads();
            for (int t0 = 0; t0 < n_pad; t0 += LOAD_AHEAD) {
#pragma unroll
                for (int sl = 0; sl < LOAD_AHEAD; ++sl) {
                    const int t = t0 + sl;
                    fetch(sl, t + LOAD_AHEAD);                       // slot sl held tile t, already published
                    publish((sl + 1) % LOAD_AHEAD, t + 1, (t + 1) & 1);  // while the compute wavefronts read stage t & 1
                    __syncthreads();
                }
            }
            // the loader wavefronts own no rows: they go on to the tail and leave there
        } else {
            __syncthreads();
            for (int t = 0; t < n_pad; ++t) {
                if (t < n_t && wave_active) {
                    ldsK = ldsK_buf[t & 1];
                    ldsV = ldsV_buf[t & 1];
                    scores_softmax(k_begin + t * TK);
                    output_product(k_begin + t * TK);
                }
                __syncthreads();
            }
        }
    } else if (PREFETCH) {
        // Small tiles: the whole next tile waits in registers while the current one is used.
        if (k_begin < k_end) {
            load_k(k_begin);
            load_v(k_begin);
        }
        for (int k0 = k_begin; k0 < k_end; k0 += TK) {
            __syncthreads();  // previous tile fully consumed
            store_k();
            store_v();
            __syncthreads();
            if (k0 + TK < k_end) {
                load_k(k0 + TK);
                load_v(k0 + TK);
            }
            // keep the loads above the math: left alone, the scheduler sinks them next to
            // their first use (the next iteration's LDS stores) and the prefetch is lost
            __builtin_amdgcn_sched_barrier(0);
            if (wave_active) {
                scores_softmax(k0);
                output_product(k0);
            }
        }
    } else {
        // Wide heads: one operand in registers at a time.  V^T of this tile is fetched
        // under the score product, K of the next tile under the output product.  Nobody
        // reads the K buffer between the second barrier of a tile and the first of the
        // next, nor the V^T buffer between a tile's output product and the next first
        // barrier, so two barriers per tile suffice.
        if (k_begin < k_end) load_k(k_begin);
        for (int k0 = k_begin; k0 < k_end; k0 += TK) {
            store_k();
            __syncthreads();
            load_v(k0);
            __builtin_amdgcn_sched_barrier(0);  // loads stay above the math they hide behind
            if (wave_active) scores_softmax(k0);
            store_v();
            __syncthreads();
            if (k0 + TK < k_end) load_k(k0 + TK);
            __builtin_amdgcn_sched_barrier(0);
            if (wave_active) output_product(k0);
        }
    }

    if constexpr (NL > 0) {
        // every wavefront is past the loop's last barrier: nobody reads the K / V^T tile buffers
        // any more, and a buffer holds exactly one wavefront's 32-row tile
        if (wave >= NW) return;  // loader wavefronts own no rows
        static_assert(TK * KS >= 32 * (D * 2 + 16) && DP * VS >= 32 * (D * 2 + 16) && NW <= 4, "a tile buffer parks one wavefront's rows");
        if (a.n_split == 1 || a.part_half) {
            flush_rows(wave < 2 ? ldsK_buf[wave] : ldsV_buf[wave - 2]);
            return;
        }
    }
    if (!row_valid) return;
    if (a.n_split > 1) {
        // unnormalised partial for the merge kernel
        const long prow = ((long)pair * a.n_split + split) * a.r_pad + row;
        if (g == 0) {
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_run;
        }
        if (a.part_half) {
            // normalised by the slice's own sum, so the values are averages of V rows (safe in
            // fp16's range) and carry 11 bits; the merge weights them with l * 2^(m - m_all)
            typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
            const float inv_l = l_run > 0.f ? 1.0f / l_run : 0.f;
            _Float16* ph = reinterpret_cast<_Float16*>(a.part_o) + prow * D;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d = db * 32 + 8 * j + 4 * g;
                    if (d >= D) continue;
                    const h4_t pk = {(_Float16)(o[db][4 * j] * inv_l), (_Float16)(o[db][4 * j + 1] * inv_l),
                                     (_Float16)(o[db][4 * j + 2] * inv_l), (_Float16)(o[db][4 * j + 3] * inv_l)};
                    *reinterpret_cast<h4_t*>(ph + d) = pk;
                }
            return;
        }
        float* po = a.part_o + prow * D;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int d = db * 32 + 8 * j + 4 * g;
                if (d >= D) continue;
                const f32x4_t pk = {o[db][4 * j], o[db][4 * j + 1], o[db][4 * j + 2], o[db][4 * j + 3]};
                *reinterpret_cast<f32x4_t*>(po + d) = pk;
            }
        return;
    }
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

// Key slices of one pair as wavefronts of different workgroups, merged without a second launch
// (attn_decode16_kernel): every slice writes its unnormalised partial rows and (max, sum), then
// counts itself in; the one that finds all others counted combines them and writes the output.
// No wavefront waits for another.  The partials cross between the per-XCD L2s as device-scope
// relaxed atomic accesses (write-through stores, loads served from memory) and the count is
// taken only after the wavefront's stores have been acknowledged, so neither side needs a
// cache-wide write-back or invalidate.  The arithmetic order is fixed by the slice index, not
// by who arrives last.  The counters are left at zero by the merging slice, for the next launch:
// a launch that is cut short (a fault elsewhere on the device, a reset) leaves the counters of
// its unfinished units non-zero and so poisons the block for every launch after it, which is
// why the owner of a workspace zeroes them at the start of each launch sequence
// (vla_attn_workspace_reset) instead of relying on the last launch alone.  At most ARRIVE_MAX_T
// (row, slice) pairs per pair of (batch, kv head), 128-wide heads.
constexpr int ARRIVE_MAX_T = 48, ARRIVE_MAX_UNITS = 16384;
__device__ __forceinline__ void st_dev64(float* p, float x, float y) {
    const unsigned long long v = (unsigned long long)__float_as_uint(x) | ((unsigned long long)__float_as_uint(y) << 32);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long ld_dev64(const float* p) {
    return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Few query rows per (batch, kv head) -- at most one 32-row tile: GR00T's 17 DiT tokens,
// single-token decode.  Nothing is shared between wavefronts then, so K and V^T go straight
// from the cache into MFMA operand registers (no LDS, no barriers): lane (g, r) of a
// wavefront reads 16 bytes of key row r for the score product and two 8-byte runs of V^T
// row r for the output product, exactly the fragments the LDS kernel would fetch.  A
// wavefront owns one (pair, key slice) and keeps ST 32-key blocks of loads in flight.
// MERGE: a workgroup is one pair and its wavefronts are the key slices; they combine
// their partial (max, sum, output) through LDS, so sliced decode is one launch.
template <int D, bool P2, int ST, bool MERGE>
__global__ void __launch_bounds__((MERGE && D <= 64) ? 512 : 256, D <= 64 ? 2 : 1) attn_direct_kernel(AttnArgs a) {
    constexpr int EB = 2, CE = 16;
    constexpr int NQ = D / CE, NDB = (D + 31) / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 5, r = lane & 31;
    const int unit = MERGE ? blockIdx.x * a.n_split + wave : blockIdx.x * (int)(blockDim.x >> 6) + wave;
    const int prb = unit / a.n_split, split = unit % a.n_split;  // (pair, 32-row block) and key slice
    const int pair = prb / a.n_rblocks, rb = prb % a.n_rblocks;
    // whole wavefront (whole workgroup with MERGE); the main loop has no barriers
    if (pair >= a.batch * a.Hkv) return;
    const int b = pair / a.Hkv, hk = pair % a.Hkv;
    const int grp = a.Hq / a.Hkv, R = grp * a.S;
    const int row = rb * 32 + r;
    const bool row_valid = row < R;
    const int hg = row_valid ? row / a.S : 0, s = row_valid ? row % a.S : 0;
    const int h = hk * grp + hg;

    const int nb_total = (a.n_keys + 31) / 32;
    // the slice's block range is the same for every lane of the wavefront; said so explicitly
    // (it is derived from the wavefront's index), the loop below runs on scalar branches
    const int kb0 = __builtin_amdgcn_readfirstlane(split * a.tiles_per_split);
    const int kb1 = __builtin_amdgcn_readfirstlane(min(nb_total, kb0 + a.tiles_per_split));

    u32x4_t qf[NQ];
    {
        const unsigned char* qrow = (const unsigned char*)a.q + (((long)b * a.S + s) * a.Hq + h) * D * EB;
#pragma unroll
        for (int c = 0; c < NQ; ++c) {
            u32x4_t z = {0u, 0u, 0u, 0u};
            qf[c] = row_valid ? *reinterpret_cast<const u32x4_t*>(qrow + (c * CE + g * 8) * EB) : z;
        }
    }
    f32x16_t o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    constexpr float LOG2E = 1.4426950408889634f;
    const float c2 = a.scale * LOG2E;

    const unsigned char* kbase = (const unsigned char*)a.k_cache + ((long)b * a.Hkv + hk) * a.t_max * D * EB;
    const unsigned char* vbase = (const unsigned char*)a.vt_cache + ((long)b * a.Hkv + hk) * D * (long)a.t_max * EB;

    u32x4_t kr[ST][NQ];
    u32x4_t vr[ST][NDB][2];  // [stage][32-row block of d][16-key half]: 8 consecutive keys per lane
    // Rows of V^T past head_dim (D = 48: the upper half of the second 32-row block) are
    // read from row D-1 instead, so every lane loads valid memory; their outputs are dropped.
    const unsigned char* vrow[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) vrow[db] = vbase + (long)min(db * 32 + r, D - 1) * a.t_max * EB;
    const int krow = key_of_score_row(r);  // the key of the block this lane fetches for the score product
    // One block of loads, the same seven instructions for every block, with no branch around
    // any of them: the compiler's count of loads in flight is then exact, and the wait in
    // front of a block's arithmetic leaves the younger blocks' loads in flight (with the
    // loads under branches it waited for all of them: the look-ahead was on paper only).
    // K rows past n_keys repeat the last key (their scores are masked); V^T runs past n_keys
    // are kept inside the cache row (t_max is a multiple of 8: a run that would start past
    // t_max - 8 reads the row's last run instead) and are zeroed by mask_partial once the
    // data is needed, so that stale cache contents (possibly NaN) cannot reach the
    // accumulators.  Blocks past the slice repeat its last block and are never multiplied.
    auto load_blk = [&](int st, int kb_any) __attribute__((always_inline)) {
        const int kb = min(kb_any, kb1 - 1);
        const int key = min(kb * 32 + krow, a.n_keys - 1);
        const unsigned char* kp = kbase + (long)key * D * EB + g * 16;
#pragma unroll
        for (int c = 0; c < NQ; ++c) kr[st][c] = *reinterpret_cast<const u32x4_t*>(kp + c * CE * EB);
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int k8 = min(kb * 32 + hh * 16 + 8 * g, a.t_max - 8);  // first of this lane's 8 consecutive keys
#pragma unroll
            for (int db = 0; db < NDB; ++db) vr[st][db][hh] = *reinterpret_cast<const u32x4_t*>(vrow[db] + k8 * EB);
        }
    };
    auto mask_partial = [&](int st, int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int nvalid = a.n_keys - (kb * 32 + hh * 16 + 8 * g);  // real keys among this lane's 8, may be <= 0
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    vr[st][db][hh][e] &= (2 * e < nvalid ? 0xffffu : 0u) | (2 * e + 1 < nvalid ? 0xffff0000u : 0u);
        }
    };
    // Per-row visibility of the generated masks, branch-free (see the LDS kernel).
    int hi = a.n_keys;
    if (a.mask_kind == VLA_MASK_CAUSAL_SUFFIX) hi = min(a.n_keys, a.n_prefix + s + 1);
    else if (a.mask_kind == VLA_MASK_PI0_STATE && s == 0) hi = min(a.n_keys, a.n_prefix + 1);
    const int pad_lo = a.pad_start, pad_hi = min(a.pad_end, a.n_prefix);
    auto compute = [&](int st, int kb) __attribute__((always_inline)) {
        const int k0 = kb * 32;
        f32x16_t sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NQ; ++c) AT<bf16_t>::mma(sc, kr[st][c], qf[c]);
        const bool blk_masked = a.mask != nullptr || k0 + 32 > a.n_keys || (k0 < pad_hi && k0 + 32 > pad_lo) ||
                                (a.mask_kind != VLA_MASK_NONE && k0 + 32 > a.n_prefix);
        float p[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i] = sc[i] * c2;
        if (blk_masked) {
            if (a.mask) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = k0 + key_of_element(e, g);
                    p[e] = key < a.n_keys ? p[e] + a.mask[(long)s * a.n_keys + key] * LOG2E : -INFINITY;
                }
            } else {
                const int kl = k0 + 8 * g, hi_blk = hi;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = kl + key_of_element(e, 0);
                    const bool visible = (key < hi_blk) & !((key >= pad_lo) & (key < pad_hi));
                    p[e] = visible ? p[e] : -INFINITY;
                }
            }
        }
        float m_blk = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) m_blk = fmaxf(m_blk, p[i]);
        m_blk = halves_max(m_blk);
        if (__builtin_amdgcn_ballot_w64(m_blk > m_run + RESCALE_LOG2) != 0) {  // lazy reference update
            const float m_new = fmaxf(m_run, m_blk);
            const float alpha = __builtin_amdgcn_exp2f(m_run - ((m_new == -INFINITY) ? 0.f : m_new));
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            p[i] = __builtin_amdgcn_exp2f(p[i] - m_use);
            psum += p[i];
        }
        psum = halves_sum(psum);
        l_run += psum;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const float* pp = &p[hh * 8];
            u32x4_t pf, pl;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t hi = pack_bf2(pp[2 * e], pp[2 * e + 1]);
                pf[e] = hi;
                if (P2) pl[e] = pack_bf2(pp[2 * e] - __uint_as_float(hi << 16), pp[2 * e + 1] - __uint_as_float(hi & 0xffff0000u));
            }
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                AT<bf16_t>::mma(o[db], vr[st][db][hh], pf);
                if (P2) AT<bf16_t>::mma(o[db], vr[st][db][hh], pl);
            }
        }
    };

    // Software pipeline over the slice's blocks [kb0, kb1) in key order: ST - 1 blocks of
    // loads stay in flight ahead of the block being multiplied.  Only the slice that reaches
    // n_keys can end in a partial block.  The conditions in the loop are uniform over the
    // wavefront (scalar branches) and none of them guards a load.
    const bool has_partial = kb1 * 32 > a.n_keys;
    const int kbp = has_partial ? kb1 - 1 : -1;  // the partial block, if any
    if (kb1 - kb0 < ST) {
        // a slice shorter than the pipeline (GR00T's 17-key self attention is one block): the
        // pipeline's repeats of the last block would be most of its loads
        for (int kb = kb0; kb < kb1; ++kb) {
            load_blk(0, kb);
            if (kb == kbp) mask_partial(0, kb);
            compute(0, kb);
        }
    } else {
#pragma unroll
        for (int i = 0; i < ST - 1; ++i) load_blk(i, kb0 + i);
        for (int base = kb0; base < kb1; base += ST) {
#pragma unroll
            for (int st = 0; st < ST; ++st) {
                const int cur = base + st;
                load_blk((st + ST - 1) % ST, cur + ST - 1);
                __builtin_amdgcn_sched_barrier(0);  // loads stay above the math they hide behind
                if (cur < kb1) {
                    if (cur == kbp) mask_partial(st, cur);
                    compute(st, cur);
                }
            }
        }
    }

    if (MERGE) {
        // LDS: [slice][row of the block][D + 2] floats (unnormalised output, then max and sum)
        extern __shared__ float merge_buf[];
        const int RS = D + 2;
        const int Rb = min(32, R - rb * 32);  // rows of this block
        const int RB = min(32, R);            // rows per slice in the buffer
        if (row_valid) {
            float* pr = merge_buf + ((long)split * RB + r) * RS;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d = db * 32 + 8 * j + 4 * g;
                    if (d >= D) continue;
                    const f32x4_t pk = {o[db][4 * j], o[db][4 * j + 1], o[db][4 * j + 2], o[db][4 * j + 3]};
                    *reinterpret_cast<f32x4_t*>(pr + d) = pk;
                }
            if (g == 0) {
                pr[D] = m_run;
                pr[D + 1] = l_run;
            }
        }
        __syncthreads();
        for (int i = threadIdx.x; i < Rb * D; i += blockDim.x) {
            const int rl = i / D, d = i % D;
            float m = -INFINITY;
            for (int sp = 0; sp < a.n_split; ++sp) m = fmaxf(m, merge_buf[((long)sp * RB + rl) * RS + D]);
            float l = 0.f, acc = 0.f;
            if (m > -INFINITY) {
                for (int sp = 0; sp < a.n_split; ++sp) {
                    const float* pr = merge_buf + ((long)sp * RB + rl) * RS;
                    const float w = exp2f(pr[D] - m);
                    l += pr[D + 1] * w;
                    acc += pr[d] * w;
                }
            }
            const int grow = rb * 32 + rl;
            const int hh = hk * grp + grow / a.S, ss = grow % a.S;
            ((bf16_t*)a.out)[(((long)b * a.S + ss) * a.Hq + hh) * D + d] = f2bf(l > 0.f ? acc / l : 0.f);
        }
        return;
    }
    if (!row_valid) return;
    if (a.n_split > 1) {
        const long prow = ((long)pair * a.n_split + split) * a.r_pad + row;
        if (g == 0) {
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_run;
        }
        float* po = a.part_o + prow * D;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int d = db * 32 + 8 * j + 4 * g;
                if (d >= D) continue;
                const f32x4_t pk = {o[db][4 * j], o[db][4 * j + 1], o[db][4 * j + 2], o[db][4 * j + 3]};
                *reinterpret_cast<f32x4_t*>(po + d) = pk;
            }
        return;
    }
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    unsigned char* orow = (unsigned char*)a.out + (((long)b * a.S + s) * a.Hq + h) * D * EB;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = db * 32 + 8 * j + 4 * g;
            if (d >= D) continue;
            const u32x2_t pk = {pack_bf2(o[db][4 * j] * inv, o[db][4 * j + 1] * inv),
                                pack_bf2(o[db][4 * j + 2] * inv, o[db][4 * j + 3] * inv)};
            *reinterpret_cast<u32x2_t*>(orow + d * EB) = pk;
        }
}

// ---- Decode with 128-wide heads and at most 16 query rows per kv head (single-token decode of
// a grouped-query model: the group's heads are the rows).  The register-direct kernel above
// pads such rows to a 32-row MFMA tile; here the products are formed transposed on
// v_mfma_f32_16x16x32_bf16, a quarter of the matrix work per key block and half the softmax:
//
//   S^T = K Q^T  two products per 32-key block; row i of product j stands for key
//                8 (i / 4) + 4 j + i % 4 of the block, so that lane (c, q) = (lane % 16, lane / 16)
//                ends up with the scores of keys 8 q .. 8 q + 7 against query c in key order --
//   O^T += V^T P^T  -- which is P^T as this instruction's right operand (32 keys x 16 queries),
//                without a lane exchange; lane (c, q) reads 8 consecutive keys of V^T row
//                16 db + c and holds output columns 16 db + 4 q .. + 3 of query c.
//
// A wavefront is one (pair, key slice) and a workgroup of its own; the slices of a pair are
// merged inside the launch by the one that arrives last, with the partial rows laid out
// [pair][row][slice] and the merge unrolled for the slice count.
constexpr int DEC_MAX_NS = 12, DEC_MAX_R = 16;

template <int NS>
__device__ __forceinline__ void merge_rows_static(const AttnArgs& a, int pair, int b, int hk, int grp, int R, int lane) {
    constexpr int D = 128;
    constexpr int MAXR = ARRIVE_MAX_T / NS < DEC_MAX_R ? ARRIVE_MAX_T / NS : DEC_MAX_R;
    const long prow0 = (long)pair * a.r_pad * NS;
    // lane t = row * NS + slice holds that partial's (max, sum)
    float mt = -INFINITY, lt = 0.f;
    if (lane < R * NS) {
        const unsigned long long v = ld_dev64(a.part_ml + (prow0 + lane) * 2);
        mt = __uint_as_float((uint32_t)v);
        lt = __uint_as_float((uint32_t)(v >> 32));
    }
    unsigned long long pv[MAXR][NS];
    const float* pb = a.part_o + prow0 * D + lane * 2;
#pragma unroll
    for (int rl = 0; rl < MAXR; ++rl) {
        if (rl < R) {  // uniform
#pragma unroll
            for (int sp = 0; sp < NS; ++sp) pv[rl][sp] = ld_dev64(pb + (rl * NS + sp) * D);
        }
    }
    int hh = hk * grp, ss = 0;
#pragma unroll
    for (int rl = 0; rl < MAXR; ++rl) {
        if (rl < R) {  // uniform
            // the row's slice maxima and sums, read from their lanes into scalar registers: every lane forms the same weights
            float mj[NS], mrow = -INFINITY;
#pragma unroll
            for (int sp = 0; sp < NS; ++sp) {
                mj[sp] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(mt), rl * NS + sp));
                mrow = fmaxf(mrow, mj[sp]);
            }
            float a0 = 0.f, a1 = 0.f, lrow = 0.f;
#pragma unroll
            for (int sp = 0; sp < NS; ++sp) {
                const float w = mrow > -INFINITY ? __builtin_amdgcn_exp2f(mj[sp] - mrow) : 0.f;
                lrow += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(lt), rl * NS + sp)) * w;
                a0 += __uint_as_float((uint32_t)pv[rl][sp]) * w;
                a1 += __uint_as_float((uint32_t)(pv[rl][sp] >> 32)) * w;
            }
            const float iv = lrow > 0.f ? 1.0f / lrow : 0.f;
            reinterpret_cast<uint32_t*>((bf16_t*)a.out + (((long)b * a.S + ss) * a.Hq + hh) * D)[lane] = pack_bf2(a0 * iv, a1 * iv);
            if (++ss == a.S) {
                ss = 0;
                ++hh;
            }
        }
    }
}

template <bool P2, int ST>
__global__ void __launch_bounds__(64) attn_decode16_kernel(AttnArgs a) {
    constexpr int D = 128, EB = 2, NKS = D / 32, NDB = D / 16;
    const int lane = threadIdx.x, c = lane & 15, q = lane >> 4;
    const int pair = blockIdx.x / a.n_split, split = blockIdx.x % a.n_split;
    const int b = pair / a.Hkv, hk = pair % a.Hkv;
    const int grp = a.Hq / a.Hkv, R = grp * a.S;
    const bool row_valid = c < R;
    const int hg = row_valid ? c / a.S : 0, s = row_valid ? c % a.S : 0;
    const int h = hk * grp + hg;
    const int nb_total = (a.n_keys + 31) / 32;
    const int kb0 = __builtin_amdgcn_readfirstlane(split * a.tiles_per_split);
    const int kb1 = __builtin_amdgcn_readfirstlane(min(nb_total, kb0 + a.tiles_per_split));

    u32x4_t qf[NKS];
    {
        const unsigned char* qrow = (const unsigned char*)a.q + (((long)b * a.S + s) * a.Hq + h) * D * EB + q * 16;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const u32x4_t z = {0u, 0u, 0u, 0u};
            qf[ks] = row_valid ? *reinterpret_cast<const u32x4_t*>(qrow + ks * 64) : z;
        }
    }
    f32x4_t o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    constexpr float LOG2E = 1.4426950408889634f;
    const float c2 = a.scale * LOG2E;

    const unsigned char* kbase = (const unsigned char*)a.k_cache + ((long)b * a.Hkv + hk) * a.t_max * D * EB + q * 16;
    const unsigned char* vbase = (const unsigned char*)a.vt_cache + (((long)b * a.Hkv + hk) * D + c) * (long)a.t_max * EB;
    const long vstep = 16l * a.t_max * EB;  // 16 rows of V^T
    const int krow = 8 * (c >> 2) + (c & 3);  // this lane's key in product 0; product 1 takes the key 4 further

    u32x4_t kr[ST][2][NKS];
    u32x4_t vr[ST][NDB];  // 8 consecutive keys of V^T row 16 db + c
    // One block of loads, the same sixteen instructions for every block and no branch around any
    // of them.  K rows past n_keys repeat the last key (their scores are masked); V^T runs past
    // n_keys stay inside the cache row and are zeroed by mask_partial before they are multiplied
    // (stale cache contents may be NaN).  Blocks past the slice repeat its last block.
    auto load_blk = [&](int st, int kb_any) __attribute__((always_inline)) {
        const int kb = min(kb_any, kb1 - 1);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int key = min(kb * 32 + krow + 4 * j, a.n_keys - 1);
            const unsigned char* kp = kbase + (long)key * D * EB;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) kr[st][j][ks] = *reinterpret_cast<const u32x4_t*>(kp + ks * 64);
        }
        const int k8 = min(kb * 32 + 8 * q, a.t_max - 8);
#pragma unroll
        for (int db = 0; db < NDB; ++db) vr[st][db] = *reinterpret_cast<const u32x4_t*>(vbase + db * vstep + k8 * EB);
    };
    auto mask_partial = [&](int st, int kb) __attribute__((always_inline)) {
        const int nvalid = a.n_keys - (kb * 32 + 8 * q);  // real keys among this lane's 8, may be <= 0
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int e = 0; e < 4; ++e) vr[st][db][e] &= (2 * e < nvalid ? 0xffffu : 0u) | (2 * e + 1 < nvalid ? 0xffff0000u : 0u);
    };
    int hi = a.n_keys;
    if (a.mask_kind == VLA_MASK_CAUSAL_SUFFIX) hi = min(a.n_keys, a.n_prefix + s + 1);
    else if (a.mask_kind == VLA_MASK_PI0_STATE && s == 0) hi = min(a.n_keys, a.n_prefix + 1);
    const int pad_lo = a.pad_start, pad_hi = min(a.pad_end, a.n_prefix);
    auto compute = [&](int st, int kb) __attribute__((always_inline)) {
        const int k0 = kb * 32;
        f32x4_t sc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            sc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
                sc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kr[st][j][ks]), __builtin_bit_cast(bf16x8_t, qf[ks]),
                                                                sc[j], 0, 0, 0);
        }
        const bool blk_masked = a.mask != nullptr || k0 + 32 > a.n_keys || (k0 < pad_hi && k0 + 32 > pad_lo) ||
                                (a.mask_kind != VLA_MASK_NONE && k0 + 32 > a.n_prefix);
        float p[8];  // keys k0 + 8 q + i
#pragma unroll
        for (int i = 0; i < 8; ++i) p[i] = sc[i >> 2][i & 3] * c2;
        if (blk_masked) {
            const int kl = k0 + 8 * q;
            if (a.mask) {
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] = kl + i < a.n_keys ? p[i] + a.mask[(long)s * a.n_keys + kl + i] * LOG2E : -INFINITY;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int key = kl + i;
                    const bool visible = (key < hi) & !((key >= pad_lo) & (key < pad_hi));
                    p[i] = visible ? p[i] : -INFINITY;
                }
            }
        }
        float m_blk = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) m_blk = fmaxf(m_blk, p[i]);
        m_blk = rows_max(m_blk);
        if (__builtin_amdgcn_ballot_w64(m_blk > m_run + RESCALE_LOG2) != 0) {  // lazy reference update
            const float m_new = fmaxf(m_run, m_blk);
            const float alpha = __builtin_amdgcn_exp2f(m_run - ((m_new == -INFINITY) ? 0.f : m_new));
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[db][e] *= alpha;
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p[i] = __builtin_amdgcn_exp2f(p[i] - m_use);
            psum += p[i];
        }
        psum = rows_sum(psum);
        l_run += psum;
        u32x4_t pf, pl;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t hw = pack_bf2(p[2 * e], p[2 * e + 1]);
            pf[e] = hw;
            if (P2) pl[e] = pack_bf2(p[2 * e] - __uint_as_float(hw << 16), p[2 * e + 1] - __uint_as_float(hw & 0xffff0000u));
        }
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vr[st][db]), __builtin_bit_cast(bf16x8_t, pf), o[db], 0, 0, 0);
            if (P2)
                o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vr[st][db]), __builtin_bit_cast(bf16x8_t, pl), o[db], 0, 0, 0);
        }
    };

    // ST blocks of loads in flight from the start (a slice is at most ST blocks in the shapes this
    // kernel is chosen for, so it makes one trip to memory); longer slices refill a stage as
    // soon as it has been multiplied.
    const bool has_partial = kb1 * 32 > a.n_keys;
    const int kbp = has_partial ? kb1 - 1 : -1;
#pragma unroll
    for (int i = 0; i < ST; ++i) load_blk(i, kb0 + i);
    // The first ST blocks outside the loop: straight-line code, so the wait in front of a block
    // leaves the younger blocks' loads in flight (behind a loop header the count would have to
    // assume the worst of both ways in).
#pragma unroll
    for (int st = 0; st < ST; ++st) {
        const int cur = kb0 + st;
        if (cur < kb1) {  // uniform
            if (cur == kbp) mask_partial(st, cur);
            compute(st, cur);
        }
        if (cur + ST < kb1) load_blk(st, cur + ST);  // uniform; only slices longer than ST blocks
    }
    for (int base = kb0 + ST; base < kb1; base += ST) {
#pragma unroll
        for (int st = 0; st < ST; ++st) {
            const int cur = base + st;
            if (cur < kb1) {
                if (cur == kbp) mask_partial(st, cur);
                compute(st, cur);
            }
            if (cur + ST < kb1) load_blk(st, cur + ST);
        }
    }

    // partial rows [pair][row][slice]: unnormalised output, then (max, sum)
    if (row_valid) {
        const long prow = ((long)pair * a.r_pad + c) * a.n_split + split;
        if (q == 0) st_dev64(a.part_ml + prow * 2, m_run, l_run);
        float* po = a.part_o + prow * D + 4 * q;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            st_dev64(po + db * 16, o[db][0], o[db][1]);
            st_dev64(po + db * 16 + 2, o[db][2], o[db][3]);
        }
    }
    // Ordering.  Hardware (gfx950, which this file is compiled for and nothing else -- see the
    // #error in common.h): the partials above are device-scope atomic stores, i.e. written
    // through to memory, and vmcnt counts a store only once memory has acknowledged it; the
    // merger's device-scope atomic loads are served from memory, not from its XCD's L2.
    // So once vmcnt is zero the partials are visible to every XCD, and the counter's value
    // tells the last slice that every other slice got that far.  Compiler: the two
    // workgroup-scope fences forbid moving the stores below the count and the merger's loads
    // above it; at workgroup scope they cost no cache maintenance (an agent-scope release
    // would write back the whole L2: 121 us per launch, measured).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's partials are in memory before it is counted
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(a.arrive + pair, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    old = __builtin_amdgcn_readfirstlane(old);
    if (old != a.n_split - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (lane == 0) __hip_atomic_store(a.arrive + pair, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    switch (a.n_split) {
        case 2: merge_rows_static<2>(a, pair, b, hk, grp, R, lane); break;
        case 3: merge_rows_static<3>(a, pair, b, hk, grp, R, lane); break;
        case 4: merge_rows_static<4>(a, pair, b, hk, grp, R, lane); break;
        case 5: merge_rows_static<5>(a, pair, b, hk, grp, R, lane); break;
        case 6: merge_rows_static<6>(a, pair, b, hk, grp, R, lane); break;
        case 7: merge_rows_static<7>(a, pair, b, hk, grp, R, lane); break;
        case 8: merge_rows_static<8>(a, pair, b, hk, grp, R, lane); break;
        case 9: merge_rows_static<9>(a, pair, b, hk, grp, R, lane); break;
        case 10: merge_rows_static<10>(a, pair, b, hk, grp, R, lane); break;
        case 11: merge_rows_static<11>(a, pair, b, hk, grp, R, lane); break;
        default: merge_rows_static<12>(a, pair, b, hk, grp, R, lane); break;
    }
}

// ---- Streaming form of the register-direct kernel: many (batch, kv head) pairs with few
// query rows over a long resident prefix (GR00T's cross blocks: 17 rows onto 296 cached keys
// of 48-wide heads, 2048 pairs at batch 64).  The launch is bound by how many cache lines a
// CU keeps in flight, so every request is made a whole line that is used once:
//
//  - K and V^T go from the cache straight into LDS (global_load_lds_dwordx4) in the order
//    they lie in memory: a 32-key block of K is one contiguous run, a 64-key stretch of the
//    V^T rows is one line per row.  Nothing is fetched twice and no request covers part of
//    a line, which the fragment-order register loads of the direct kernel do for V^T.
//  - One wavefront per SIMD owns a private LDS ring (four K blocks, three V^T stretches,
//    one Q tile: 38 KiB) and walks its pairs one after the other.  The ring does not stop
//    at a pair's end: the next pair's first blocks and its query tile are requested while
//    the current pair's last blocks are multiplied, so only the first pair's head and the
//    last pair's tail are exposed.  No barriers: a ring belongs to one wavefront.
//  - Loads complete in order and every step issues the same loads, so "block b has
//    landed" is s_waitcnt vmcnt(24) at every step (the once-per-pair query loads only make
//    that wait cover a little more).  No register is a load target: nothing to keep alive.
//
// LDS rows are 128 bytes (K and Q rows padded from 96), 16-byte pieces XOR-swizzled by
// (row >> 1) & 7: the loading lane picks the global piece that belongs in its slot.  The
// arithmetic per block is the direct kernel's, in the same order: the two give the same bits.
__device__ __forceinline__ void dma16(uint32_t voff, const void* sbase, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(sbase) : "memory");
}
// A wavefront-uniform pointer the compiler may hold in vector registers, moved to scalar ones (the address operand above).
__device__ __forceinline__ const unsigned char* uniform_ptr(const unsigned char* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const unsigned char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
template <int N>
__device__ __forceinline__ void wait_vm_mem() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int D>
__global__ void __launch_bounds__(256, 1) attn_stream_kernel(AttnArgs a, int n_units) {
    constexpr int EB = 2, NQ = D / 16, NDB = (D + 31) / 32, PIECES = D * EB / 16;
    constexpr int KBLK = 32 * 128, VBLK = D * 128, QBUF = 32 * 128, NKS = 4, NVS = 3, NVI = D / 8;
    constexpr int WAVE_LDS = NKS * KBLK + NVS * VBLK + QBUF;
    static_assert(WAVE_LDS % 1024 == 0 && 4 * WAVE_LDS <= 160 * 1024, "four rings per CU");
    static_assert(D % 16 == 0 && D * EB <= 128, "rows of at most 128 bytes");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * WAVE_LDS];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, r = lane & 31;
    const int n_waves = gridDim.x * 4, w = blockIdx.x * 4 + wave;
    if (w >= n_units) return;  // whole wavefront; the kernel has no barriers
    const int n_my = (n_units - w + n_waves - 1) / n_waves;  // pairs w, w + n_waves, ...
    const int grp = a.Hq / a.Hkv, R = grp * a.S;
    const int NBU = 2 * ((a.n_keys + 63) / 64);  // 32-key blocks per pair (whole 64-key stretches)
    const int total = n_my * NBU;

    unsigned char* const wl = lds + wave * WAVE_LDS;
    const uint32_t ldsK = (uint32_t)(uintptr_t)wl, ldsV = ldsK + NKS * KBLK, ldsQ = ldsV + NVS * VBLK;
    const unsigned char* const pK = wl;
    const unsigned char* const pV = wl + NKS * KBLK;
    const unsigned char* const pQ = wl + NKS * KBLK + NVS * VBLK;

    // Loader side: lane i fills slot i % 8 of row i / 8 of each 1 KiB slab.
    const int lrow = lane >> 3, slot = lane & 7;
    uint32_t kvoff[4], vvoff[NVI], qvoff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = 8 * j + lrow;
        int piece = slot ^ ((row >> 1) & 7);
        piece = piece < PIECES ? piece : 0;  // the padding slots of a row repeat its first piece (same line, never read)
        kvoff[j] = (uint32_t)(row * D * EB + piece * 16);
        int rr = min(row, R - 1);  // query rows past R repeat the last one; their outputs are dropped
        qvoff[j] = (uint32_t)((((rr % a.S) * a.Hq + rr / a.S) * D) * EB + piece * 16);
    }
#pragma unroll
    for (int j = 0; j < NVI; ++j) {
        const int d = 8 * j + lrow;
        const int piece = slot ^ ((d >> 1) & 7);
        vvoff[j] = (uint32_t)(d * a.t_max * EB + piece * 16);
    }
    // Issue streams: each keeps its own (pair index, position); past the last pair they repeat its last item.
    int kI_u = 0, kI_b = 0, vI_u = 0, vI_s = 0, qI_u = 0;
    const int NSU = NBU / 2;
    auto pair_of = [&](int ui) { return w + min(ui, n_my - 1) * n_waves; };
    auto issueK = [&](int st) __attribute__((always_inline)) {
        const int pr = pair_of(kI_u), lb = kI_u < n_my ? kI_b : NBU - 1;
        const unsigned char* base = uniform_ptr((const unsigned char*)a.k_cache + ((long)pr * a.t_max + (long)lb * 32) * D * EB);
        // eight-row slabs wholly past n_keys repeat the block's first slab (lines already on their way) instead of
        // fetching rows nobody reads: the load count per block stays the same, the bytes do not
        const int rows_left = a.n_keys - lb * 32;
#pragma unroll
        for (int j = 0; j < 4; ++j) dma16(8 * j < rows_left ? kvoff[j] : kvoff[0], base, ldsK + st * KBLK + j * 1024);
        if (++kI_b == NBU) { kI_b = 0; ++kI_u; }
    };
    auto issueV = [&](int st) __attribute__((always_inline)) {
        const int pr = pair_of(vI_u), ls = vI_u < n_my ? vI_s : NSU - 1;
        const unsigned char* base = uniform_ptr((const unsigned char*)a.vt_cache + (long)pr * D * a.t_max * EB + (long)ls * 128);
#pragma unroll
        for (int j = 0; j < NVI; ++j) dma16(vvoff[j], base, ldsV + st * VBLK + j * 1024);
        if (++vI_s == NSU) { vI_s = 0; ++vI_u; }
    };
    auto issueQ = [&]() __attribute__((always_inline)) {
        const int pr = pair_of(qI_u), b = pr / a.Hkv, hk = pr % a.Hkv;
        const unsigned char* base = uniform_ptr((const unsigned char*)a.q + (((long)b * a.S) * a.Hq + hk * grp) * D * EB);
#pragma unroll
        for (int j = 0; j < 4; ++j) dma16(qvoff[j], base, ldsQ + j * 1024);
        ++qI_u;
    };

    // Consumer side (the direct kernel's fragments): score row r of a block is key
    // key_of_score_row(r); V^T row d = 32 db + r (rows past D repeat row D - 1, outputs dropped).
    const int krow = key_of_score_row(r);
    const int kfrag = krow * 128, ksw = (krow >> 1) & 7;
    int vfrag[NDB], vsw[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        const int d = min(db * 32 + r, D - 1);
        vfrag[db] = d * 128;
        vsw[db] = (d >> 1) & 7;
    }
    const int qfrag = r * 128, qsw = (r >> 1) & 7;

    u32x4_t qf[NQ];
    f32x16_t o[NDB];
    float m_run = -INFINITY, l_run = 0.f;
    constexpr float LOG2E = 1.4426950408889634f;
    const float c2 = a.scale * LOG2E;
    auto reset = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
        m_run = -INFINITY;
        l_run = 0.f;
    };
    reset();

    auto compute = [&](int kst, int vst, int half, int k0) __attribute__((always_inline)) {
        const unsigned char* kb = pK + kst * KBLK + kfrag;
        u32x4_t kr[NQ];
#pragma unroll
        for (int c = 0; c < NQ; ++c) kr[c] = *reinterpret_cast<const u32x4_t*>(kb + (((2 * c + g) ^ ksw) * 16));
        u32x4_t vr[NDB][2];
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
#pragma unroll
            for (int db = 0; db < NDB; ++db)
                vr[db][hh] = *reinterpret_cast<const u32x4_t*>(pV + vst * VBLK + vfrag[db] + (((half * 4 + hh * 2 + g) ^ vsw[db]) * 16));
        f32x16_t sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NQ; ++c) AT<bf16_t>::mma(sc, kr[c], qf[c]);
        float p[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i] = sc[i] * c2;
        if (k0 + 32 > a.n_keys) {  // uniform: the pair's last blocks; stale cache contents past n_keys must not reach the sums
            const int kl = k0 + 8 * g;
#pragma unroll
            for (int e = 0; e < 16; ++e) p[e] = (kl + key_of_element(e, 0) < a.n_keys) ? p[e] : -INFINITY;
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int nvalid = a.n_keys - (k0 + hh * 16 + 8 * g);
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        vr[db][hh][e] &= (2 * e < nvalid ? 0xffffu : 0u) | (2 * e + 1 < nvalid ? 0xffff0000u : 0u);
            }
        }
        float m_blk = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) m_blk = fmaxf(m_blk, p[i]);
        m_blk = halves_max(m_blk);
        if (__builtin_amdgcn_ballot_w64(m_blk > m_run + RESCALE_LOG2) != 0) {  // lazy reference update
            const float m_new = fmaxf(m_run, m_blk);
            const float alpha = __builtin_amdgcn_exp2f(m_run - ((m_new == -INFINITY) ? 0.f : m_new));
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            p[i] = __builtin_amdgcn_exp2f(p[i] - m_use);
            psum += p[i];
        }
        psum = halves_sum(psum);
        l_run += psum;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const float* pp = &p[hh * 8];
            u32x4_t pf;
#pragma unroll
            for (int e = 0; e < 4; ++e) pf[e] = pack_bf2(pp[2 * e], pp[2 * e + 1]);
#pragma unroll
            for (int db = 0; db < NDB; ++db) AT<bf16_t>::mma(o[db], vr[db][hh], pf);
        }
    };

    // Prologue: the issue order of the steps before the first (Q, then V stretch, K block, K block, ...).
    issueQ();
    issueV(0);
    issueK(0);
    issueK(1);
    issueV(1);
    issueK(2);
    issueK(3);
    issueV(2);
    // At step b the youngest load needed is K block b, issued at the end of step b - 4.  Younger than it:
    // three K blocks (12 loads) and two V^T stretches (2 NVI), whichever the parity of b.
    constexpr int YOUNGER = 12 + 2 * NVI;
    int lb = 0, ui = 0, kst = 0, vst = 0;
    for (int gb = 0; gb < total; gb += 2) {
        wait_vm_mem<YOUNGER>();
        if (lb == 0) {  // uniform: a pair begins
#pragma unroll
            for (int c = 0; c < NQ; ++c) qf[c] = *reinterpret_cast<const u32x4_t*>(pQ + qfrag + (((2 * c + g) ^ qsw) * 16));
            // the next pair's query tile: the data lands long after the reads above have left the LDS pipeline
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            issueQ();
        }
        compute(kst, vst, 0, lb * 32);
        issueK(kst);
        kst = (kst + 1) & 3;
        wait_vm_mem<YOUNGER>();
        compute(kst, vst, 1, lb * 32 + 32);
        issueK(kst);
        kst = (kst + 1) & 3;
        issueV(vst);
        vst = vst == NVS - 1 ? 0 : vst + 1;
        lb += 2;
        if (lb == NBU) {  // uniform: the pair is complete
            const int pr = w + ui * n_waves, b = pr / a.Hkv, hk = pr % a.Hkv;
            if (r < R) {
                const int hg = r / a.S, s = r % a.S, h = hk * grp + hg;
                const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
                unsigned char* orow = (unsigned char*)a.out + (((long)b * a.S + s) * a.Hq + h) * D * EB;
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int d = db * 32 + 8 * j + 4 * g;
                        if (d >= D) continue;
                        const u32x2_t pk = {pack_bf2(o[db][4 * j] * inv, o[db][4 * j + 1] * inv),
                                            pack_bf2(o[db][4 * j + 2] * inv, o[db][4 * j + 3] * inv)};
                        *reinterpret_cast<u32x2_t*>(orow + d * EB) = pk;
                    }
            }
            reset();
            lb = 0;
            ++ui;
        }
    }
    wait_vm_mem<0>();  // the ring's trailing loads still target this wavefront's LDS
}

// Merge of key-split partials as a launch of its own: one wavefront per (pair, row).
template <typename T, bool HALF>
__global__ void __launch_bounds__(256) attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                         T* __restrict__ out, int n_pairs, int n_split, int r_pad, int R, int S,
                                                         int Hq, int Hkv, int D, DivC dR, DivC dHkv, DivC dS) {
    const int lane = threadIdx.x & 63;
    const int ridx = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (ridx >= n_pairs * R) return;  // whole wavefront
    const int pair = (int)div_c(ridx, dR), row = ridx - pair * R;
    const int grp = Hq / Hkv, b = (int)div_c(pair, dHkv), hk = pair - b * Hkv;
    const int hs = (int)div_c(row, dS);
    const int h = hk * grp + hs, s = row - hs * S;
    T* orow = out + (((long)b * S + s) * Hq + h) * D;
    const long prow0 = (long)pair * n_split * r_pad + row;
    switch (n_split) {  // wavefront-uniform
        case 2: merge_row_static<T, HALF, 2>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 3: merge_row_static<T, HALF, 3>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 4: merge_row_static<T, HALF, 4>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 5: merge_row_static<T, HALF, 5>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 6: merge_row_static<T, HALF, 6>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 7: merge_row_static<T, HALF, 7>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 8: merge_row_static<T, HALF, 8>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 9: merge_row_static<T, HALF, 9>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 10: merge_row_static<T, HALF, 10>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 11: merge_row_static<T, HALF, 11>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 12: merge_row_static<T, HALF, 12>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 13: merge_row_static<T, HALF, 13>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 14: merge_row_static<T, HALF, 14>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 15: merge_row_static<T, HALF, 15>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        case 16: merge_row_static<T, HALF, 16>(part_o, part_ml, orow, prow0, r_pad, D, lane); break;
        default: merge_row<T, HALF>(part_o, part_ml, orow, prow0, n_split, r_pad, D, lane); break;
    }
}

// ---- scratch memory of a call ---------------------------------------------------------
// Shapes whose keys are sliced across workgroups need device memory beyond the inputs and
// outputs: the slices' partial (max, sum, output) rows and, for the in-launch merge, one
// arrival counter per (pair, row block).  One block holds both:
//     [0, ARRIVE_BYTES)      int counters, zero between launches (a new block is zero-filled,
//                            every launch that uses them leaves them at zero)
//     [ARRIVE_BYTES, ...)    partials, rows x (D + 2) floats
// It comes from the library's per-stream blocks (vla_attn_prefix_suffix), from the caller
// (vla_attn_prefix_suffix_ws) or from a static device array (vla_attn_prefix_suffix_noalloc);
// a dry run only reports the size (vla_attn_workspace_bytes).
constexpr size_t ARRIVE_BYTES = (size_t)ARRIVE_MAX_UNITS * sizeof(int);
struct Scratch {
    enum Kind { LIBRARY, CALLER, DRY };
    Kind kind = LIBRARY;
    unsigned char* base = nullptr;  // CALLER: the block handed in
    size_t bytes = 0;
    size_t need = 0;  // bytes the shape asked for (every kind)
};
size_t scratch_bytes(size_t rows, int D) { return ARRIVE_BYTES + (rows * (size_t)(D + 2) * sizeof(float) + 255) / 256 * 256; }

// Binds the partial rows (and the counters) of a sliced call.  Returns VLA_K_OK with
// a.part_o == nullptr on a dry run: the caller then returns without launching.
int bind_scratch(AttnArgs& a, Scratch& sc, hipStream_t st, size_t rows, int D) {
    sc.need = scratch_bytes(rows, D);
    a.part_o = nullptr;
    if (sc.kind == Scratch::DRY) return VLA_K_OK;
    unsigned char* base = sc.base;
    if (sc.kind == Scratch::LIBRARY) {
        base = (unsigned char*)stream_scratch(SCRATCH_ATTN, st, sc.need);
        if (!base) return VLA_K_ERR_LAUNCH;
    } else if (!base || sc.bytes < sc.need || ((uintptr_t)base & 15)) {
        return VLA_K_ERR_WORKSPACE;
    }
    a.arrive = reinterpret_cast<int*>(base);
    a.part_o = reinterpret_cast<float*>(base + ARRIVE_BYTES);
    a.part_ml = a.part_o + rows * D;
    return VLA_K_OK;
}

// Second launch of a key-split LDS-kernel call: combines the workgroups' partials.
template <typename T, int D>
int launch_merge(AttnArgs& a, hipStream_t st) {
    if (a.n_split > 1) {
        const int n_pairs = a.batch * a.Hkv;
        const int R = (a.Hq / a.Hkv) * a.S;
        const unsigned mgrid = (unsigned)(((long)n_pairs * R + 3) / 4);
        const long mx = (long)n_pairs * R + 4;
        const DivC dR = make_divc(R, mx), dHkv = make_divc(a.Hkv, mx), dS = make_divc(a.S, mx);
        if (a.part_half)
            attn_merge_kernel<T, true><<<mgrid, 256, 0, st>>>(a.part_o, a.part_ml, (T*)a.out, n_pairs, a.n_split, a.r_pad, R, a.S, a.Hq, a.Hkv, D, dR, dHkv, dS);
        else
            attn_merge_kernel<T, false><<<mgrid, 256, 0, st>>>(a.part_o, a.part_ml, (T*)a.out, n_pairs, a.n_split, a.r_pad, R, a.S, a.Hq, a.Hkv, D, dR, dHkv, dS);
        if (hipGetLastError() != hipSuccess) return VLA_K_ERR_LAUNCH;
    }
    return VLA_K_OK;
}

template <typename T, int D, int NW>
int launch_nw(AttnArgs& a, hipStream_t st) {
    const int n_pairs = a.batch * a.Hkv;
    const int grid = (n_pairs + 7) / 8 * 8 * a.n_groups * a.n_split;
    set_divisors(a, grid);
    if constexpr (sizeof(T) == 2 && D == 64) {
        // 64-wide bf16 heads: tiles go straight into a swizzled LDS ring (the tuning override
        // attn_dl = 0 pins the register-staged path), and with three or more key tiles they
        // are split over two wavefronts per row tile (attn_slices = 1 | 2 overrides).  The
        // kernel also builds for 128-wide heads, where its register use makes it the slower choice.
        if (tuning().attn_dl != 0) {
            const int nsl = a.n_slices;
            if constexpr (D == 64 && NW <= 2) {
                if (nsl == 2) {
                    if (a.p2) attn_kernel<T, D, NW, true, 0, 2, 2><<<grid, NW * 128, 0, st>>>(a);
                    else attn_kernel<T, D, NW, false, 0, 2, 2><<<grid, NW * 128, 0, st>>>(a);
                }
            }
            if (nsl == 2 && !(D == 64 && NW <= 2)) return VLA_K_ERR_SHAPE;  // launch_d never asks for this
            if (nsl == 1) {
                if (a.p2) attn_kernel<T, D, NW, true, 0, 1, 3><<<grid, NW * 64, 0, st>>>(a);
                else attn_kernel<T, D, NW, false, 0, 1, 3><<<grid, NW * 64, 0, st>>>(a);
            }
            if (hipGetLastError() != hipSuccess) return VLA_K_ERR_LAUNCH;
            return launch_merge<T, D>(a, st);
        }
    }
    if constexpr (sizeof(T) == 2) {
        // Wide heads: four loader wavefronts.  Narrow heads prefetch in registers instead
        // (with loader wavefronts a batch-32 SmolVLA launch no longer fits the chip in one round).
        constexpr int NL = (D * sizeof(T) >= 512) ? 4 : 0;
        if (a.p2) attn_kernel<T, D, NW, true, NL><<<grid, (NW + NL) * 64, 0, st>>>(a);
        else attn_kernel<T, D, NW, false, NL><<<grid, (NW + NL) * 64, 0, st>>>(a);
    } else {
        attn_kernel<T, D, NW, false, 0><<<grid, NW * 64, 0, st>>>(a);
    }
    if (hipGetLastError() != hipSuccess) return VLA_K_ERR_LAUNCH;
    return launch_merge<T, D>(a, st);
}

template <int D>
int launch_direct(AttnArgs& a, hipStream_t st, Scratch& sc) {
    constexpr int ST = D <= 64 ? 3 : 2;
    const Tuning& tn = tuning();
    const int n_pairs = a.batch * a.Hkv;
    const int R = (a.Hq / a.Hkv) * a.S;
    if constexpr (D == 48) {
        // Enough pairs for every SIMD to walk at least one, keys in whole 64-key stretches inside the cache rows, nothing
        // masked: the streaming form (the same bits as the kernel below).
        if (!a.p2 && R <= 32 && n_pairs >= 1024 && a.n_keys >= 128 && a.t_max % 64 == 0 && a.mask == nullptr &&
            a.mask_kind == VLA_MASK_NONE && a.pad_start >= a.pad_end && !tn.attn_no_stream && sc.kind != Scratch::DRY) {
            // (a dry run does not know the cache rows' length: it sizes for the kernel below, which needs at least as much)
            a.n_rblocks = 1;
            a.n_split = 1;
            const unsigned grid = (unsigned)std::min(256, (n_pairs + 3) / 4);
            attn_stream_kernel<D><<<grid, 256, 0, st>>>(a, n_pairs);
            return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
        }
    }
    a.n_rblocks = (R + 31) / 32;
    const int n_units = n_pairs * a.n_rblocks;  // (pair, 32-row block)
    const int nb_total = (a.n_keys + 31) / 32;
    // Enough wavefronts to keep every CU's memory pipeline busy (8 per CU); a slice is
    // at least two 32-key blocks unless the whole sequence is shorter.
    int n_split = 1;
    if (n_units < 2048) n_split = (2048 + n_units - 1) / n_units;
    if (n_split > (nb_total + 1) / 2) n_split = (nb_total + 1) / 2;
    if (n_split < 1) n_split = 1;
    if (tn.attn_split_set) n_split = tn.attn_split > 0 ? (tn.attn_split < nb_total ? tn.attn_split : nb_total) : 1;
    // Slices of one pair as the wavefronts of one workgroup (merged through LDS, one launch)
    // when few enough; with fewer than 32 pairs more slices go through global partials and
    // the merge kernel instead.
    constexpr int MERGE_MAX = D <= 64 ? 8 : 4;  // wide heads need the registers of a 4-wavefront workgroup
    bool wg_merge = n_split > 1 && (n_split <= MERGE_MAX || n_units >= 32);
    // 128-wide heads with at most 16 rows (single-token decode): more slices than one workgroup
    // holds, as single-wavefront workgroups over more CUs, merged by the slice that arrives last
    // (attn_decode16_kernel).  Slices of three blocks there, all of their loads requested at
    // once: each slice costs the merging wavefront a row of loads, and the hand-over is three
    // dependent trips to memory whatever the count.
    const int Rb = R < 32 ? R : 32;
    int n_arrive = n_split < (nb_total + 2) / 3 || tn.attn_split_set ? n_split : (nb_total + 2) / 3;
    if (n_arrive > DEC_MAX_NS) n_arrive = DEC_MAX_NS;
    if (n_arrive * Rb > ARRIVE_MAX_T) n_arrive = ARRIVE_MAX_T / Rb;
    bool arrive = D == 128 && R <= DEC_MAX_R && n_arrive > MERGE_MAX && a.n_rblocks == 1 && n_units <= ARRIVE_MAX_UNITS && !tn.attn_no_arrive;
    if (arrive) {
        n_split = n_arrive;
        wg_merge = false;
    }
    if (wg_merge && n_split > MERGE_MAX) n_split = MERGE_MAX;
    a.tiles_per_split = (nb_total + n_split - 1) / n_split;
    a.n_split = (nb_total + a.tiles_per_split - 1) / a.tiles_per_split;
    a.r_pad = a.n_rblocks * 32;
    a.n_groups = 1;
    a.arrive = nullptr;
    if (wg_merge && a.n_split > 1) {
        const size_t lds = (size_t)a.n_split * (R < 32 ? R : 32) * (D + 2) * sizeof(float);  // at most 8 * 32 * 66 * 4 or 4 * 32 * 130 * 4 = 66 KB
        if (lds <= 64 * 1024) {
            if (sc.kind == Scratch::DRY) return VLA_K_OK;
            if (a.p2) attn_direct_kernel<D, true, ST, true><<<n_units, a.n_split * 64, lds, st>>>(a);
            else attn_direct_kernel<D, false, ST, true><<<n_units, a.n_split * 64, lds, st>>>(a);
            return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
        }
    }
    if (a.n_split > 1) {
        const int rc = bind_scratch(a, sc, st, (size_t)n_pairs * a.n_split * a.r_pad, D);
        if (rc != VLA_K_OK) return rc;
    }
    if (sc.kind == Scratch::DRY) return VLA_K_OK;
    arrive = arrive && a.n_split > 1 && a.n_split <= DEC_MAX_NS && a.n_split * Rb <= ARRIVE_MAX_T;
    if (!arrive) a.arrive = nullptr;
    if constexpr (D == 128) {
        if (arrive) {  // a wavefront per (pair, slice)
            const unsigned grid16 = (unsigned)(n_units * a.n_split);
            if (a.p2) attn_decode16_kernel<true, 3><<<grid16, 64, 0, st>>>(a);
            else attn_decode16_kernel<false, 3><<<grid16, 64, 0, st>>>(a);
            return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
        }
    }
    const int wgw = 4;  // wavefronts per workgroup
    const unsigned grid = (unsigned)(((long)n_units * a.n_split + wgw - 1) / wgw);
    if (a.p2) attn_direct_kernel<D, true, ST, false><<<grid, wgw * 64, 0, st>>>(a);
    else attn_direct_kernel<D, false, ST, false><<<grid, wgw * 64, 0, st>>>(a);
    if (hipGetLastError() != hipSuccess) return VLA_K_ERR_LAUNCH;
    if (a.n_split > 1) {
        const long mx = (long)n_pairs * R + 4;
        attn_merge_kernel<bf16_t, false><<<(unsigned)(((long)n_pairs * R + 3) / 4), 256, 0, st>>>(a.part_o, a.part_ml, (bf16_t*)a.out,
                                                                                           n_pairs, a.n_split, a.r_pad, R, a.S, a.Hq,
                                                                                           a.Hkv, D, make_divc(R, mx), make_divc(a.Hkv, mx),
                                                                                           make_divc(a.S, mx));
        if (hipGetLastError() != hipSuccess) return VLA_K_ERR_LAUNCH;
    }
    return VLA_K_OK;
}

template <typename T, int D>
int launch_d(AttnArgs& a, vla_stream_t stream, Scratch& sc) {
    const Tuning& tn = tuning();
    hipStream_t st = (hipStream_t)stream;
    const int R = (a.Hq / a.Hkv) * a.S;
    if constexpr (sizeof(T) == 2 && D <= 128) {
        // At most attn_direct_rows (32) rows per kv head: the register-direct kernel.  With more
        // rows, 16-byte runs per key row cost more than sharing tiles through LDS saves.
        if (R <= tn.attn_direct_rows && !tn.attn_no_direct) return launch_direct<D>(a, st, sc);
    }
    const int n_tiles = (R + 31) / 32;
    // 64-wide bf16 heads with three or more key tiles: two key slices per row tile (the
    // direct-to-LDS variant of the kernel).  Two wavefronts per row tile then, and at most
    // two row tiles per workgroup, so that a batch-32 launch stays resident at once (two
    // 4-wavefront workgroups per CU).
    a.n_slices = 1;
    if constexpr (sizeof(T) == 2 && D == 64) {
        if (tn.attn_dl != 0) {
            a.n_slices = (a.n_keys + SPLIT_KEYS - 1) / SPLIT_KEYS >= 3 ? 2 : 1;
            if (tn.attn_slices) a.n_slices = tn.attn_slices == 2 ? 2 : 1;
        }
    }
    // One wavefront (per slice) per row tile, at most one wavefront of a workgroup per SIMD;
    // more row tiles than that are spread evenly over groups.
    const int NW_MAX = a.n_slices == 2 ? 2 : 4;
    a.n_groups = (n_tiles + NW_MAX - 1) / NW_MAX;
    const int nw = (n_tiles + a.n_groups - 1) / a.n_groups;
    a.r_pad = a.n_groups * nw * 32;
    // Too few workgroups to cover the 256 compute units: split the keys as well.
    const long wgs = (long)a.batch * a.Hkv * a.n_groups;
    const int key_tiles = (a.n_keys + SPLIT_KEYS - 1) / SPLIT_KEYS;
    a.n_split = 1;
    // Only worthwhile while a partial (r_pad rows of D+2 floats) stays small next to the
    // K/V slice it summarises; with many query rows the partials would outweigh the cache.
    const size_t partial_bytes = (size_t)a.r_pad * (D + 2) * 4, tile_bytes = (size_t)2 * SPLIT_KEYS * D * sizeof(T);
    // fp32 launches with few row tiles in all (batch 1) also split while the partials of the
    // whole launch stay within a few MiB: a key tile takes such a launch about 6 us, whatever
    // it shares, so the serial walk over the keys is its whole cost and the partials are noise
    // (SmolVLA's single fp32 layer at batch 1: 31 -> 15 us with the merge pass).  The bf16
    // kernels walk a tile in 2 us and lose more to the merge launch than they gain.
    const bool cheap = sizeof(T) == 4 && (long)a.batch * a.Hkv * n_tiles <= 64 && !tn.attn_no_small &&
                       (size_t)a.batch * a.Hkv * partial_bytes * (size_t)(key_tiles < 32 ? key_tiles : 32) <= ((size_t)4 << 20);
    if (wgs < 256 && key_tiles > 1 && (partial_bytes <= tile_bytes || cheap)) {
        int want = (int)((512 + wgs - 1) / wgs);
        if (want > key_tiles) want = key_tiles;
        if (want > 32) want = 32;
        a.n_split = want;
    } else if (D * sizeof(T) >= 512 && wgs <= 128 && key_tiles >= 4) {
        // Wide heads (pi0's 256): a workgroup spends ~2.7 us per key tile whatever the batch, so
        // a 14-tile walk costs 40 us on a quarter of the chip.  Slices of at least two tiles,
        // as many as still fit the chip in one round; the partial outputs travel as fp16
        // (normalised per slice: 1.7 MB per slice at batch 16) and the merge pass costs less
        // than the tiles it removes from the critical path.
        int want = (int)(256 / wgs);
        if (want > key_tiles / 2) want = key_tiles / 2;
        if (want >= 2) {
            a.n_split = want;
            a.part_half = (tn.attn_part_f32 || sizeof(T) != 2) ? 0 : 1;
        }
    }
    if (tn.attn_split_set) a.n_split = tn.attn_split > 0 ? (tn.attn_split < key_tiles ? tn.attn_split : key_tiles) : 1;
    a.tiles_per_split = (key_tiles + a.n_split - 1) / a.n_split;
    a.n_split = (key_tiles + a.tiles_per_split - 1) / a.tiles_per_split;  // no empty slices
    if (a.n_split > 1) {
        const int rc = bind_scratch(a, sc, st, (size_t)a.batch * a.Hkv * a.n_split * a.r_pad, D);
        if (rc != VLA_K_OK) return rc;
    }
    if (sc.kind == Scratch::DRY) return VLA_K_OK;
    a.arrive = nullptr;
    switch (nw) {
        case 1: return launch_nw<T, D, 1>(a, st);
        case 2: return launch_nw<T, D, 2>(a, st);
        case 3: return launch_nw<T, D, 3>(a, st);
        case 4: return launch_nw<T, D, 4>(a, st);
        default: break;
    }
    return VLA_K_ERR_SHAPE;
}


// fp32 attention for 256-wide heads (pi0's default activation type in the reference is F32,
// src/models/pi0.cpp:90, 174-176).  The MFMA kernel's fp32 tiles of such heads exceed the
// static LDS budget and its accumulators the register file, and this case is about matching
// the reference's precision, not about speed: a plain FMA kernel.  A workgroup (256 threads)
// owns WR query rows of one (batch, query head): pass 1, thread t forms the scores of keys
// t, t + 256, ... against the WR rows (its K row streamed once for all of them); exact
// two-pass softmax per row over the scores kept in LDS; pass 2, thread d accumulates output
// column d over V^T tiles of 16 keys staged in LDS.  fp32 throughout, keys added in order.
constexpr int WIDE_D = 256, WIDE_R = 8, WIDE_VK = 16, WIDE_MAX_KEYS = 1152;
__global__ void __launch_bounds__(256) attn_f32_wide_kernel(AttnArgs a) {
    __shared__ float qs[WIDE_R][WIDE_D];
    __shared__ float sc[WIDE_R][WIDE_MAX_KEYS];
    __shared__ float vt[WIDE_D][WIDE_VK + 1];
    __shared__ float red[16];
    const int tid = threadIdx.x;
    const int n_rt = (a.S + WIDE_R - 1) / WIDE_R;
    const int rt = blockIdx.x % n_rt, bh = blockIdx.x / n_rt;
    const int h = bh % a.Hq, b = bh / a.Hq;
    const int hk = h / (a.Hq / a.Hkv);
    const int s0 = rt * WIDE_R, nr = min(WIDE_R, a.S - s0);
    const float* kbase = (const float*)a.k_cache + ((long)b * a.Hkv + hk) * a.t_max * WIDE_D;
    const float* vbase = (const float*)a.vt_cache + ((long)b * a.Hkv + hk) * WIDE_D * (long)a.t_max;
    for (int i = tid; i < WIDE_R * WIDE_D; i += 256) {
        const int r = i / WIDE_D, d = i % WIDE_D;
        qs[r][d] = r < nr ? ((const float*)a.q)[(((long)b * a.S + s0 + r) * a.Hq + h) * WIDE_D + d] : 0.f;
    }
    __syncthreads();
    const int pad_lo = a.pad_start, pad_hi = min(a.pad_end, a.n_prefix);
    for (int key = tid; key < a.n_keys; key += 256) {
        float acc[WIDE_R];
#pragma unroll
        for (int r = 0; r < WIDE_R; ++r) acc[r] = 0.f;
        const f32x4_t* kr = reinterpret_cast<const f32x4_t*>(kbase + (long)key * WIDE_D);
        for (int d4 = 0; d4 < WIDE_D / 4; ++d4) {
            const f32x4_t kv = kr[d4];
#pragma unroll
            for (int r = 0; r < WIDE_R; ++r) {
                const f32x4_t qv = *reinterpret_cast<const f32x4_t*>(&qs[r][d4 * 4]);
                acc[r] = fmaf(kv[0], qv[0], acc[r]);
                acc[r] = fmaf(kv[1], qv[1], acc[r]);
                acc[r] = fmaf(kv[2], qv[2], acc[r]);
                acc[r] = fmaf(kv[3], qv[3], acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < WIDE_R; ++r) {
            const int s = s0 + r;
            float v = acc[r] * a.scale;
            if (a.mask) {
                v += r < nr ? a.mask[(long)s * a.n_keys + key] : 0.f;
            } else {
                int hi = a.n_keys;
                if (a.mask_kind == VLA_MASK_CAUSAL_SUFFIX) hi = min(a.n_keys, a.n_prefix + s + 1);
                else if (a.mask_kind == VLA_MASK_PI0_STATE && s == 0) hi = min(a.n_keys, a.n_prefix + 1);
                if (!(key < hi) || (key >= pad_lo && key < pad_hi)) v = -INFINITY;
            }
            sc[r][key] = v;
        }
    }
    __syncthreads();
    // softmax per row: max, exp, sum (ggml_soft_max_ext's order, src/layers/attn.h:43)
    float inv[WIDE_R];
    for (int r = 0; r < WIDE_R; ++r) {
        float m = -INFINITY;
        for (int key = tid; key < a.n_keys; key += 256) m = fmaxf(m, sc[r][key]);
        m = block_max(m, red);
        float sum = 0.f;
        for (int key = tid; key < a.n_keys; key += 256) {
            const float e = m == -INFINITY ? 0.f : expf(sc[r][key] - m);
            sc[r][key] = e;
            sum += e;
        }
        sum = block_sum(sum, red);
        inv[r] = sum > 0.f ? 1.0f / sum : 0.f;
    }
    __syncthreads();
    float o[WIDE_R];
#pragma unroll
    for (int r = 0; r < WIDE_R; ++r) o[r] = 0.f;
    for (int k0 = 0; k0 < a.n_keys; k0 += WIDE_VK) {
        __syncthreads();
        for (int i = tid; i < WIDE_D * WIDE_VK; i += 256) {
            const int d = i / WIDE_VK, kk = i % WIDE_VK;
            vt[d][kk] = k0 + kk < a.n_keys ? vbase[(long)d * a.t_max + k0 + kk] : 0.f;
        }
        __syncthreads();
        const int nk = min(WIDE_VK, a.n_keys - k0);
        for (int kk = 0; kk < nk; ++kk) {
            const float v = vt[tid][kk];
#pragma unroll
            for (int r = 0; r < WIDE_R; ++r) o[r] = fmaf(sc[r][k0 + kk], v, o[r]);
        }
    }
    for (int r = 0; r < nr; ++r)
        ((float*)a.out)[(((long)b * a.S + s0 + r) * a.Hq + h) * WIDE_D + tid] = o[r] * inv[r];
}

int launch_f32_wide(AttnArgs& a, hipStream_t st, Scratch& sc) {
    if (a.n_keys > WIDE_MAX_KEYS) return VLA_K_ERR_SHAPE;
    if (sc.kind == Scratch::DRY) return VLA_K_OK;
    const unsigned grid = (unsigned)((long)a.batch * a.Hq * ((a.S + WIDE_R - 1) / WIDE_R));
    attn_f32_wide_kernel<<<grid, 256, 0, st>>>(a);
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

template <typename T>
int launch_t(AttnArgs& a, int D, vla_stream_t stream, Scratch& sc) {
    switch (D) {
        case 48: return launch_d<T, 48>(a, stream, sc);
        case 64: return launch_d<T, 64>(a, stream, sc);
        case 128: return launch_d<T, 128>(a, stream, sc);
        case 256:
            if constexpr (sizeof(T) == 2) return launch_d<T, 256>(a, stream, sc);
            else return launch_f32_wide(a, (hipStream_t)stream, sc);  // its own kernel, see there
        default: return VLA_K_ERR_SHAPE;
    }
}

int attn_entry(const void* q, const void* k_cache, const void* vt_cache, void* out, int dtype, int batch, int S, int n_q_heads,
               int n_kv_heads, int head_dim, int t_max, int n_keys, float scale, int mask_kind, int n_prefix, int pad_start,
               int pad_end, const float* mask, vla_stream_t stream, Scratch& sc) {
    const bool dry = sc.kind == Scratch::DRY;
    if ((!dry && (!q || !k_cache || !vt_cache || !out)) || batch < 0 || S <= 0 || n_q_heads <= 0 || n_kv_heads <= 0)
        return VLA_K_ERR_ARG;
    if (n_q_heads % n_kv_heads || t_max % 8 || n_keys <= 0 || n_keys > t_max) return VLA_K_ERR_SHAPE;
    if (mask_kind < VLA_MASK_NONE || mask_kind > VLA_MASK_PI0_STATE) return VLA_K_ERR_ARG;
    if (batch == 0) return VLA_K_OK;
    AttnArgs a = {};
    a.q = q; a.k_cache = k_cache; a.vt_cache = vt_cache; a.out = out;
    a.batch = batch; a.S = S; a.Hq = n_q_heads; a.Hkv = n_kv_heads; a.t_max = t_max; a.n_keys = n_keys;
    a.scale = scale; a.mask_kind = mask_kind;
    a.n_prefix = n_prefix < 0 ? 0 : (n_prefix > n_keys ? n_keys : n_prefix);
    a.pad_start = pad_start; a.pad_end = pad_end; a.mask = mask;
    a.p2 = dtype == VLA_DT_BF16_P2;
    if (dtype == VLA_DT_BF16 || dtype == VLA_DT_BF16_P2) return launch_t<bf16_t>(a, head_dim, stream, sc);
    if (dtype == VLA_DT_F32) return launch_t<float>(a, head_dim, stream, sc);
    return VLA_K_ERR_ARG;
}

}  // namespace

// The no-allocation entry point's scratch: the block a sliced call needs, as a static device
// array (zero-initialised when the code object is loaded; every GPU the library runs on holds
// its own copy until the process ends).  In host code the name is only a handle for
// hipGetSymbolAddress: the address kernels and copies use is looked up once per device.
static __device__ __align__(256) unsigned char scratch[VLA_ATTN_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
unsigned char* g_scratch_ptr[MAX_DEVICES] = {};
std::mutex g_scratch_ptr_mu;

// The current device's copy of `scratch`, looked up on first use with that device current.
int noalloc_scratch(unsigned char** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return VLA_K_ERR_LAUNCH;
    std::lock_guard<std::mutex> lk(g_scratch_ptr_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return VLA_K_ERR_LAUNCH;
        g_scratch_ptr[dev] = (unsigned char*)p;
    }
    *out = g_scratch_ptr[dev];
    return VLA_K_OK;
}
}  // namespace

extern "C" int vla_attn_prefix_suffix(const void* q, const void* k_cache, const void* vt_cache, void* out, int dtype,
                                      int batch, int S, int n_q_heads, int n_kv_heads, int head_dim, int t_max,
                                      int n_keys, float scale, int mask_kind, int n_prefix, int pad_start, int pad_end,
                                      const float* mask, vla_stream_t stream) {
    Scratch sc;
    sc.kind = Scratch::LIBRARY;
    return attn_entry(q, k_cache, vt_cache, out, dtype, batch, S, n_q_heads, n_kv_heads, head_dim, t_max, n_keys, scale,
                      mask_kind, n_prefix, pad_start, pad_end, mask, stream, sc);
}

extern "C" size_t vla_attn_workspace_bytes(int dtype, int batch, int S, int n_q_heads, int n_kv_heads, int head_dim,
                                           int n_keys) {
    Scratch sc;
    sc.kind = Scratch::DRY;
    const int t_max = (n_keys + 7) / 8 * 8;
    const int rc = attn_entry(nullptr, nullptr, nullptr, nullptr, dtype, batch, S, n_q_heads, n_kv_heads, head_dim, t_max,
                              n_keys, 1.0f, VLA_MASK_NONE, 0, 0, 0, nullptr, nullptr, sc);
    return rc == VLA_K_OK ? sc.need : VLA_ATTN_WORKSPACE_UNSUPPORTED;
}

extern "C" int vla_attn_prefix_suffix_ws(const void* q, const void* k_cache, const void* vt_cache, void* out, int dtype,
                                         int batch, int S, int n_q_heads, int n_kv_heads, int head_dim, int t_max,
                                         int n_keys, float scale, int mask_kind, int n_prefix, int pad_start,
                                         int pad_end, const float* mask, void* workspace, size_t workspace_bytes,
                                         vla_stream_t stream) {
    Scratch sc;
    sc.kind = Scratch::CALLER;
    sc.base = (unsigned char*)workspace;
    sc.bytes = workspace ? workspace_bytes : 0;
    return attn_entry(q, k_cache, vt_cache, out, dtype, batch, S, n_q_heads, n_kv_heads, head_dim, t_max, n_keys, scale,
                      mask_kind, n_prefix, pad_start, pad_end, mask, stream, sc);
}

extern "C" int vla_attn_prefix_suffix_noalloc(const void* q, const void* k_cache, const void* vt_cache, void* out,
                                              int dtype, int batch, int S, int n_q_heads, int n_kv_heads, int head_dim,
                                              int t_max, int n_keys, float scale, int mask_kind, int n_prefix,
                                              int pad_start, int pad_end, const float* mask, vla_stream_t stream) {
    Scratch sc;
    sc.kind = Scratch::CALLER;
    const int rc = noalloc_scratch(&sc.base);
    if (rc != VLA_K_OK) return rc;
    sc.bytes = VLA_ATTN_NOALLOC_SCRATCH_BYTES;
    return attn_entry(q, k_cache, vt_cache, out, dtype, batch, S, n_q_heads, n_kv_heads, head_dim, t_max, n_keys, scale,
                      mask_kind, n_prefix, pad_start, pad_end, mask, stream, sc);
}

// The arrival counters of a workspace back at zero, as a fill kernel (no memset node under
// graph capture).  A launch that ran to its end leaves them at zero by itself; one that did not
// (a device fault, a reset in the middle of a sequence) leaves the counters of its unfinished
// units at whatever they had reached, and every later launch on that workspace would then take
// the wrong slice for the last one.  Callers that own a workspace run this at the start of
// each launch sequence.
__global__ void __launch_bounds__(256) zero_words_kernel(int* p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}
extern "C" int vla_attn_workspace_reset(void* workspace, size_t workspace_bytes, vla_stream_t stream) {
    if (!workspace || workspace_bytes == 0) return VLA_K_OK;  // a shape that needs none
    if (((uintptr_t)workspace & 15) || workspace_bytes < ARRIVE_BYTES) return VLA_K_ERR_WORKSPACE;
    zero_words_kernel<<<(ARRIVE_MAX_UNITS + 255) / 256, 256, 0, (hipStream_t)stream>>>((int*)workspace, ARRIVE_MAX_UNITS);
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

extern "C" int vla_kernels_init(void) {
    (void)tuning();
    unsigned char* p = nullptr;
    return noalloc_scratch(&p);
}
