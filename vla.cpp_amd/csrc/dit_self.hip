// A DiT self-attention block's front half in one launch: modulated LayerNorm, the Q / K / V
// projections and the attention over the block's own tokens (src/modules/dit_head.cpp:111-125
// with enc = nullptr: adaln -> attn_q / attn_k / attn_v -> attention over the S tokens of the
// observation).  Nothing of it reaches memory but the attention output: the block's K and V
// are used by this attention and by nothing else.
//
// Tiling.  The projection is small next to the chip (GR00T at batch 64: 1088 x 4608 x 1536),
// so what counts is that every CU gets the same share and no CU waits for another launch.
// A workgroup owns OB <= 8 observations (OB S <= 144 rows; 8 observations of 17 tokens = 136 rows)
// and ONE head: the head's 48 query, 48 key and 48 value rows of W, 144 output columns.  At
// batch 64 with 32 heads that is 256 workgroups of identical size, and all operands of the
// attention of its (observation, head) pairs end up in the workgroup's LDS.  Workgroup i runs
// on XCD i % 8 and takes head i % H: an XCD's L2 holds the W rows of a few heads and all of x.
//
// Product.  v_mfma_f32_16x16x32_bf16, 9 x 9 blocks of 16 x 16 over four wavefronts: three of
// them take three block rows each against block columns 0 .. 6 (q, k and the first third of v),
// the fourth all nine block rows against block columns 7 and 8: 21 + 21 + 21 + 18 blocks.  The
// walk lasts as long as the instruction stream of its busiest wavefront (a lone wavefront issues
// an MFMA of this shape every 17 clocks and everything else on top of that); a 2 x 2 split gives
// that one 25 blocks.  Eight wavefronts with smaller shares read each fragment more often: 41
// fragment reads of 1 KiB per 32-k chunk already keep the LDS busy for 250 clocks next to the
// 360 of a wavefront's MFMAs, and 64 reads take longer than the MFMAs.  K is walked in tiles of 64 through a four-stage LDS ring filled by
// global_load_lds_dwordx4 (16 bytes per lane straight into LDS, 128-byte rows, the 16-byte
// piece p of row r kept at position p ^ ((r >> 1) & 7) so that the 16 rows of a fragment read
// cover all banks once), three tiles in flight and one barrier per tile; the fragments of a
// 32-k chunk are read between the MFMAs of the chunk before it.  The LayerNorm is taken
// inside: the launch multiplies raw rows of x by weights that carry (1 + scale)
// (vla_fold_adaln_weight_host), sums each row and its squares from the fragments it multiplies
// anyway, and forms rstd (acc - mean colsum[n]) + bias[n] on the way out.
//
// Attention.  Q, K and V^T of the tile go to LDS as bf16 (the precision the unfused path keeps
// them in).  A wavefront takes whole (observation, head) pairs: scores as S^T = K Q^T with
// v_mfma_f32_16x16x16_bf16, so that a lane ends up with four consecutive keys of one query,
// which is the layout the same instruction wants for P as the left operand of P V; softmax in
// registers (max and sum over the lane's values and the three other lanes of the query, which
// meet through the row-swap instructions).
#include "common.h"

namespace vk {
namespace {

constexpr int FS_D = 48;            // head width this kernel is built for
constexpr int FS_COLS = 3 * FS_D;   // q, k, v columns of one head
constexpr int FS_ROWS = 144;        // rows of x per workgroup (9 blocks of 16)
constexpr int FS_KB = 128;          // bytes of K per staged row (64 bf16)
constexpr int FS_NS = 4;            // ring depth
constexpr int FS_STAGE = (FS_ROWS + FS_COLS) * FS_KB;  // 36 KiB
constexpr int FS_QS = 104;          // bf16 per row of the Q | K tile in LDS (208 bytes: 16 rows start in 16 different banks)
constexpr int FS_VS = 36;           // bf16 per row of a V^T tile: 32 keys and padding (72 bytes)
constexpr int FS_MAX_S = 32;        // tokens per observation: two 16-wide MFMA blocks
constexpr int FS_MAX_OB = 8;        // observations per workgroup (V^T tiles held in LDS)
constexpr int FS_MAX_STAT = 24;     // 64-column tiles of x whose handed-over row sums a row adds up (K <= 1536)

struct SelfArgs {
    const bf16_t* x;
    const bf16_t* W;
    const float* colsum;
    const float* bias;
    bf16_t* out;
    int M, K, S, H, OB;
    float scale, eps;
    const float* stats_in;  // (sum of squares, sum) per (row, 64-column tile of x) from the launch that wrote x, or null
    int n_stat;
};

__device__ __forceinline__ float sum_squares_bf16x2(uint32_t u, float acc) {
    const __bf16 __attribute__((ext_vector_type(2))) v = __builtin_bit_cast(__bf16 __attribute__((ext_vector_type(2))), u);
    return __builtin_amdgcn_fdot2_f32_bf16(v, v, acc, false);
}
__device__ __forceinline__ float sum_pair_bf16x2(uint32_t u, float acc) {
    typedef __bf16 __attribute__((ext_vector_type(2))) bf2_t;
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2_t, u), __builtin_bit_cast(bf2_t, 0x3f803f80u), acc, false);
}

// The K walk of one wavefront: NR x NC blocks, block rows rb0 .. rb0 + NR - 1 and block columns cb0 .. cb0 + NC - 1.
// The 9 x 9 blocks of a tile are shared out as 21 + 21 + 21 + 18: wavefronts 0 .. 2 take three block rows each
// against block columns 0 .. 6, wavefront 3 all nine block rows against block columns 7 and 8 (the walk is as long as
// its busiest wavefront's instruction stream: a 2 x 2 split of 9 x 9 gives that one 25 blocks).  Straight-line per
// (NR, NC): each class runs its own copy, so no block is computed twice and none sits behind a branch (a branch
// inside the loop body cuts it into pieces the scheduler cannot interleave).
constexpr int FS_MAX_NR = 9, FS_MAX_NC = 7, FS_MAX_BLK = 21;
template <int NR, int NC, bool PRE, typename AfterIssue>
__device__ __forceinline__ void self_k_walk(const SelfArgs& a, unsigned char* lds, const unsigned char* const (&ap)[5],
                                            const unsigned char* const (&wp)[5], uint32_t lds0, int koff, bool tail, int rb0, int cb0,
                                            int c, int q, f32x4_t (&acc)[FS_MAX_BLK], float (&ssq)[FS_MAX_NR], float (&ssum)[FS_MAX_NR],
                                            AfterIssue&& after_issue) {
    static_assert(NR * NC <= FS_MAX_BLK && NR <= FS_MAX_NR && NC <= FS_MAX_NC, "block share of a wavefront");
    // row sums: the two wavefronts that multiply the same rows (a three-row one and the nine-row one) take alternate
    // 32-k chunks (PRE: the sums come from the launch that wrote the rows: no chunk takes them)
    constexpr int STATS_SET = PRE ? 7 : NR == 3 ? 0 : 1;
    const int fsw = (c >> 1) & 7;
    auto issue = [&](int kt, int stage) __attribute__((always_inline)) {
        const long kb = ((long)kt * 64 + koff) * 2;
        const uint32_t base = lds0 + stage * FS_STAGE;
#pragma unroll
        for (int v = 0; v < 4; ++v) load_to_lds16(ap[v] + kb, base + v * 4096);
#pragma unroll
        for (int v = 0; v < 4; ++v) load_to_lds16(wp[v] + kb, base + FS_ROWS * FS_KB + v * 4096);
        if (tail) {
            load_to_lds16(ap[4] + kb, base + 4 * 4096);
            load_to_lds16(wp[4] + kb, base + FS_ROWS * FS_KB + 4 * 4096);
        }
    };
    // request l of a tile's ten: the four 32-row slabs of x, the four of W, then the two 16-row remainders (tail)
    auto issue_one = [&](int l, int kt, int stage) __attribute__((always_inline)) {
        const long kb = ((long)kt * 64 + koff) * 2;
        const uint32_t base = lds0 + stage * FS_STAGE;
        if (l < 4) load_to_lds16(ap[l] + kb, base + l * 4096);
        else if (l < 8) load_to_lds16(wp[l - 4] + kb, base + FS_ROWS * FS_KB + (l - 4) * 4096);
        else if (tail) {
            if (l == 8) load_to_lds16(ap[4] + kb, base + 4 * 4096);
            else load_to_lds16(wp[4] + kb, base + FS_ROWS * FS_KB + 4 * 4096);
        }
    };
    u32x4_t fa[2][NR], fw[2][NC];  // fragment sets of two consecutive chunks
    auto read_frags = [&](int set, int stage, int ch) __attribute__((always_inline)) {
        const unsigned char* base = lds + stage * FS_STAGE;
        const int off = ((4 * ch + q) ^ fsw) * 16;
#pragma unroll
        for (int i = 0; i < NR; ++i) fa[set][i] = *reinterpret_cast<const u32x4_t*>(base + ((rb0 + i) * 16 + c) * FS_KB + off);
#pragma unroll
        for (int j = 0; j < NC; ++j)
            fw[set][j] = *reinterpret_cast<const u32x4_t*>(base + FS_ROWS * FS_KB + ((cb0 + j) * 16 + c) * FS_KB + off);
    };
    auto mfma_chunk = [&](int set) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NR; ++i)
#pragma unroll
            for (int j = 0; j < NC; ++j)
                acc[i * NC + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, fa[set][i]),
                                                                        __builtin_bit_cast(bf16x8_t, fw[set][j]), acc[i * NC + j], 0, 0, 0);
        if (set == STATS_SET) {  // a constant at both call sites
#pragma unroll
            for (int i = 0; i < NR; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ssq[i] = sum_squares_bf16x2(fa[set][i][e], ssq[i]);
                    ssum[i] = sum_pair_bf16x2(fa[set][i][e], ssum[i]);
                }
        }
    };
    // Chunk 1 of a tile, in groups of two MFMAs in a fixed order: each group reads one fragment of the next tile's chunk 0
    // and (LOAD) requests a share of the tile four further on into the stage the workgroup has just left.  Requested in
    // one burst after the barrier instead, the ten loads (an M0 write and a 64-bit address each) keep the matrix pipe
    // idle for their whole issue time, once per tile.
    constexpr int NM = NR * NC, NG = (NM + 1) / 2;
    static_assert(NR + NC <= NG + 2 && NG >= 8, "a fragment read and a request per group");
    auto chunk1_groups = [&](auto do_load, int kt_load, int st_load, int st_next) __attribute__((always_inline)) {
        constexpr bool LOAD = decltype(do_load)::value;
        const unsigned char* base = lds + st_next * FS_STAGE;
        const int off = (q ^ fsw) * 16;  // chunk 0
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            // fragment reads: NR + NC of them over the first groups (two in a group while more reads than groups remain)
#pragma unroll
            for (int f = 0; f < NR + NC; ++f) {
                if (f * NG / (NR + NC) != g) continue;
                if (f < NR) fa[0][f] = *reinterpret_cast<const u32x4_t*>(base + ((rb0 + f) * 16 + c) * FS_KB + off);
                else fw[0][f - NR] = *reinterpret_cast<const u32x4_t*>(base + FS_ROWS * FS_KB + ((cb0 + f - NR) * 16 + c) * FS_KB + off);
            }
#pragma unroll
            for (int m = 2 * g; m < 2 * g + 2 && m < NM; ++m)
                acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, fa[1][m / NC]),
                                                               __builtin_bit_cast(bf16x8_t, fw[1][m % NC]), acc[m], 0, 0, 0);
            if (LOAD) {
#pragma unroll
                for (int l = 0; l < 10; ++l)
                    if (l * NG / 10 == g) issue_one(l, kt_load, st_load);
            }
            if (STATS_SET == 1 && g < NR) {  // this chunk's row sums, a block row per group
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ssq[g] = sum_squares_bf16x2(fa[1][g][e], ssq[g]);
                    ssum[g] = sum_pair_bf16x2(fa[1][g][e], ssum[g]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Stage kt % 4 holds tile kt.  Chunk 0 of tile kt is multiplied while chunk 1's fragments
    // are read; then the wavefront waits for its loads of tile kt + 1 and meets the others (every
    // fragment of tile kt is in registers by then, so its stage takes tile kt + 4), reads chunk 0
    // of tile kt + 1 and multiplies chunk 1 of tile kt meanwhile.  K >= 256 (four tiles), so the
    // ring fills before the loop; nothing is fetched past the last tile.
    const int nkt = a.K / 64;
#pragma unroll
    for (int t = 0; t < FS_NS; ++t) issue(t, t);
    after_issue();  // work on loads requested before the ring's: they land first, and the ring's trip runs under it
    if (tail) wait_vmcnt<30>();
    else wait_vmcnt<24>();
    __syncthreads();
    read_frags(0, 0, 0);
    int st = 0;
    // chunk 0 of tile kt under the reads of its chunk 1
    auto chunk0 = [&]() __attribute__((always_inline)) {
        read_frags(1, st, 1);
        mfma_chunk(0);
        // a fragment read between every two MFMAs: the reads' issue slots hide behind the matrix pipe
#pragma unroll
        for (int g = 0; g < NR + NC; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // MFMA
            if (STATS_SET == 0) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // the chunk's row sums, spread between the MFMAs
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // Main part: every tile requests the one four further on (no branch in the body).  Tile kt + 1 has landed when
    // two younger tiles' requests may still be on their way.
    for (int kt = 0; kt + FS_NS < nkt; ++kt) {
        const int nx = st == FS_NS - 1 ? 0 : st + 1;
        chunk0();
        if (tail) wait_vmcnt<20>();
        else wait_vmcnt<16>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // chunk 1's fragments have left the stage
        __syncthreads();
        chunk1_groups(std::true_type{}, kt + FS_NS, st, nx);
        st = nx;
    }
    // The last four tiles: nothing left to request.
    for (int kt = nkt - FS_NS; kt < nkt; ++kt) {
        const int nx = st == FS_NS - 1 ? 0 : st + 1;
        chunk0();
        if (kt + 3 < nkt) {
            if (tail) wait_vmcnt<20>();
            else wait_vmcnt<16>();
        } else if (kt + 3 == nkt) {
            if (tail) wait_vmcnt<10>();
            else wait_vmcnt<8>();
        } else {
            wait_vmcnt<0>();
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __syncthreads();
        chunk1_groups(std::false_type{}, 0, 0, nx);
        st = nx;
    }
    wait_vmcnt<0>();
}

// The accumulators leave for LDS as bf16: rstd (acc - mean colsum) + bias, Q and K columns into the
// [row][q | k] tile, V columns transposed into their observation's V^T tile.  Per wavefront class like the
// walk, so that every loop bound and the kind of a block column (block columns 0 .. 5 are q | k, 6 .. 8 are
// v: the first NQK of a class's columns are q | k) are constants; what depends on the row
// only is formed once per row, an element costs two multiply-adds, half a conversion and a 2-byte store.
// FINAL: stat holds (rstd, -mean) per row, formed once by the row's thread; otherwise two partial (sum of squares, sum)
// pairs per row that every lane combines for its rows.
template <int NR, int NC, int NQK, bool FINAL>
__device__ __forceinline__ void self_tile_to_lds(const SelfArgs& a, const f32x4_t (&acc)[FS_MAX_BLK], const float (&cs)[FS_MAX_NC],
                                                 const float (&bs)[FS_MAX_NC], const float* stat, unsigned char* lds, int rb0, int cb0, int c,
                                                 int q, int n_valid) {
    const float inv_k = 1.0f / (float)a.K;
    const int S = a.S, inv_s = (65536 + S - 1) / S;
    unsigned char* const vt0 = lds + FS_ROWS * FS_QS * 2;
    int coff[NC];  // byte offset of the lane's column inside a row of the q | k tile, or of its V^T row inside an observation's tile
#pragma unroll
    for (int j = 0; j < NC; ++j) {
        const int col = (cb0 + j) * 16 + c;
        coff[j] = j < NQK ? col * 2 : (col - 2 * FS_D) * FS_VS * 2;
    }
    // the rows' sums first, three block rows a batch (one batch of LDS reads), then the arithmetic
    constexpr int RB = 3;
    static_assert(NR % RB == 0, "whole batches of block rows");
#pragma unroll
    for (int i0 = 0; i0 < NR; i0 += RB) {
    f32x2_t sa[RB][4], sb[RB][4];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = (rb0 + i0 + i) * 16 + 4 * q + e;
            sa[i][e] = *reinterpret_cast<const f32x2_t*>(stat + row * 2);
            if (!FINAL) sb[i][e] = *reinterpret_cast<const f32x2_t*>(stat + (FS_ROWS + row) * 2);
        }
    // Two rows (e, e + 1) at a time: one conversion gives both rows' bf16 values of a column, stored as the low
    // and the high half.  Rows past the tile's last observation write their V values to an unused part of LDS
    // (the address is selected once per row) instead of sitting behind a branch per element.
    unsigned char* const dead = lds + 96 * 1024;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
            float rstd[2], nmean[2];
            unsigned char* qrow[2];
            unsigned char* vrow[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int row = (rb0 + i0 + i) * 16 + 4 * q + e + h;
                if (FINAL) {
                    rstd[h] = sa[i][e + h][0];
                    nmean[h] = sa[i][e + h][1];
                } else {
                    const float s2 = sa[i][e + h][0] + sb[i][e + h][0], s1 = sa[i][e + h][1] + sb[i][e + h][1];
                    const float mean = s1 * inv_k;
                    rstd[h] = rsqrtf(fmaxf(s2 * inv_k - mean * mean, 0.f) + a.eps);
                    nmean[h] = -mean;
                }
                const int u = (row * inv_s) >> 16, key = row - u * S;  // row / S, exact for S <= 32 and row < 160
                qrow[h] = lds + row * FS_QS * 2;
                vrow[h] = row < n_valid ? vt0 + (u * FS_D * FS_VS + key) * 2 : dead;
            }
#pragma unroll
            for (int j = 0; j < NC; ++j) {
                // rstd (acc - mean colsum) + bias
                const float v0 = __builtin_fmaf(__builtin_fmaf(nmean[0], cs[j], acc[(i0 + i) * NC + j][e]), rstd[0], bs[j]);
                const float v1 = __builtin_fmaf(__builtin_fmaf(nmean[1], cs[j], acc[(i0 + i) * NC + j][e + 1]), rstd[1], bs[j]);
                const uint32_t pk = pack_bf2(v0, v1);
                unsigned char* const d0 = (j < NQK ? qrow[0] : vrow[0]) + coff[j];  // q: 0..47, k: 48..95; V^T[u][d][key]
                unsigned char* const d1 = (j < NQK ? qrow[1] : vrow[1]) + coff[j];
                *reinterpret_cast<bf16_t*>(d0) = (bf16_t)(pk & 0xffffu);
                *reinterpret_cast<bf16_t*>(d1) = (bf16_t)(pk >> 16);
            }
        }
    }
    }
}

template <bool PRE>
__global__ void __launch_bounds__(256, 1) dit_self_block_kernel(SelfArgs a) {
    __shared__ __attribute__((aligned(1024))) unsigned char lds[FS_NS * FS_STAGE];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool wide = wave < 3;                                  // three block rows x seven block columns, or nine x two
    const int rb0 = wide ? 3 * wave : 0, cb0 = wide ? 0 : 7;
    const int c = lane & 15, q = lane >> 4;
    const int head = blockIdx.x % a.H, group = blockIdx.x / a.H;
    const int rows_per = a.OB * a.S;
    const int m0 = group * rows_per;
    const int n_valid = min(rows_per, a.M - m0);  // rows of this tile that exist (whole observations)
    const long HD = (long)a.H * FS_D;

    // PRE: this thread's row of the tile (threads 0 .. 143) and its handed-over sums: requested first of all and
    // added up once the K walk has requested its ring (their trip runs under the address arithmetic below, the
    // ring's under the additions), which leaves two registers to carry through the walk instead of 48
    f32x2_t pre_pv[PRE ? FS_MAX_STAT : 1];
    if (PRE && tid < FS_ROWS) {
        const float* sp = a.stats_in + (long)min(m0 + tid, a.M - 1) * a.n_stat * 2;
#pragma unroll
        for (int t = 0; t < FS_MAX_STAT; ++t) pre_pv[t] = *reinterpret_cast<const f32x2_t*>(sp + 2 * min(t, a.n_stat - 1));
    }

    // ---- loader: thread tid fills slot tid of each 256-slot slab (32 rows x 8 pieces); slabs 0..3
    // are whole, slab 4 holds rows 128..143 and is filled by wavefronts 0 and 1 alone
    const int lrow = tid >> 3;
    const int koff = ((tid & 7) ^ ((lrow >> 1) & 7)) * 8;  // logical piece that belongs in this slot, in elements
    const unsigned char* ap[5];
    const unsigned char* wp[5];
#pragma unroll
    for (int v = 0; v < 5; ++v) {
        const int r = min(v * 32 + lrow, FS_ROWS - 1);
        ap[v] = (const unsigned char*)(a.x + (long)min(m0 + r, a.M - 1) * a.K);
        const int seg = r / FS_D, d = r - seg * FS_D;
        wp[v] = (const unsigned char*)(a.W + ((long)seg * HD + (long)head * FS_D + d) * a.K);
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds + wave * 1024;
    const bool tail = wave < 2;  // uniform

    // this lane's output columns: bias and column sums, requested ahead of the ring (they are the
    // oldest loads, so the first wait on the ring covers them)
    float cs[FS_MAX_NC], bs[FS_MAX_NC];
#pragma unroll
    for (int j = 0; j < FS_MAX_NC; ++j) {
        const int col = min((cb0 + j) * 16 + c, FS_COLS - 1);
        const int seg = col / FS_D, d = col - seg * FS_D;
        const long n = (long)seg * HD + (long)head * FS_D + d;
        cs[j] = a.colsum[n];
        bs[j] = a.bias ? a.bias[n] : 0.f;
    }

    f32x4_t acc[FS_MAX_BLK];
#pragma unroll
    for (int i = 0; i < FS_MAX_BLK; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float ssq[FS_MAX_NR], ssum[FS_MAX_NR];
#pragma unroll
    for (int i = 0; i < FS_MAX_NR; ++i) ssq[i] = ssum[i] = 0.f;
    float pre_q = 0.f, pre_u = 0.f;
    auto sum_pre = [&]() __attribute__((always_inline)) {
        if (PRE && tid < FS_ROWS) {
#pragma unroll
            for (int t = 0; t < FS_MAX_STAT; ++t) {
                pre_q += t < a.n_stat ? pre_pv[t][0] : 0.f;
                pre_u += t < a.n_stat ? pre_pv[t][1] : 0.f;
            }
        }
    };
    const int nr = wide ? 3 : 9;
    if (wide) self_k_walk<3, 7, PRE>(a, lds, ap, wp, lds0, koff, tail, rb0, cb0, c, q, acc, ssq, ssum, sum_pre);
    else self_k_walk<9, 2, PRE>(a, lds, ap, wp, lds0, koff, tail, rb0, cb0, c, q, acc, ssq, ssum, sum_pre);
    __syncthreads();

    // ---- the tile leaves the accumulators: row statistics first
    bf16_t* qk = reinterpret_cast<bf16_t*>(lds);                                        // [FS_ROWS][FS_QS]: q | k
    bf16_t* vt = qk + FS_ROWS * FS_QS;                                                  // [OB][FS_D][FS_VS]: V^T per observation
    float* stat = reinterpret_cast<float*>(lds + (FS_ROWS * FS_QS + FS_MAX_OB * FS_D * FS_VS) * 2);  // [2][FS_ROWS][2]: (sum of squares, sum), a partial pair from each of a row's two wavefronts
    if (!PRE) {
#pragma unroll
        for (int i = 0; i < FS_MAX_NR; ++i) {
            const float s2 = rows_sum(ssq[i]), s1 = rows_sum(ssum[i]);
            const int rb = rb0 + i, part = wide ? 0 : 1;
            if (q == 0 && i < nr) {  // one partial pair per wavefront of the row's two
                stat[(part * FS_ROWS + rb * 16 + c) * 2] = s2;
                stat[(part * FS_ROWS + rb * 16 + c) * 2 + 1] = s1;
            }
        }
    }
    if (PRE && tid < FS_ROWS) {  // the row's (rstd, -mean), formed once here rather than by every lane that holds the row
        const float inv_k = 1.0f / (float)a.K;
        const float mean = pre_u * inv_k;
        stat[tid * 2] = rsqrtf(fmaxf(pre_q * inv_k - mean * mean, 0.f) + a.eps);
        stat[tid * 2 + 1] = -mean;
    }
    // keys past S of every V^T row are multiplied by probabilities that are zero: they must be finite
    const int S = a.S;
    for (int row = tid; row < a.OB * FS_D; row += 256)
        for (int k4 = S >> 2; k4 < FS_VS / 4; ++k4)  // the groups of four keys that reach past S
            *reinterpret_cast<u32x2_t*>(vt + row * FS_VS + 4 * k4) = u32x2_t{0u, 0u};
    __syncthreads();
    if (wide) self_tile_to_lds<3, 7, 6, PRE>(a, acc, cs, bs, stat, lds, rb0, cb0, c, q, n_valid);
    else self_tile_to_lds<9, 2, 0, PRE>(a, acc, cs, bs, stat, lds, rb0, cb0, c, q, n_valid);
    __syncthreads();

    // ---- attention: wavefront w takes observations w, w + 4, ... of the tile
    typedef short bf16x4_t __attribute__((ext_vector_type(4)));
    const float sl2 = a.scale * 1.4426950408889634f;
    // Two observations at a time (u and u + 4), their instructions side by side: one pair's chain
    // of fragment reads, MFMAs, lane exchanges and exponentials is mostly waiting.
    for (int u0 = wave; u0 * S < n_valid; u0 += 8) {
        const bool two = (u0 + 4) * S < n_valid;  // uniform
        int r0[2];
        r0[0] = u0 * S;
        r0[1] = two ? (u0 + 4) * S : r0[0];
        const int uu[2] = {u0, two ? u0 + 4 : u0};
        // S^T = K Q^T: sT[kb][qb][e] = score of key 16 kb + 4 q + e against query 16 qb + c
        f32x4_t sT[2][2][2];
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) sT[p][kb][qb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < FS_D / 16; ++ks) {
            bf16x4_t kf[2][2], qf[2][2];
#pragma unroll
            for (int p = 0; p < 2; ++p)
#pragma unroll
                for (int b2 = 0; b2 < 2; ++b2) {
                    const int row = r0[p] + min(16 * b2 + c, S - 1);  // rows past S repeat the last token; masked below
                    kf[p][b2] = *reinterpret_cast<const bf16x4_t*>(qk + row * FS_QS + FS_D + 16 * ks + 4 * q);
                    qf[p][b2] = *reinterpret_cast<const bf16x4_t*>(qk + row * FS_QS + 16 * ks + 4 * q);
                }
#pragma unroll
            for (int p = 0; p < 2; ++p)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int qb = 0; qb < 2; ++qb)
                        sT[p][kb][qb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf[p][kb], qf[p][qb], sT[p][kb][qb], 0, 0, 0);
        }
        // softmax over the keys of query 16 qb + c: this lane's 8 values and the lanes q = 0..3 of column c
        bf16x4_t pf[2][2][2];  // P as an operand: [pair][key block][query block], keys 4 q .. 4 q + 3
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                float mx = -INFINITY;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (16 * kb + 4 * q + e >= S) sT[p][kb][qb][e] = -INFINITY;
                        mx = fmaxf(mx, sT[p][kb][qb][e]);
                    }
                mx = rows_max(mx);
                float sum = 0.f;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float pr = exp2f((sT[p][kb][qb][e] - mx) * sl2);
                        sT[p][kb][qb][e] = pr;
                        sum += pr;
                    }
                sum = rows_sum(sum);
                const float inv = 1.0f / sum;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const uint32_t lo = pack_bf2(sT[p][kb][qb][0] * inv, sT[p][kb][qb][1] * inv),
                                   hi = pack_bf2(sT[p][kb][qb][2] * inv, sT[p][kb][qb][3] * inv);
                    pf[p][kb][qb] = __builtin_bit_cast(bf16x4_t, u32x2_t{lo, hi});
                }
            }
        // O^T = V^T P^T: o[e] = column 16 db + 4 q + e of query 16 qb + c, four consecutive columns per lane
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            if (p == 1 && !two) break;
#pragma unroll
            for (int db = 0; db < FS_D / 16; ++db) {
                bf16x4_t vf[2];
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
                    vf[kb] = *reinterpret_cast<const bf16x4_t*>(vt + (uu[p] * FS_D + 16 * db + c) * FS_VS + 16 * kb + 4 * q);
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    f32x4_t o = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) o = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[kb], pf[p][kb][qb], o, 0, 0, 0);
                    const int qi = 16 * qb + c;
                    if (qi < S)
                        *reinterpret_cast<u32x2_t*>(a.out + (long)(m0 + r0[p] + qi) * HD + (long)head * FS_D + 16 * db + 4 * q) =
                            u32x2_t{pack_bf2(o[0], o[1]), pack_bf2(o[2], o[3])};
                }
            }
        }
    }
}

}  // namespace
}  // namespace vk

static int self_block_impl(const void* x, const void* W_folded, const float* colsum, const float* bias, const float* row_stats,
                           int n_stat_tiles, int dtype, int M, int K, int S, int n_heads, int head_dim, float scale, float ln_eps,
                           void* out, vla_stream_t stream) {
    using namespace vk;
    if (!x || !W_folded || !colsum || !out || M < 0 || K <= 0 || S <= 0 || n_heads <= 0) return VLA_K_ERR_ARG;
    if (dtype != VLA_DT_BF16 || head_dim != FS_D || S > FS_MAX_S || M % S || K % 64 || K < 64 * FS_NS || n_heads % 8) return VLA_K_ERR_SHAPE;
    if (((uintptr_t)x | (uintptr_t)W_folded | (uintptr_t)out) & 15) return VLA_K_ERR_SHAPE;
    if (row_stats && (n_stat_tiles < 1 || n_stat_tiles > FS_MAX_STAT || n_stat_tiles * 64 != K || ((uintptr_t)row_stats & 7))) return VLA_K_ERR_SHAPE;
    if (M == 0) return VLA_K_OK;
    SelfArgs a;
    a.x = (const bf16_t*)x; a.W = (const bf16_t*)W_folded; a.colsum = colsum; a.bias = bias; a.out = (bf16_t*)out;
    a.M = M; a.K = K; a.S = S; a.H = n_heads; a.OB = FS_ROWS / S < FS_MAX_OB ? FS_ROWS / S : FS_MAX_OB; a.scale = scale; a.eps = ln_eps;
    a.stats_in = row_stats; a.n_stat = n_stat_tiles;
    const int n_obs = M / S, groups = (n_obs + a.OB - 1) / a.OB;
    if (row_stats) dit_self_block_kernel<true><<<(unsigned)(groups * n_heads), 256, 0, (hipStream_t)stream>>>(a);
    else dit_self_block_kernel<false><<<(unsigned)(groups * n_heads), 256, 0, (hipStream_t)stream>>>(a);
    return hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH;
}

extern "C" VLA_KAPI int vla_layernorm_qkv_self_attention(const void* x, const void* W_folded, const float* colsum, const float* bias,
                                                int dtype, int M, int K, int S, int n_heads, int head_dim, float scale,
                                                float ln_eps, void* out, vla_stream_t stream) {
    return self_block_impl(x, W_folded, colsum, bias, nullptr, 0, dtype, M, K, S, n_heads, head_dim, scale, ln_eps, out, stream);
}

extern "C" VLA_KAPI int vla_layernorm_qkv_self_attention_stats(const void* x, const void* W_folded, const float* colsum, const float* bias,
                                                      const float* row_stats, int n_stat_tiles, int dtype, int M, int K, int S,
                                                      int n_heads, int head_dim, float scale, float ln_eps, void* out,
                                                      vla_stream_t stream) {
    if (!row_stats) return VLA_K_ERR_ARG;
    return self_block_impl(x, W_folded, colsum, bias, row_stats, n_stat_tiles, dtype, M, K, S, n_heads, head_dim, scale, ln_eps, out, stream);
}
