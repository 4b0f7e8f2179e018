// Row-wise and element-wise kernels around the attention path: NeoX RoPE,
// RMSNorm / adaLN pre-norms, the flow-matching embed / Euler glue, and the
// BitVLA layer helpers whose signatures follow
// src/kernels/bitvla/bitvla_lm_cuda.h:54-155.  All are HBM / latency bound;
// each row is handled by one workgroup with 64-lane shuffle reductions.

#include <math.h>

#include "common.h"
#include "vla_kernels.h"

namespace {

using namespace vk;

#define VLA_CHECK_LAUNCH() (hipGetLastError() == hipSuccess ? VLA_K_OK : VLA_K_ERR_LAUNCH)

// ------------------------------------------------------------------ RoPE ---
// x [n_rows][H][D]; one thread per rotation pair.  (a, b) = (x[i], x[i + D/2])
// -> (a c - b s, b c + a s), computed in fp32.
template <typename T>
__global__ void rope_neox_kernel(T* __restrict__ x, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                 int table_rows, int H, int D, long total_pairs) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total_pairs) return;
    const int half = D >> 1;
    const int p = (int)(i % half);
    const long rh = i / half;  // row * H + head
    const int row = (int)(rh / H);
    const int tr = row % table_rows;
    const float c = cos_t[(long)tr * half + p], s = sin_t[(long)tr * half + p];
    T* base = x + rh * D;
    const float a = Elem<T>::load(base + p), b = Elem<T>::load(base + p + half);
    Elem<T>::store(base + p, a * c - b * s);
    Elem<T>::store(base + p + half, b * c + a * s);
}

// Head-major variant of the BitVLA layer: inout [H][S][D], tables [S][D/2].
__global__ void rope_neox_hsd_bf16_kernel(bf16_t* __restrict__ x, const float* __restrict__ cos_t,
                                          const float* __restrict__ sin_t, int S, int D, long total_pairs) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total_pairs) return;
    const int half = D >> 1;
    const int p = (int)(i % half);
    const long hs = i / half;  // head * S + s
    const int s_idx = (int)(hs % S);
    const float c = cos_t[(long)s_idx * half + p], s = sin_t[(long)s_idx * half + p];
    bf16_t* base = x + hs * D;
    const float a = bf2f(base[p]), b = bf2f(base[p + half]);
    base[p] = f2bf(a * c - b * s);
    base[p + half] = f2bf(b * c + a * s);
}

// Split a fused [M][(Hq+2Hkv)*D] projection (Q | K | V columns), rotate Q and K
// and scatter: Q token-major, K / V into the resident cache.  One thread per
// rotation pair (Q, K) or per element pair (V).
template <typename T>
__global__ void qkv_split_rope_append_kernel(const T* __restrict__ qkv, const float* __restrict__ cos_t,
                                             const float* __restrict__ sin_t, T* __restrict__ q_out,
                                             T* __restrict__ k_cache, T* __restrict__ vt_cache, int S, int Hq, int Hkv,
                                             int D, int t_max, int tok_offset, long total) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int half = D >> 1;
    const int heads = Hq + 2 * Hkv;
    const int p = (int)(i % half);
    long rh = i / half;
    const int hh = (int)(rh % heads);
    const int m = (int)(rh / heads);
    const int b = m / S, s = m % S;
    const T* src = qkv + ((long)m * heads + hh) * D;
    float a = Elem<T>::load(src + p), c2 = Elem<T>::load(src + p + half);
    if (hh < Hq + Hkv && cos_t) {
        const float c = cos_t[(long)s * half + p], sn = sin_t[(long)s * half + p];
        const float x0 = a, x1 = c2;
        a = x0 * c - x1 * sn;
        c2 = x1 * c + x0 * sn;
    }
    if (hh < Hq) {
        T* dst = q_out + ((long)m * Hq + hh) * D;
        Elem<T>::store(dst + p, a);
        Elem<T>::store(dst + p + half, c2);
    } else if (hh < Hq + Hkv) {
        T* dst = k_cache + (((long)b * Hkv + (hh - Hq)) * t_max + tok_offset + s) * D;
        Elem<T>::store(dst + p, a);
        Elem<T>::store(dst + p + half, c2);
    } else {
        T* dst = vt_cache + ((long)b * Hkv + (hh - Hq - Hkv)) * D * (long)t_max + tok_offset + s;
        Elem<T>::store(dst + (long)p * t_max, a);
        Elem<T>::store(dst + (long)(p + half) * t_max, c2);
    }
}

// ----------------------------------------------------------------- norms ---
template <typename T>
__global__ void rms_norm_kernel(const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, int K, float eps) {
    __shared__ float red[16];
    const T* xr = x + (long)blockIdx.x * K;
    T* yr = y + (long)blockIdx.x * K;
    float ss = 0.f;
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        const float v = Elem<T>::load(xr + k);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)K + eps);
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        float v = Elem<T>::load(xr + k) * scale;
        if (w) v *= Elem<T>::load(w + k);
        Elem<T>::store(yr + k, v);
    }
}

template <typename T>
__global__ void adaln_kernel(const T* __restrict__ x, const float* __restrict__ sc, const float* __restrict__ sh,
                             T* __restrict__ y, int K, float eps, int rms) {
    __shared__ float red[16];
    const T* xr = x + (long)blockIdx.x * K;
    T* yr = y + (long)blockIdx.x * K;
    float s1 = 0.f;
    for (int k = threadIdx.x; k < K; k += blockDim.x) s1 += Elem<T>::load(xr + k);
    const float mean = rms ? 0.f : block_sum(s1, red) / (float)K;  // rms: no centring (build_adarms)
    float s2 = 0.f;
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        const float d = Elem<T>::load(xr + k) - mean;
        s2 += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum(s2, red) / (float)K + eps);
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        const float xn = (Elem<T>::load(xr + k) - mean) * inv;
        Elem<T>::store(yr + k, xn + xn * sc[k] + sh[k]);
    }
}

// Row normalisations, one wavefront per row (four rows per workgroup): the row is read once
// with 16-byte loads and stays in registers, the reductions are wavefront shuffles, and there
// is no LDS and no barrier.  RMS: y = x * rsqrt(mean(x^2) + eps) * w.  ADALN: LayerNorm
// without affine, then y = xn * (1 + scale) + shift.  RMS_AQ: the RMS result, rounded to bf16
// as it would be stored, quantised per row to int8 (scale 127 / max(amax, 1e-5), round half
// even) with its row sum -- bitvla_rmsnorm_bf16 followed by act_quant without the round trip.
enum { NORM_RMS = 0, NORM_ADALN = 1, NORM_RMS_AQ = 2, NORM_ADARMS = 3 };  // ADARMS: RMS statistics, then (1 + scale), shift
template <typename T, int NV, int MODE, bool GLU = false>
__global__ void __launch_bounds__(256) row_norm_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                       const float* __restrict__ sc, const float* __restrict__ sh,
                                                       T* __restrict__ y, int8_t* __restrict__ q, float* __restrict__ scales,
                                                       int32_t* __restrict__ rowsum, int M, int K, float eps) {
    constexpr int EPV = 16 / sizeof(T);
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    if constexpr (MODE == NORM_RMS_AQ && sizeof(T) == 2) {
        float scale;
        int sum;
        // GLU: x holds [gate(K) | up(K)] rows and the row normalised is relu(gate)^2 * up
        rms_act_quant_row<NV, GLU>((const bf16_t*)x + (long)row * K * (GLU ? 2 : 1), (const bf16_t*)w, K, eps, lane,
                                   q + (long)row * K, scale, sum);
        if (lane == 0) {
            scales[row] = scale;
            if (rowsum) rowsum[row] = sum;
        }
        return;
    }
    const int nvec = K / EPV;
    const T* xr = x + (long)row * K;
    float v[NV][EPV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int vec = lane + 64 * i;
        u32x4_t raw = {0u, 0u, 0u, 0u};
        if (vec < nvec) raw = *reinterpret_cast<const u32x4_t*>(xr + (long)vec * EPV);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
            if (sizeof(T) == 2) v[i][e] = __uint_as_float((e & 1) ? (raw[e >> 1] & 0xffff0000u) : (raw[e >> 1] << 16));
            else v[i][e] = __uint_as_float(raw[e]);
        }
    }
    float mean = 0.f, inv;
    if (MODE == NORM_ADALN) {
        float s1 = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < EPV; ++e) s1 += v[i][e];
        mean = wave_sum(s1) / (float)K;
        float s2 = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                const float d = (lane + 64 * i < nvec) ? v[i][e] - mean : 0.f;
                s2 += d * d;
            }
        inv = 1.0f / sqrtf(wave_sum(s2) / (float)K + eps);
    } else {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < EPV; ++e) ss += v[i][e] * v[i][e];
        inv = 1.0f / sqrtf(wave_sum(ss) / (float)K + eps);
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int vec = lane + 64 * i;
        if (vec >= nvec) continue;
        const int k0 = vec * EPV;
        float o[EPV];
        if (MODE == NORM_ADALN || MODE == NORM_ADARMS) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                const float xn = (v[i][e] - mean) * inv;  // mean stays 0 for ADARMS
                o[e] = xn + xn * sc[k0 + e] + sh[k0 + e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                o[e] = v[i][e] * inv;
                if (w) o[e] *= Elem<T>::load(w + k0 + e);
            }
        }
        if (MODE == NORM_RMS_AQ) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                v[i][e] = bf2f(f2bf(o[e]));  // the activation as the bf16 it would be stored as
                amax = fmaxf(amax, fabsf(v[i][e]));
            }
        } else if (sizeof(T) == 2) {
            u32x4_t pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = (uint32_t)f2bf(o[2 * e]) | ((uint32_t)f2bf(o[2 * e + 1]) << 16);
            *reinterpret_cast<u32x4_t*>(y + (long)row * K + k0) = pk;
        } else {
            const u32x4_t pk = {__float_as_uint(o[0]), __float_as_uint(o[1]), __float_as_uint(o[2]), __float_as_uint(o[3])};
            *reinterpret_cast<u32x4_t*>(y + (long)row * K + k0) = pk;
        }
    }
    if (MODE == NORM_RMS_AQ) {
        amax = wave_max(amax);
        if (amax < 1e-5f) amax = 1e-5f;
        const float scale = 127.0f / amax;
        int sum = 0;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int vec = lane + 64 * i;
            if (vec >= nvec) continue;
            uint32_t pk[2] = {0u, 0u};
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                float qf = rintf(v[i][e] * scale);
                qf = fminf(fmaxf(qf, -128.0f), 127.0f);
                const int qi = (int)qf;
                sum += qi;
                pk[e >> 2] |= (uint32_t)(qi & 0xff) << (8 * (e & 3));
            }
            *reinterpret_cast<u32x2_t*>(q + (long)row * K + (long)vec * EPV) = u32x2_t{pk[0], pk[1]};
        }
        sum = wave_sum_i(sum);
        if (lane == 0) {
            scales[row] = scale;
            if (rowsum) rowsum[row] = sum;
        }
    }
}

// Rows longer than 4096 (the 6912-wide BitNet FFN) through RMSNorm + int8 quantisation: one
// workgroup of four wavefronts per row, four vectors per lane at most (a single wavefront
// would hold sixteen and spend its time in the arithmetic of 128 elements per lane).
template <bool GLU>
__global__ void __launch_bounds__(256) row_norm_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                            int8_t* __restrict__ q, float* __restrict__ scales,
                                                            int32_t* __restrict__ rowsum, int K, float eps) {
    __shared__ float red[16];
    const int row = blockIdx.x;
    float scale;
    int sum;
    rms_act_quant_row<4, GLU, 4>(x + (long)row * K * (GLU ? 2 : 1), w, K, eps, threadIdx.x, q + (long)row * K, scale, sum, red);
    if (threadIdx.x == 0) {
        scales[row] = scale;
        if (rowsum) rowsum[row] = sum;
    }
}

// Launches row_norm_kernel when the row fits a wavefront's registers and the buffers allow
// 16-byte accesses; returns false otherwise (the callers fall back to the scalar kernels).
// The choice depends on the row length only, never on the number of rows, so an
// observation's result does not depend on the batch it is run in.
template <typename T, int MODE, bool GLU = false>
bool launch_row_norm(const void* x, const void* w, const float* sc, const float* sh, void* y, int8_t* q, float* scales,
                     int32_t* rowsum, int M, int K, float eps, hipStream_t st) {
    constexpr int EPV = 16 / sizeof(T);
    if (K % EPV || (((uintptr_t)x | (uintptr_t)y | (uintptr_t)q) & 15)) return false;
    if (MODE == NORM_RMS_AQ && (K % 8)) return false;
    const int nvec = K / EPV, blocks = (M + 3) / 4;
#define VLA_ROW_NORM(NV) \
    row_norm_kernel<T, NV, MODE, GLU><<<blocks, 256, 0, st>>>((const T*)x, (const T*)w, sc, sh, (T*)y, q, scales, rowsum, M, K, eps)
    if (nvec <= 64 * 2) VLA_ROW_NORM(2);
    else if (nvec <= 64 * 4) VLA_ROW_NORM(4);
    else if (nvec <= 64 * 8) VLA_ROW_NORM(8);
    else if constexpr (MODE == NORM_RMS_AQ && sizeof(T) == 2) {  // the 6912-wide BitNet FFN rows
        if (nvec > 64 * 16) return false;
        row_norm_wide_kernel<GLU><<<M, 256, 0, st>>>((const bf16_t*)x, (const bf16_t*)w, q, scales, rowsum, K, eps);
    } else {
        return false;
    }
#undef VLA_ROW_NORM
    return true;
}

// ------------------------------------------------- flow-matching glue ---
// Workgroup (x, y) forms EMB_ROWS consecutive (batch, token) rows of column slab y (EMB_COLS
// columns).  The action rows and the slab of W_in sit in LDS, both read with contiguous,
// coalesced loads issued together; thread (rq, cl) then forms the dot products of rows
// rq, rq+4, ... with column cl (summed over the action dimension in ascending order), and
// stores are coalesced along the width.  One load round trip per workgroup.
constexpr int EMB_ROWS = 32;
constexpr int EMB_MAX_A = 64;
constexpr int EMB_WIDE_A = 136;  // GR00T N1.6 / N1.7: 128 / 132 action values per row
constexpr int EMB_COLS = 64;
template <typename T, int AMAX = EMB_MAX_A>  // AMAX: the padded action width the staging loops are unrolled for
__global__ void __launch_bounds__(256) embed_suffix_kernel(const float* __restrict__ x_t, const float* __restrict__ W_in,
                                                            const float* __restrict__ bias_step,
                                                            const float* __restrict__ lead, T* __restrict__ h, int n_rows,
                                                            int S, int n_lead, int A, int W, int act) {
    // rows padded to a multiple of four floats: every a-loop step below is one 16-byte LDS read
    // of the thread's weight row (row stride 68 floats: 16 lanes cover all 64 banks once) and one
    // 16-byte broadcast read per output row, 9 LDS instructions per 32 multiply-adds
    // (stride 140 for the wide form: 140 mod 64 = 12 spreads 16 lanes the same way)
    constexpr int LD = AMAX > EMB_MAX_A ? AMAX : EMB_MAX_A;
    __shared__ __attribute__((aligned(16))) float xs[EMB_ROWS][LD];
    __shared__ __attribute__((aligned(16))) float ws[EMB_COLS][LD + 4];
    const int row0 = blockIdx.x * EMB_ROWS, c0 = blockIdx.y * EMB_COLS;
    const int ncol = min(EMB_COLS, W - c0);
    const int A4 = (A + 3) & ~3;
    // Every global load of the workgroup is issued before the first is used, none under a
    // branch (addresses of elements that do not exist are clamped to element 0 and the value is
    // replaced by zero): loads under branches are waited for one by one, a dozen round trips
    // to memory instead of one.  Element i of a staged array is (i / A4, i % A4); a thread's
    // elements are 256 apart, so the pair advances by (256 / A4, 256 % A4) without dividing again.
    // (batch, token) of the workgroup's rows, divided once per row rather than once per use
    __shared__ int row_b[EMB_ROWS], row_s[EMB_ROWS];
    if (threadIdx.x < EMB_ROWS) {
        const int row = min(row0 + (int)threadIdx.x, n_rows - 1);
        row_b[threadIdx.x] = row / S;
        row_s[threadIdx.x] = row % S;
    }
    __syncthreads();
    constexpr int XI = EMB_ROWS * AMAX / 256, WI = EMB_COLS * AMAX / 256;
    const int dq = 256 / A4, dr = 256 % A4;
    float xv[XI], wv[WI];
    {
        int rr = threadIdx.x / A4, a = threadIdx.x % A4;
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            const int row = row0 + rr;
            const int b = row_b[min(rr, EMB_ROWS - 1)], sx = row_s[min(rr, EMB_ROWS - 1)];
            const bool ok = rr < EMB_ROWS && row < n_rows && a < A && sx >= n_lead;
            const float v = x_t[ok ? ((long)b * (S - n_lead) + (sx - n_lead)) * A + a : 0];
            xv[it] = ok ? v : 0.f;
            rr += dq;
            a += dr;
            if (a >= A4) {
                a -= A4;
                ++rr;
            }
        }
    }
    {
        int cc = threadIdx.x / A4, a = threadIdx.x % A4;
#pragma unroll
        for (int it = 0; it < WI; ++it) {
            const bool ok = cc < ncol && a < A;
            const float v = W_in[ok ? (long)(c0 + cc) * A + a : 0];
            wv[it] = ok ? v : 0.f;
            cc += dq;
            a += dr;
            if (a >= A4) {
                a -= A4;
                ++cc;
            }
        }
    }
    const int cl = threadIdx.x & 63, rq = threadIdx.x >> 6;  // column in slab, row residue mod 4
    const int c = c0 + cl, cc_ok = min(c, W - 1);
    const float bias = bias_step[cc_ok];
    // the rows copied from `lead` (s < n_lead), fetched for every row of the thread and dropped where not needed
    constexpr int NR = EMB_ROWS / 4;
    float lv[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        const int b = row_b[rq + 4 * k], sx = row_s[rq + 4 * k];
        lv[k] = n_lead > 0 ? lead[((long)b * n_lead + min(sx, n_lead - 1)) * W + cc_ok] : 0.f;
    }
    {
        int rr = threadIdx.x / A4, a = threadIdx.x % A4;
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            if (rr < EMB_ROWS) xs[rr][a] = xv[it];
            rr += dq;
            a += dr;
            if (a >= A4) {
                a -= A4;
                ++rr;
            }
        }
        int cc = threadIdx.x / A4;
        a = threadIdx.x % A4;
#pragma unroll
        for (int it = 0; it < WI; ++it) {
            if (cc < EMB_COLS) ws[cc][a] = wv[it];
            cc += dq;
            a += dr;
            if (a >= A4) {
                a -= A4;
                ++cc;
            }
        }
    }
    __syncthreads();
    if (c >= W) return;
    float acc[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) acc[k] = 0.f;
    for (int a = 0; a < A4; a += 4) {  // products added in the order of a, as a scalar loop would
        const f32x4_t w4 = *reinterpret_cast<const f32x4_t*>(&ws[cl][a]);
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const f32x4_t x4 = *reinterpret_cast<const f32x4_t*>(&xs[rq + 4 * k][a]);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[k] += w4[e] * x4[e];
        }
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        const int rr = rq + 4 * k, row = row0 + rr;
        if (row >= n_rows) continue;
        const float v = row_s[rr] < n_lead ? lv[k] : apply_act(acc[k] + bias, act);
        Elem<T>::store(h + (long)row * W + c, v);
    }
}

// h[b][s][:] = lead[b][s][:] for s < n_lead (the state token rows of a suffix whose action
// rows came out of a projection over all rows).
template <typename T>
__global__ void lead_rows_kernel(const float* __restrict__ lead, T* __restrict__ h, long total, int S, int n_lead, int W) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = (int)(i % W);
    const long bs = i / W;
    const int s = (int)(bs % n_lead);
    const long b = bs / n_lead;
    Elem<T>::store(h + ((long)b * S + s) * W + c, lead[i]);
}

// h[b][s][:] = lead[b][s][:] for s < n_lead, else acc[b][s][:] + table[s - n_lead][:], converted
// to T: the last step of a suffix embedding whose action rows came out of an fp32 projection
// over all rows and carry a learned per-position term.
template <typename T>
__global__ void finish_suffix_rows_kernel(const float* __restrict__ acc, const float* __restrict__ table,
                                          const float* __restrict__ lead, T* __restrict__ h, long total, int S, int n_lead, int W) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = (int)(i % W);
    const long bs = i / W;
    const int s = (int)(bs % S);
    const long b = bs / S;
    float v;
    if (s < n_lead) v = lead[((long)b * n_lead + s) * W + c];
    else v = acc[i] + (table ? table[(long)(s - n_lead) * W + c] : 0.f);
    Elem<T>::store(h + i, v);
}

// Workgroup (x, y): EUL_WAVES wavefronts, each owning ROWS action rows, all working on the
// AU action outputs of group y.  A lane keeps elements lane, lane+64, ... of its rows in
// registers (NC chunks cover the width); the chunk loads of the AU rows of W_out are
// independent and issued together; the products are summed per lane in ascending k and then
// across the wavefront, and lane (i, u) applies the update of row i, output u.
//
// NORM >= 0: hn holds the rows before the stack's final norm, and the wavefront normalises its
// rows in registers first (the statistics of row_norm_kernel's modes, each element rounded to T
// as the stand-alone launch would have stored it), so the norm launch in front is not needed.
// Workgroups of different action groups y repeat the norm of the same rows: a few hundred
// operations against a launch.
//
// VEC (W a multiple of 8, 16-byte aligned operands): a lane's elements are runs of eight
// (8 (lane + 64 j) .. +7), fetched with 16-byte loads: an eighth of the load instructions,
// which were most of what the kernel issued.  The products are then summed in another order
// than in the element-per-lane form (fp32, agreeing to rounding).
constexpr int EUL_WAVES = 4;
constexpr int EUL_NO_NORM = -1;
__device__ __forceinline__ void eul_load8(const bf16_t* p, float* o) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        o[2 * j] = __uint_as_float(raw[j] << 16);
        o[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
    }
}
__device__ __forceinline__ void eul_load8(const float* p, float* o) {
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(p), b = *reinterpret_cast<const f32x4_t*>(p + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        o[j] = a[j];
        o[4 + j] = b[j];
    }
}
template <typename T, int NC, int AU, int ROWS, int NORM = EUL_NO_NORM, bool VEC = false>
__global__ void __launch_bounds__(EUL_WAVES * 64) euler_step_kernel(float* __restrict__ x_t, const T* __restrict__ hn,
                                                                    const float* __restrict__ W_out,
                                                                    const float* __restrict__ b_out, int n_rows, int S,
                                                                    int n_lead, int A, int W, float dt,
                                                                    const T* __restrict__ norm_w = nullptr,
                                                                    const float* __restrict__ sc = nullptr,
                                                                    const float* __restrict__ sh = nullptr, float eps = 0.f) {
    const int Sa = S - n_lead;
    // the wavefront's index as a scalar: row bases are then scalar too and a load's address is
    // base + 32-bit lane offset (64-bit per-lane addresses for every chunk would crowd the
    // register file and leave the loads waited for one by one)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r0 = (blockIdx.x * EUL_WAVES + wave) * ROWS, a0 = blockIdx.y * AU;
    if (r0 >= n_rows) return;
    static_assert(!VEC || NC % 8 == 0, "runs of eight");
    float hv[ROWS][NC], wv[AU][NC];
    // element held in slot c, and the load of a row's slots from p (clamped into the row)
    auto kidx = [&](int c) { return VEC ? 8 * (lane + 64 * (c >> 3)) + (c & 7) : lane + 64 * c; };
    auto load_slots = [&](auto* p, float* dst) __attribute__((always_inline)) {
        if constexpr (VEC) {
#pragma unroll
            for (int cv = 0; cv < NC / 8; ++cv) eul_load8(p + 8u * (unsigned)min(lane + 64 * cv, W / 8 - 1), dst + 8 * cv);
        } else {
#pragma unroll
            for (int c = 0; c < NC; ++c) dst[c] = Elem<std::remove_cv_t<std::remove_pointer_t<decltype(p)>>>::load(p + (unsigned)min(lane + 64 * c, W - 1));
        }
    };
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int row = min(r0 + i, n_rows - 1);
        const int b = row / Sa, s = row % Sa;
        const T* hr = hn + ((long)b * S + n_lead + s) * W;
        load_slots(hr, hv[i]);
    }
    // The rows of W_out are requested together with the activation rows when the norm's own
    // operands leave room for them; with long rows they are requested after the norm instead
    // (holding everything at once overflows the register file, and the compiler then takes
    // the loads one at a time, a round trip to memory each).
    constexpr bool W_EARLY = NORM == EUL_NO_NORM || NC * (ROWS + AU + 2) <= 192;
    auto load_w_rows = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const float* wr = W_out + (long)min(a0 + u, A - 1) * W;
            load_slots(wr, wv[u]);
        }
    };
    if constexpr (W_EARLY) load_w_rows();
    if constexpr (NORM != EUL_NO_NORM) {
        // per-column operands of the norm: the same for every row
        // (loads without a branch around them: a missing weight reads the rows' own memory and
        // the value is dropped; under a branch each load would be waited for on its own)
        float g0[NC], g1[NC];
        const T* gw = norm_w ? norm_w : hn;
        if (NORM == NORM_RMS) {
            load_slots(gw, g0);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                g0[c] = norm_w ? g0[c] : 1.f;
                g1[c] = 0.f;
            }
        } else {
            load_slots(sc, g0);
            load_slots(sh, g1);
        }
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            float mean = 0.f;
            if (NORM == NORM_ADALN) {
                float s1 = 0.f;
#pragma unroll
                for (int c = 0; c < NC; ++c) s1 += (kidx(c) < W) ? hv[i][c] : 0.f;
                mean = wave_sum(s1) / (float)W;
            }
            float s2 = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float d = (kidx(c) < W) ? hv[i][c] - mean : 0.f;
                s2 += d * d;
            }
            const float inv = 1.0f / sqrtf(wave_sum(s2) / (float)W + eps);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                float o;
                if (NORM == NORM_RMS) {
                    o = hv[i][c] * inv;
                    if (norm_w) o *= g0[c];
                } else {
                    const float xn = (hv[i][c] - mean) * inv;
                    o = xn + xn * g0[c] + g1[c];
                }
                hv[i][c] = Elem<T>::round(o);
            }
        }
    }
    if constexpr (!W_EARLY) {
        __builtin_amdgcn_sched_barrier(0);  // not hoisted back in front of the norm
        load_w_rows();
    }
    // The V = ROWS x AU per-lane sums.  From eight sums on they are added across the wavefront
    // together: each exchange step halves the values a lane carries (a lane keeps the upper half
    // of its values if its bit of that step is set and hands the other half to its partner),
    // V - 1 exchanges instead of 6 V, then the remaining steps on the one value left; lane l ends
    // with the total of value l >> (6 - log2 V).  Sixteen sums do the two widest steps with the
    // half-wave and 16-lane-row swaps (both lanes' new values from one instruction); with eight
    // that measured slower than the shuffles, and with fewer than eight the one-sum-at-a-time
    // reduction below is the faster one.
    constexpr int V = ROWS * AU;
    static_assert((V & (V - 1)) == 0 && V <= 64, "a power of two of sums");
    constexpr bool TREE = V >= 8, SWAP = V >= 16;
    constexpr int SH = !TREE ? 0 : V == 8 ? 3 : V == 16 ? 2 : V == 32 ? 1 : 0;
    float vals[V];
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            float acc = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c)
                if (kidx(c) < W) acc += wv[u][c] * hv[i][c];
            if (TREE) {
                vals[i * AU + u] = acc;
            } else {
                acc = wave_sum(acc);
                if (lane == i * AU + u) mine = acc;
            }
        }
    if (TREE) {
        int off = 32;
#pragma unroll
        for (int n = V; n > 1; n >>= 1, off >>= 1) {
            const bool up = (lane & off) != 0;
#pragma unroll
            for (int k = 0; k < n / 2; ++k) {
                const float lo = vals[k], hi = vals[k + n / 2];
                if (SWAP && off == 32) {
                    const auto sw =
                        __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                    vals[k] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
                } else if (SWAP && off == 16) {
                    const auto sw =
                        __builtin_amdgcn_permlane16_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                    vals[k] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
                } else {
                    vals[k] = (up ? hi : lo) + __shfl_xor(up ? lo : hi, off, 64);
                }
            }
        }
        mine = vals[0];
        for (; off > 0; off >>= 1) mine += __shfl_xor(mine, off, 64);
    }
    const int v = lane >> SH;
    const int i = v / AU, a = a0 + v % AU;
    if ((lane & ((1 << SH) - 1)) == 0 && v < V && r0 + i < n_rows && a < A) {
        float* xp = x_t + (long)(r0 + i) * A + a;
        *xp = *xp + dt * (mine + (b_out ? b_out[a] : 0.f));
    }
}

// ------------------------------------------------ BitVLA layer helpers ---
// bitvla_softmax_scaled_bf16 (bitvla_lm_cuda.cu:100-159): in-place, no mask.
__global__ void softmax_scaled_bf16_kernel(bf16_t* __restrict__ inout, float scale, int S) {
    __shared__ float red[16];
    bf16_t* r = inout + (long)blockIdx.x * S;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < S; i += blockDim.x) mx = fmaxf(mx, bf2f(r[i]) * scale);
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int i = threadIdx.x; i < S; i += blockDim.x) sum += expf(bf2f(r[i]) * scale - mx);
    sum = block_sum(sum, red);
    const float inv = 1.0f / sum;
    for (int i = threadIdx.x; i < S; i += blockDim.x) r[i] = f2bf(expf(bf2f(r[i]) * scale - mx) * inv);
}

// BitNet FFN activation on a fused [gate | up] projection (gate_up_fused_sqrelu_mul_bf16,
// src/kernels/bitvla/bitvla_lm_cuda.cu:525-548): out[s][k] = relu(gate)^2 * up, rounded once.
// One thread per 8 columns when ffn allows 16-byte accesses.
__global__ void sqrelu_mul_bf16_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int ffn, long total8) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total8) return;
    const int per_row = ffn / 8;
    const long s = i / per_row;
    const int k = (int)(i % per_row) * 8;
    const u32x4_t g = *reinterpret_cast<const u32x4_t*>(gu + s * 2 * ffn + k);
    const u32x4_t u = *reinterpret_cast<const u32x4_t*>(gu + s * 2 * ffn + ffn + k);
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float g0 = __uint_as_float(g[e] << 16), g1 = __uint_as_float(g[e] & 0xffff0000u);
        const float u0 = __uint_as_float(u[e] << 16), u1 = __uint_as_float(u[e] & 0xffff0000u);
        if (g0 < 0.f) g0 = 0.f;
        if (g1 < 0.f) g1 = 0.f;
        o[e] = (uint32_t)f2bf(g0 * g0 * u0) | ((uint32_t)f2bf(g1 * g1 * u1) << 16);
    }
    *reinterpret_cast<u32x4_t*>(out + s * ffn + k) = o;
}
__global__ void sqrelu_mul_bf16_scalar_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int ffn, long total) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long s = i / ffn;
    const int k = (int)(i % ffn);
    float g = bf2f(gu[s * 2 * ffn + k]);
    const float u = bf2f(gu[s * 2 * ffn + ffn + k]);
    if (g < 0.f) g = 0.f;
    out[i] = f2bf(g * g * u);
}

__global__ void add_bf16_kernel(const bf16_t* a, const bf16_t* b, bf16_t* out, int N) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < N) out[i] = f2bf(bf2f(a[i]) + bf2f(b[i]));
}

// Generic 3-level permuting copy of rows of `hd` elements:
// out[(o0*n1 + o1)*hd + k] = in[(i0*s0 + i1)*hd + k] with per-kernel index maps.
enum { MAP_REPEAT_KV = 0, MAP_SHD_TO_HSD = 1, MAP_HSD_TO_SHD = 2 };
template <int kMap>
__global__ void row_permute_bf16_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out, int a, int b, int c,
                                        int hd) {
    // grid (x, y); meaning depends on kMap (mirrors the reference's launches)
    const int x = blockIdx.x, y = blockIdx.y;
    long src, dst;
    if (kMap == MAP_REPEAT_KV) {  // a=n_q, b=n_kv, c=seq; x=q_h, y=s
        const int kv_h = x * b / a;
        dst = ((long)x * c + y) * hd;
        src = ((long)kv_h * c + y) * hd;
    } else if (kMap == MAP_SHD_TO_HSD) {  // a=S, b=H; x=h, y=s
        dst = ((long)x * a + y) * hd;
        src = ((long)y * b + x) * hd;
    } else {  // MAP_HSD_TO_SHD: a=H, b=S; x=h, y=s
        dst = ((long)y * a + x) * hd;
        src = ((long)x * b + y) * hd;
    }
    for (int k = threadIdx.x; k < hd; k += blockDim.x) out[dst + k] = in[src + k];
}

__global__ void gather_rows_bf16_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out,
                                        const int32_t* __restrict__ ids, int K) {
    const long r = ids[blockIdx.x];
    for (int k = threadIdx.x; k < K; k += blockDim.x) out[(long)blockIdx.x * K + k] = in[r * K + k];
}

// --------------------------------------------------------- act quant ---
// act_quant_kernel (bitnet_kernels.h:465-521) plus the per-row sum of the
// quantised values.  One workgroup per row.
__global__ void act_quant_bf16_kernel(const bf16_t* __restrict__ in, int8_t* __restrict__ out,
                                      float* __restrict__ scales, int32_t* __restrict__ rowsum, int K) {
    __shared__ float red[16];
    __shared__ int redi[16];
    const bf16_t* xr = in + (long)blockIdx.x * K;
    int8_t* qr = out + (long)blockIdx.x * K;
    float amax = 0.f;
    for (int k = threadIdx.x; k < K; k += blockDim.x) amax = fmaxf(amax, fabsf(bf2f(xr[k])));
    amax = block_max(amax, red);
    if (amax < 1e-5f) amax = 1e-5f;
    const float scale = 127.0f / amax;
    int sum = 0;
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        float q = rintf(bf2f(xr[k]) * scale);
        q = fminf(fmaxf(q, -128.0f), 127.0f);
        const int qi = (int)q;
        qr[k] = (int8_t)qi;
        sum += qi;
    }
    sum = wave_sum_i(sum);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) redi[w] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int i = 0; i < nw; ++i) t += redi[i];
        scales[blockIdx.x] = scale;
        if (rowsum) rowsum[blockIdx.x] = t;
    }
}

// RMSNorm (bf16 result) immediately quantised per row to int8: the pair
// bitvla_rmsnorm_bf16 + act_quant in one pass, the row held in registers between the two.
// Same thread <-> element assignment and the same reductions as the separate kernels, so
// the int8 rows, scales and row sums are bit-identical to running them back to back.
constexpr int RNAQ_MAX_PER_THREAD = 16;
__global__ void rmsnorm_act_quant_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, int8_t* __restrict__ out,
                                         float* __restrict__ scales, int32_t* __restrict__ rowsum, int K, float eps) {
    __shared__ float red[16];
    __shared__ int redi[16];
    const bf16_t* xr = x + (long)blockIdx.x * K;
    int8_t* qr = out + (long)blockIdx.x * K;
    float v[RNAQ_MAX_PER_THREAD];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < RNAQ_MAX_PER_THREAD; ++i) {
        const int k = threadIdx.x + i * blockDim.x;
        v[i] = k < K ? bf2f(xr[k]) : 0.f;
        ss += v[i] * v[i];
    }
    ss = block_sum(ss, red);
    const float nscale = 1.0f / sqrtf(ss / (float)K + eps);
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < RNAQ_MAX_PER_THREAD; ++i) {
        const int k = threadIdx.x + i * blockDim.x;
        float n = v[i] * nscale;
        if (w && k < K) n *= bf2f(w[k]);
        v[i] = k < K ? bf2f(f2bf(n)) : 0.f;  // the normalised activation as the bf16 it would be stored as
        amax = fmaxf(amax, fabsf(v[i]));
    }
    amax = block_max(amax, red);
    if (amax < 1e-5f) amax = 1e-5f;
    const float scale = 127.0f / amax;
    int sum = 0;
#pragma unroll
    for (int i = 0; i < RNAQ_MAX_PER_THREAD; ++i) {
        const int k = threadIdx.x + i * blockDim.x;
        if (k >= K) continue;
        float q = rintf(v[i] * scale);
        q = fminf(fmaxf(q, -128.0f), 127.0f);
        const int qi = (int)q;
        qr[k] = (int8_t)qi;
        sum += qi;
    }
    sum = wave_sum_i(sum);
    const int wv = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) redi[wv] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int i = 0; i < nw; ++i) t += redi[i];
        scales[blockIdx.x] = scale;
        if (rowsum) rowsum[blockIdx.x] = t;
    }
}

inline int row_threads(int K) { return K >= 2048 ? 256 : (K >= 512 ? 128 : 64); }

}  // namespace

namespace {
template <int MODE>
int mod_norm(const void* x, const float* sc, const float* sh, void* y, int dtype, int M, int K, float eps,
                    vla_stream_t stream) {
    if (!x || !y || !sc || !sh || M < 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M == 0) return VLA_K_OK;
    hipStream_t st = (hipStream_t)stream;
    const int th = row_threads(K);
    if (dtype == VLA_DT_F32 && launch_row_norm<float, MODE>(x, nullptr, sc, sh, y, nullptr, nullptr, nullptr, M, K, eps, st))
        return VLA_CHECK_LAUNCH();
    if (dtype == VLA_DT_BF16 && launch_row_norm<bf16_t, MODE>(x, nullptr, sc, sh, y, nullptr, nullptr, nullptr, M, K, eps, st))
        return VLA_CHECK_LAUNCH();
    const int rms = MODE == NORM_ADARMS;
    if (dtype == VLA_DT_F32)
        adaln_kernel<float><<<M, th, 0, st>>>((const float*)x, sc, sh, (float*)y, K, eps, rms);
    else if (dtype == VLA_DT_BF16)
        adaln_kernel<bf16_t><<<M, th, 0, st>>>((const bf16_t*)x, sc, sh, (bf16_t*)y, K, eps, rms);
    else
        return VLA_K_ERR_ARG;
    return VLA_CHECK_LAUNCH();
}

}  // namespace

namespace {
// norm < 0: hn is already normalised.  Otherwise one of row_norm_kernel's modes, applied to
// the rows inside the launch.
int euler_launch(float* x_t, const void* hn, int norm, const void* norm_w, const float* sc, const float* sh, float eps,
                 const float* W_out, const float* b_out, int dtype, int batch, int S, int n_lead, int A, int W, float dt,
                 vla_stream_t stream) {
    if (!x_t || !hn || !W_out || batch < 0 || S <= 0 || n_lead < 0 || n_lead >= S || A <= 0 || W <= 0)
        return VLA_K_ERR_ARG;
    if (batch == 0) return VLA_K_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype != VLA_DT_F32 && dtype != VLA_DT_BF16) return VLA_K_ERR_ARG;
    if (W > 64 * 64) return VLA_K_ERR_SHAPE;
    const int n_rows = batch * (S - n_lead);
    // runs of eight with 16-byte loads when every row starts on a 16-byte boundary
    const bool vec = W % 8 == 0 && (((uintptr_t)hn | (uintptr_t)W_out | (uintptr_t)norm_w | (uintptr_t)sc | (uintptr_t)sh) & 15) == 0;
#define VLA_EULER_V(T, NC, AU, ROWS, NORM, VEC)                                                                     \
    euler_step_kernel<T, NC, AU, ROWS, NORM, VEC>                                                                   \
        <<<dim3((n_rows + EUL_WAVES * ROWS - 1) / (EUL_WAVES * ROWS), (A + AU - 1) / AU), EUL_WAVES * 64, 0, st>>>(  \
            x_t, (const T*)hn, W_out, b_out, n_rows, S, n_lead, A, W, dt, (const T*)norm_w, sc, sh, eps)
#define VLA_EULER_N(T, NC, AU, ROWS, NORM)                               \
    do {                                                                 \
        if (vec && (NC) % 8 == 0) VLA_EULER_V(T, (NC) % 8 ? 8 : (NC), AU, ROWS, NORM, true); \
        else VLA_EULER_V(T, NC, AU, ROWS, NORM, false);                  \
    } while (0)
#define VLA_EULER(T, NC, AU, ROWS)                                       \
    do {                                                                 \
        if (norm == NORM_RMS) VLA_EULER_N(T, NC, AU, ROWS, NORM_RMS);    \
        else if (norm == NORM_ADALN) VLA_EULER_N(T, NC, AU, ROWS, NORM_ADALN);   \
        else if (norm == NORM_ADARMS) VLA_EULER_N(T, NC, AU, ROWS, NORM_ADARMS); \
        else VLA_EULER_N(T, NC, AU, ROWS, EUL_NO_NORM);                  \
    } while (0)
#define VLA_EULER_T(T)                                      \
    do {                                                    \
        if (W <= 64 * 8) VLA_EULER(T, 8, 8, 2);             \
        else if (W <= 64 * 12 && !vec) VLA_EULER(T, 12, 8, 2); \
        else if (W <= 64 * 16) VLA_EULER(T, 16, 8, 2);      \
        else if (W <= 64 * 24) VLA_EULER(T, 24, 4, 2);      \
        else if (W <= 64 * 32) VLA_EULER(T, 32, 4, 2);      \
        else VLA_EULER(T, 64, 2, 1);                        \
    } while (0)
    if (dtype == VLA_DT_F32)
        VLA_EULER_T(float);
    else
        VLA_EULER_T(bf16_t);
#undef VLA_EULER_T
#undef VLA_EULER
#undef VLA_EULER_N
#undef VLA_EULER_V
    return VLA_CHECK_LAUNCH();
}
}  // namespace

extern "C" {

int vla_rope_tables_host(const int32_t* pos, int n, int head_dim, double base, float* cos_tab, float* sin_tab) {
    if (!pos || !cos_tab || !sin_tab || n < 0 || head_dim <= 0 || (head_dim & 1)) return VLA_K_ERR_ARG;
    const int half = head_dim / 2;
    for (int s = 0; s < n; ++s)
        for (int i = 0; i < half; ++i) {
            const double ang = (double)pos[s] * pow(base, -2.0 * (double)i / (double)head_dim);
            cos_tab[(size_t)s * half + i] = (float)cos(ang);
            sin_tab[(size_t)s * half + i] = (float)sin(ang);
        }
    return VLA_K_OK;
}

int vla_rope_neox(void* x, const float* cos_tab, const float* sin_tab, int dtype, int n_rows, int table_rows,
                  int n_heads, int head_dim, vla_stream_t stream) {
    if (!x || !cos_tab || !sin_tab || n_rows < 0 || table_rows <= 0 || n_heads <= 0) return VLA_K_ERR_ARG;
    if (head_dim <= 0 || (head_dim & 1)) return VLA_K_ERR_SHAPE;
    const long total = (long)n_rows * n_heads * (head_dim / 2);
    if (total == 0) return VLA_K_OK;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VLA_DT_F32)
        rope_neox_kernel<float><<<blocks, 256, 0, st>>>((float*)x, cos_tab, sin_tab, table_rows, n_heads, head_dim, total);
    else if (dtype == VLA_DT_BF16)
        rope_neox_kernel<bf16_t><<<blocks, 256, 0, st>>>((bf16_t*)x, cos_tab, sin_tab, table_rows, n_heads, head_dim, total);
    else
        return VLA_K_ERR_ARG;
    return VLA_CHECK_LAUNCH();
}

int vla_qkv_split_rope_append(const void* qkv, const float* cos_tab, const float* sin_tab, void* q_out, void* k_cache,
                              void* vt_cache, int dtype, int M, int S, int n_q_heads, int n_kv_heads, int head_dim,
                              int t_max, int tok_offset, vla_stream_t stream) {
    if (!qkv || !q_out || !k_cache || !vt_cache || M < 0 || S <= 0 || n_q_heads <= 0 || n_kv_heads <= 0)
        return VLA_K_ERR_ARG;
    if ((cos_tab == nullptr) != (sin_tab == nullptr)) return VLA_K_ERR_ARG;
    if (head_dim <= 0 || (head_dim & 1) || M % S || tok_offset < 0 || tok_offset + S > t_max) return VLA_K_ERR_SHAPE;
    const long total = (long)M * (n_q_heads + 2 * n_kv_heads) * (head_dim / 2);
    if (total == 0) return VLA_K_OK;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VLA_DT_F32)
        qkv_split_rope_append_kernel<float><<<blocks, 256, 0, st>>>((const float*)qkv, cos_tab, sin_tab, (float*)q_out,
                                                                   (float*)k_cache, (float*)vt_cache, S, n_q_heads,
                                                                   n_kv_heads, head_dim, t_max, tok_offset, total);
    else if (dtype == VLA_DT_BF16)
        qkv_split_rope_append_kernel<bf16_t><<<blocks, 256, 0, st>>>((const bf16_t*)qkv, cos_tab, sin_tab, (bf16_t*)q_out,
                                                                    (bf16_t*)k_cache, (bf16_t*)vt_cache, S, n_q_heads,
                                                                    n_kv_heads, head_dim, t_max, tok_offset, total);
    else
        return VLA_K_ERR_ARG;
    return VLA_CHECK_LAUNCH();
}

int vla_rms_norm(const void* x, const void* w, void* y, int dtype, int M, int K, float eps, vla_stream_t stream) {
    if (!x || !y || M < 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M == 0) return VLA_K_OK;
    hipStream_t st = (hipStream_t)stream;
    const int th = row_threads(K);
    if (dtype == VLA_DT_F32 && launch_row_norm<float, NORM_RMS>(x, w, nullptr, nullptr, y, nullptr, nullptr, nullptr, M, K, eps, st))
        return VLA_CHECK_LAUNCH();
    if (dtype == VLA_DT_BF16 && launch_row_norm<bf16_t, NORM_RMS>(x, w, nullptr, nullptr, y, nullptr, nullptr, nullptr, M, K, eps, st))
        return VLA_CHECK_LAUNCH();
    if (dtype == VLA_DT_F32)
        rms_norm_kernel<float><<<M, th, 0, st>>>((const float*)x, (const float*)w, (float*)y, K, eps);
    else if (dtype == VLA_DT_BF16)
        rms_norm_kernel<bf16_t><<<M, th, 0, st>>>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, K, eps);
    else
        return VLA_K_ERR_ARG;
    return VLA_CHECK_LAUNCH();
}

int vla_adaln(const void* x, const float* sc, const float* sh, void* y, int dtype, int M, int K, float eps,
              vla_stream_t stream) {
    return mod_norm<NORM_ADALN>(x, sc, sh, y, dtype, M, K, eps, stream);
}

int vla_adarms(const void* x, const float* sc, const float* sh, void* y, int dtype, int M, int K, float eps,
               vla_stream_t stream) {
    return mod_norm<NORM_ADARMS>(x, sc, sh, y, dtype, M, K, eps, stream);
}

int vla_embed_suffix(const float* x_t, const float* W_in, const float* bias_step, const float* lead, void* h,
                     int out_dtype, int batch, int S, int n_lead, int A, int W, vla_stream_t stream) {
    return vla_embed_suffix_act(x_t, W_in, bias_step, lead, h, out_dtype, batch, S, n_lead, A, W, VLA_ACT_NONE, stream);
}

int vla_set_lead_rows(const float* lead, void* h, int dtype, int batch, int S, int n_lead, int W, vla_stream_t stream) {
    if (!lead || !h || batch < 0 || S <= 0 || n_lead <= 0 || n_lead > S || W <= 0) return VLA_K_ERR_ARG;
    if (batch == 0) return VLA_K_OK;
    const long total = (long)batch * n_lead * W;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (dtype == VLA_DT_F32) lead_rows_kernel<float><<<blocks, 256, 0, (hipStream_t)stream>>>(lead, (float*)h, total, S, n_lead, W);
    else if (dtype == VLA_DT_BF16) lead_rows_kernel<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>(lead, (bf16_t*)h, total, S, n_lead, W);
    else return VLA_K_ERR_ARG;
    return VLA_CHECK_LAUNCH();
}

int vla_finish_suffix_rows(const float* acc, const float* row_table, const float* lead, void* h, int dtype, int batch, int S,
                           int n_lead, int W, vla_stream_t stream) {
    if (!acc || !h || batch < 0 || S <= 0 || n_lead < 0 || n_lead > S || W <= 0 || (n_lead > 0 && !lead)) return VLA_K_ERR_ARG;
    if (batch == 0) return VLA_K_OK;
    const long total = (long)batch * S * W;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (dtype == VLA_DT_F32)
        finish_suffix_rows_kernel<float><<<blocks, 256, 0, (hipStream_t)stream>>>(acc, row_table, lead, (float*)h, total, S, n_lead, W);
    else if (dtype == VLA_DT_BF16)
        finish_suffix_rows_kernel<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>(acc, row_table, lead, (bf16_t*)h, total, S, n_lead, W);
    else
        return VLA_K_ERR_ARG;
    return VLA_CHECK_LAUNCH();
}

int vla_embed_suffix_act(const float* x_t, const float* W_in, const float* bias_step, const float* lead, void* h,
                         int out_dtype, int batch, int S, int n_lead, int A, int W, int act, vla_stream_t stream) {
    if (!x_t || !W_in || !bias_step || !h || batch < 0 || S <= 0 || n_lead < 0 || n_lead > S || A <= 0 || W <= 0)
        return VLA_K_ERR_ARG;
    if (act < VLA_ACT_NONE || act > VLA_ACT_RELU) return VLA_K_ERR_ARG;
    if (n_lead > 0 && !lead) return VLA_K_ERR_ARG;
    if (A > EMB_WIDE_A) return VLA_K_ERR_SHAPE;
    if (batch == 0) return VLA_K_OK;
    hipStream_t st = (hipStream_t)stream;
    const int n_rows = batch * S;
    const dim3 blocks((n_rows + EMB_ROWS - 1) / EMB_ROWS, (W + EMB_COLS - 1) / EMB_COLS);
    const bool narrow = A <= 32;  // half the staging passes
    const bool wide = A > EMB_MAX_A;
    if (out_dtype == VLA_DT_F32) {
        if (narrow) embed_suffix_kernel<float, 32><<<blocks, 256, 0, st>>>(x_t, W_in, bias_step, lead, (float*)h, n_rows, S, n_lead, A, W, act);
        else if (wide) embed_suffix_kernel<float, EMB_WIDE_A><<<blocks, 256, 0, st>>>(x_t, W_in, bias_step, lead, (float*)h, n_rows, S, n_lead, A, W, act);
        else embed_suffix_kernel<float><<<blocks, 256, 0, st>>>(x_t, W_in, bias_step, lead, (float*)h, n_rows, S, n_lead, A, W, act);
    } else if (out_dtype == VLA_DT_BF16) {
        if (narrow) embed_suffix_kernel<bf16_t, 32><<<blocks, 256, 0, st>>>(x_t, W_in, bias_step, lead, (bf16_t*)h, n_rows, S, n_lead, A, W, act);
        else if (wide) embed_suffix_kernel<bf16_t, EMB_WIDE_A><<<blocks, 256, 0, st>>>(x_t, W_in, bias_step, lead, (bf16_t*)h, n_rows, S, n_lead, A, W, act);
        else embed_suffix_kernel<bf16_t><<<blocks, 256, 0, st>>>(x_t, W_in, bias_step, lead, (bf16_t*)h, n_rows, S, n_lead, A, W, act);
    } else {
        return VLA_K_ERR_ARG;
    }
    return VLA_CHECK_LAUNCH();
}

int vla_euler_step(float* x_t, const void* hn, const float* W_out, const float* b_out, int dtype, int batch, int S,
                   int n_lead, int A, int W, float dt, vla_stream_t stream) {
    return euler_launch(x_t, hn, EUL_NO_NORM, nullptr, nullptr, nullptr, 0.f, W_out, b_out, dtype, batch, S, n_lead, A, W, dt,
                        stream);
}

int vla_rmsnorm_euler_step(float* x_t, const void* h, const void* norm_w, float eps, const float* W_out, const float* b_out,
                           int dtype, int batch, int S, int n_lead, int A, int W, float dt, vla_stream_t stream) {
    if (!h) return VLA_K_ERR_ARG;
    return euler_launch(x_t, h, NORM_RMS, norm_w, nullptr, nullptr, eps, W_out, b_out, dtype, batch, S, n_lead, A, W, dt, stream);
}

int vla_adanorm_euler_step(float* x_t, const void* h, const float* scale, const float* shift, int centred, float eps,
                           const float* W_out, const float* b_out, int dtype, int batch, int S, int n_lead, int A, int W,
                           float dt, vla_stream_t stream) {
    if (!h || !scale || !shift) return VLA_K_ERR_ARG;
    return euler_launch(x_t, h, centred ? NORM_ADALN : NORM_ADARMS, nullptr, scale, shift, eps, W_out, b_out, dtype, batch, S,
                        n_lead, A, W, dt, stream);
}

int vla_act_quant_bf16(const uint16_t* in, int8_t* out, float* scales, int32_t* rowsum, int M, int K,
                       vla_stream_t stream) {
    if (!in || !out || !scales || M < 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M == 0) return VLA_K_OK;
    act_quant_bf16_kernel<<<M, 256, 0, (hipStream_t)stream>>>(in, out, scales, rowsum, K);
    return VLA_CHECK_LAUNCH();
}

int vla_rmsnorm_act_quant_bf16(const uint16_t* x, const uint16_t* w, int8_t* out, float* scales, int32_t* rowsum, float eps,
                               int M, int K, vla_stream_t stream) {
    if (!x || !out || !scales || M < 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M == 0) return VLA_K_OK;
    if (launch_row_norm<bf16_t, NORM_RMS_AQ>(x, w, nullptr, nullptr, nullptr, out, scales, rowsum, M, K, eps, (hipStream_t)stream))
        return VLA_CHECK_LAUNCH();
    int th = row_threads(K);
    while (K > th * RNAQ_MAX_PER_THREAD && th < 1024) th *= 2;  // long rows (the 6912-wide BitNet FFN): up to 16 wavefronts
    if (K > th * RNAQ_MAX_PER_THREAD) return VLA_K_ERR_SHAPE;
    rmsnorm_act_quant_kernel<<<M, th, 0, (hipStream_t)stream>>>(x, w, out, scales, rowsum, K, eps);
    return VLA_CHECK_LAUNCH();
}

int vla_sqrelu_rmsnorm_act_quant_bf16(const uint16_t* gate_up, const uint16_t* w, int8_t* out, float* scales, int32_t* rowsum,
                                      float eps, int M, int K, vla_stream_t stream) {
    if (!gate_up || !out || !scales || M < 0 || K <= 0) return VLA_K_ERR_ARG;
    if (M == 0) return VLA_K_OK;
    if (!launch_row_norm<bf16_t, NORM_RMS_AQ, true>(gate_up, w, nullptr, nullptr, nullptr, out, scales, rowsum, M, K, eps,
                                                    (hipStream_t)stream))
        return VLA_K_ERR_SHAPE;
    return VLA_CHECK_LAUNCH();
}

int bitvla_act_quant(const uint16_t* in, int8_t* out, float* scales, int M, int K, vla_stream_t stream) {
    return vla_act_quant_bf16(in, out, scales, nullptr, M, K, stream);
}

int bitvla_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* out, float eps, int M, int K,
                        vla_stream_t stream) {
    return vla_rms_norm(x, w, out, VLA_DT_BF16, M, K, eps, stream);
}

int bitvla_rope_neox_bf16(uint16_t* inout, const float* cos_tab, const float* sin_tab, int H, int S, int D,
                          vla_stream_t stream) {
    if (!inout || !cos_tab || !sin_tab || H < 0 || S < 0 || D <= 0 || (D & 1)) return VLA_K_ERR_ARG;
    const long total = (long)H * S * (D / 2);
    if (total == 0) return VLA_K_OK;
    rope_neox_hsd_bf16_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(inout, cos_tab,
                                                                                               sin_tab, S, D, total);
    return VLA_CHECK_LAUNCH();
}

int bitvla_softmax_scaled_bf16(uint16_t* inout, float scale, int n_rows, int S, vla_stream_t stream) {
    if (!inout || n_rows < 0 || S <= 0) return VLA_K_ERR_ARG;
    if (n_rows == 0) return VLA_K_OK;
    softmax_scaled_bf16_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>(inout, scale, S);
    return VLA_CHECK_LAUNCH();
}

int bitvla_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out, int N, vla_stream_t stream) {
    if (!a || !b || !out || N < 0) return VLA_K_ERR_ARG;
    if (N == 0) return VLA_K_OK;
    add_bf16_kernel<<<(N + 255) / 256, 256, 0, (hipStream_t)stream>>>(a, b, out, N);
    return VLA_CHECK_LAUNCH();
}

int gate_up_fused_sqrelu_mul_bf16(const uint16_t* gu, uint16_t* out, int seq, int ffn, vla_stream_t stream) {
    if (!gu || !out || seq < 0 || ffn <= 0) return VLA_K_ERR_ARG;
    if (seq == 0) return VLA_K_OK;
    const long total = (long)seq * ffn;
    if (ffn % 8 == 0 && !(((uintptr_t)gu | (uintptr_t)out) & 15))
        sqrelu_mul_bf16_kernel<<<(unsigned)((total / 8 + 255) / 256), 256, 0, (hipStream_t)stream>>>(gu, out, ffn, total / 8);
    else
        sqrelu_mul_bf16_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(gu, out, ffn, total);
    return VLA_CHECK_LAUNCH();
}

int bitvla_repeat_kv_bf16(const uint16_t* in, uint16_t* out, int n_q, int n_kv, int seq, int hd, vla_stream_t stream) {
    if (!in || !out || n_q <= 0 || n_kv <= 0 || seq < 0 || hd <= 0) return VLA_K_ERR_ARG;
    if (n_q % n_kv != 0) return VLA_K_ERR_SHAPE;
    if (seq == 0) return VLA_K_OK;
    row_permute_bf16_kernel<MAP_REPEAT_KV><<<dim3(n_q, seq), 64, 0, (hipStream_t)stream>>>(in, out, n_q, n_kv, seq, hd);
    return VLA_CHECK_LAUNCH();
}

int bitvla_transpose_sNhd_to_NshHd_bf16(const uint16_t* in, uint16_t* out, int S, int N, int hd, vla_stream_t stream) {
    if (!in || !out || S < 0 || N <= 0 || hd <= 0) return VLA_K_ERR_ARG;
    if (S == 0) return VLA_K_OK;
    row_permute_bf16_kernel<MAP_SHD_TO_HSD><<<dim3(N, S), 64, 0, (hipStream_t)stream>>>(in, out, S, N, 0, hd);
    return VLA_CHECK_LAUNCH();
}

int bitvla_transpose_NshHd_to_sNhd_bf16(const uint16_t* in, uint16_t* out, int N, int S, int hd, vla_stream_t stream) {
    if (!in || !out || S < 0 || N <= 0 || hd <= 0) return VLA_K_ERR_ARG;
    if (S == 0) return VLA_K_OK;
    row_permute_bf16_kernel<MAP_HSD_TO_SHD><<<dim3(N, S), 64, 0, (hipStream_t)stream>>>(in, out, N, S, 0, hd);
    return VLA_CHECK_LAUNCH();
}

int bitvla_gather_rows_bf16(const uint16_t* in, uint16_t* out, const int32_t* row_ids, int n_rows, int K,
                            vla_stream_t stream) {
    if (!in || !out || !row_ids || n_rows < 0 || K <= 0) return VLA_K_ERR_ARG;
    if (n_rows == 0) return VLA_K_OK;
    gather_rows_bf16_kernel<<<n_rows, 128, 0, (hipStream_t)stream>>>(in, out, row_ids, K);
    return VLA_CHECK_LAUNCH();
}

}  // extern "C"
