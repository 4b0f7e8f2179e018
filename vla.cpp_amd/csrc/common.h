// Shared device helpers for the gfx950 kernels: bf16 bit conversions, vector
// types, wavefront (64-lane) reductions and the MFMA fragment typedefs.
#pragma once
#include "vla_kernels.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#define VLA_WAVE 64

#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "these kernels are written for gfx950 (MI355X) only"
#endif

namespace vk {

// Overrides of the by-shape kernel selection, for tests and tuning.  Read from the
// environment once (vla_kernels_init, or the first launch that asks) and again only by
// vla_kernels_reload_env: no launch path calls getenv.
struct Tuning {
    int attn_dl = -1;           // VLA_ATTN_DL: 0 pins the register-staged LDS kernel for 64-wide bf16 heads
    int attn_slices = 0;        // VLA_ATTN_SLICES: 1 | 2 key slices per row tile in the direct-to-LDS kernel
    int attn_split = -1;        // VLA_ATTN_SPLIT: key slices across workgroups (<= 0 pins one)
    bool attn_split_set = false;
    bool attn_part_f32 = false;  // VLA_ATTN_PART_F32: fp32 partials where fp16 would be used
    bool attn_no_arrive = false; // VLA_ATTN_NO_ARRIVE: no in-launch merge by the last slice to arrive
    bool attn_no_direct = false; // VLA_ATTN_NO_DIRECT: never the register-direct kernel
    bool attn_no_stream = false; // VLA_ATTN_NO_STREAM: never the streaming (LDS-ring) form of the register-direct kernel
    int gemm_rows_max = 32;      // VLA_GEMM_ROWS_MAX: bf16 projections of at most this many rows (up to 64) take the split-K kernel, 0 = never
    bool attn_no_small = false;  // VLA_ATTN_NO_SMALL: fp32 launches with few row tiles do not split their keys beyond the usual rule
    int attn_direct_rows = 32;   // VLA_ATTN_DIRECT_ROWS: row limit of the register-direct kernel
    int gemm_tile = -1;          // VLA_GEMM_TILE: 0..5
    int gemm_panel = 0;          // VLA_GEMM_PANEL: N tiles per panel of an XCD's walk over its tiles; 0 = by size
    int gemm_dl = -1;            // VLA_GEMM_DL: 0 pins the register-staged GEMM
    int gemm_stages = 0;         // VLA_GEMM_STAGES: ring depth of the direct-to-LDS GEMM
    int ternary_tile = 0;        // VLA_TERNARY_TILE: 64 | 128 | 256 (32x32x32 kernels) | 16 (16x16x64 kernel)
};
const Tuning& tuning();

// Scratch memory the library owns on behalf of entry points whose signature has no
// workspace argument: one block per (purpose, device, stream), grown on demand and never
// freed before the process ends, so a captured graph that holds an older block keeps
// pointing at live memory and calls on different streams never share a block.  New blocks
// are zero-filled.  Allocates (never under stream capture: run a shape once before
// capturing it).  Returns nullptr when the allocation fails.
enum { SCRATCH_ATTN = 0, SCRATCH_ROWSUM = 1 };
void* stream_scratch(int purpose, hipStream_t stream, size_t bytes);

typedef uint16_t bf16_t;  // raw bf16 bits

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef uint16_t u16x4_t __attribute__((ext_vector_type(4)));
typedef uint16_t u16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// bf16 <-> f32, round to nearest even, NaN quieted: the hardware converter (v_cvt_pk_bf16_f32),
// one instruction where the integer formulation takes seven.
__device__ __forceinline__ float bf2f(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ bf16_t f2bf(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }
// Two floats -> packed bf16 pair with the hardware converter (v_cvt_pk_bf16_f32,
// round to nearest even).
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Element traits: storage type <-> float.
template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int kVec = 4;  // elements per 16-byte vector
    __device__ static __forceinline__ float load(const float* p) { return *p; }
    __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
    __device__ static __forceinline__ float round(float v) { return v; }  // the value a store and a load would give back
};
template <> struct Elem<bf16_t> {
    static constexpr int kVec = 8;
    __device__ static __forceinline__ float load(const bf16_t* p) { return bf2f(*p); }
    __device__ static __forceinline__ void store(bf16_t* p, float v) { *p = f2bf(v); }
    __device__ static __forceinline__ float round(float v) { return bf2f(f2bf(v)); }
};

// 64-lane wavefront reductions; every lane ends with the result.  No trip through LDS (a
// ds_bpermute butterfly costs six dependent LDS round trips, which is most of the time of a
// kernel that is one wavefront's chain of dependent steps): inside a row of 16 lanes the
// partners come from DPP operands (neighbour, neighbour pair, the mirrored half, the
// mirrored row), the four rows are combined by gfx950's row swaps (v_permlane16_swap of a
// register with itself leaves rows (0, 0, 2, 2) in one copy and (1, 1, 3, 3) in the other;
// v_permlane32_swap does the same for the halves).  Both partners of a step form the same
// sum of the same two values, so every lane ends with the same bits.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_ROW_MIRROR = 0x140;
template <typename Op>
__device__ __forceinline__ uint32_t wave_combine_u32(uint32_t v, Op op) {
    v = op(v, dpp_u32<DPP_XOR1>(v));
    v = op(v, dpp_u32<DPP_XOR2>(v));
    v = op(v, dpp_u32<DPP_HALF_MIRROR>(v));
    v = op(v, dpp_u32<DPP_ROW_MIRROR>(v));
    u32x2_t r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = op(r[0], r[1]);
    r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return op(r[0], r[1]);
}
__device__ __forceinline__ float wave_max(float v) {
    return __uint_as_float(wave_combine_u32(__float_as_uint(v), [](uint32_t a, uint32_t b) {
        return __float_as_uint(fmaxf(__uint_as_float(a), __uint_as_float(b)));
    }));
}
__device__ __forceinline__ float wave_sum(float v) {
    return __uint_as_float(wave_combine_u32(__float_as_uint(v), [](uint32_t a, uint32_t b) {
        return __float_as_uint(__uint_as_float(a) + __uint_as_float(b));
    }));
}
__device__ __forceinline__ int wave_sum_i(int v) {
    return (int)wave_combine_u32((uint32_t)v, [](uint32_t a, uint32_t b) { return a + b; });
}

// A value combined over the two halves of the wavefront (lanes r and r + 32): one row swap
// instead of a trip through LDS.
__device__ __forceinline__ float halves_max(float x) {
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float x) {
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// A value combined over the four 16-lane rows of the wavefront (lanes c, c + 16, c + 32, c + 48)
// with gfx950's row swaps instead of two trips through LDS: after v_permlane16_swap of a register
// with itself one copy holds rows (0, 0, 2, 2) and the other rows (1, 1, 3, 3); v_permlane32_swap does
// the same for the two halves.
__device__ __forceinline__ float rows_max(float x) {
    u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float rows_sum(float x) {
    u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Block reductions through LDS for blocks of up to 16 wavefronts.  `red` holds
// at least 16 floats.  All threads of the block must call.
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < nw; ++i) r = fmaxf(r, red[i]);
    return r;
}
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; ++i) r += red[i];
    return r;
}

// One bf16 row through RMSNorm and the per-row int8 quantisation of the BitNet activations,
// by one wavefront (bitvla_rmsnorm_bf16 then act_quant, src/kernels/bitnet_kernels.h:49-54,
// without the round trip): lane L holds the 16-byte vectors L, L + 64, ... of the row, NV of
// them.  y = x * rsqrt(mean(x^2) + eps) * w is rounded to bf16 as it would be stored; the
// scale is 127 / max(amax, 1e-5); q = clamp(round-half-even(y * scale)).  The int8 row goes
// to qrow (global or LDS, 8 bytes per vector); scale and the sum of the row's int8 values
// are returned in every lane.  K % 8 == 0 and K <= 512 NV.
// GLU: the row is formed on the fly from a fused projection, x[k] = bf16(relu(gate[k])^2 * up[k])
// with gate = xr and up = xr + K (gate_up_fused_sqrelu_mul_bf16, src/kernels/bitvla/bitvla_lm_cuda.cu:525-548).
// WAVES > 1: the row is shared by the WAVES wavefronts of a workgroup (`lane` = the thread's
// index in it, vectors lane, lane + 64 WAVES, ...; `red` = 16 floats of LDS for the three
// reductions; every thread of the workgroup calls).  The squares are then added in another
// order than by one wavefront, so the two forms agree to rounding, not bit for bit.
template <int NV, bool GLU = false, int WAVES = 1>
__device__ __forceinline__ void rms_act_quant_row(const bf16_t* __restrict__ xr, const bf16_t* __restrict__ w, int K,
                                                  float eps, int lane, int8_t* qrow, float& scale_out, int& sum_out,
                                                  float* red = nullptr) {
    constexpr int LS = 64 * WAVES;  // vectors per pass over the row
    const int nvec = K / 8;
    // Every value kept between the passes is a bf16 (the input, then the rounded normalised
    // row), so the row stays packed: 4 registers per 16-byte vector.
    u32x4_t xp[NV];
    u32x4_t wraw[NV];  // the weight's vectors, requested with the row's so that one round trip covers both
    const bool w_vec = w && !((uintptr_t)w & 15);
    auto lo = [](uint32_t u) { return __uint_as_float(u << 16); };
    auto hi = [](uint32_t u) { return __uint_as_float(u & 0xffff0000u); };
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int vec = lane + LS * i;
        u32x4_t raw = {0u, 0u, 0u, 0u}, upr = {0u, 0u, 0u, 0u};
        wraw[i] = raw;
        if (vec < nvec) {
            raw = *reinterpret_cast<const u32x4_t*>(xr + (long)vec * 8);
            if (GLU) upr = *reinterpret_cast<const u32x4_t*>(xr + K + (long)vec * 8);
            if (w_vec) wraw[i] = *reinterpret_cast<const u32x4_t*>(w + (long)vec * 8);
        }
        if (GLU) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float g0 = lo(raw[e]), g1 = hi(raw[e]);
                if (g0 < 0.f) g0 = 0.f;
                if (g1 < 0.f) g1 = 0.f;
                raw[e] = pack_bf2(g0 * g0 * lo(upr[e]), g1 * g1 * hi(upr[e]));
            }
        }
        xp[i] = raw;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = lo(xp[i][e]), b = hi(xp[i][e]);
            ss += a * a;
            ss += b * b;
        }
    const float inv = 1.0f / sqrtf((WAVES > 1 ? block_sum(ss, red) : wave_sum(ss)) / (float)K + eps);
    // the packed words are opaque from here on, or the compiler keeps the first pass's unpacked
    // floats alive across the reduction (8 registers per vector instead of 4)
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) asm volatile("" : "+v"(xp[i][e]));
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int vec = lane + LS * i;
        if (vec >= nvec) continue;
        const int k0 = vec * 8;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float o0 = lo(xp[i][e]) * inv, o1 = hi(xp[i][e]) * inv;
            if (w_vec) {
                o0 *= lo(wraw[i][e]);
                o1 *= hi(wraw[i][e]);
            } else if (w) {
                o0 *= bf2f(w[k0 + 2 * e]);
                o1 *= bf2f(w[k0 + 2 * e + 1]);
            }
            const uint32_t pr = pack_bf2(o0, o1);  // the activation as the bf16 it would be stored as
            xp[i][e] = pr;
            amax = fmaxf(amax, fmaxf(fabsf(lo(pr)), fabsf(hi(pr))));
        }
    }
    amax = WAVES > 1 ? block_max(amax, red) : wave_max(amax);
    if (amax < 1e-5f) amax = 1e-5f;
    const float scale = 127.0f / amax;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) asm volatile("" : "+v"(xp[i][e]));
    int sum = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int vec = lane + LS * i;
        if (vec >= nvec) continue;
        uint32_t pk[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t u = xp[i][e >> 1];
            float qf = rintf(((e & 1) ? hi(u) : lo(u)) * scale);
            qf = fminf(fmaxf(qf, -128.0f), 127.0f);
            pk[e >> 2] |= (uint32_t)((int)qf & 0xff) << (8 * (e & 3));
        }
        sum = __builtin_amdgcn_sdot4((int)pk[0], 0x01010101, sum, false);  // + the four signed bytes
        sum = __builtin_amdgcn_sdot4((int)pk[1], 0x01010101, sum, false);
        *reinterpret_cast<u32x2_t*>(qrow + (long)vec * 8) = u32x2_t{pk[0], pk[1]};
    }
    scale_out = scale;
    sum = wave_sum_i(sum);
    if (WAVES > 1) {  // exact in any order
        int* redi = reinterpret_cast<int*>(red);
        __syncthreads();
        if ((lane & 63) == 0) redi[lane >> 6] = sum;
        __syncthreads();
        sum = 0;
        for (int i = 0; i < WAVES; ++i) sum += redi[i];
    }
    sum_out = sum;
}

// ggml_silu / ggml_gelu (tanh form) / ggml_relu, fp32 (src/layers/ffn.h:24-40, src/modules/action_expert.cpp:41-59).
__device__ __forceinline__ float apply_act(float x, int act) {
    if (act == VLA_ACT_SILU) return x / (1.0f + __expf(-x));
    if (act == VLA_ACT_GELU) return 0.5f * x * (1.0f + tanhf(0.79788456080286535588f * x * (1.0f + 0.044715f * x * x)));
    if (act == VLA_ACT_RELU) return x > 0.f ? x : 0.f;
    return x;
}

// s_waitcnt on the vector-memory counter alone (vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits
// 15:14; the export and LDS/scalar counter fields at their maxima, i.e. not waited on).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
// Division by a launch-wide constant without the divider sequence (some thirty dependent instructions per quotient, in
// front of a kernel's first load): the host forms 2^32 / d + 1 once, the quotient of any x < 2^16 is then the high half
// of one multiplication (exact while d < 2^16).  mg == 0 keeps the plain division (d or the dividends out of range).
struct DivC {
    unsigned d, mg;
};
inline DivC make_divc(long d, long max_x) {
    DivC c;
    c.d = (unsigned)d;
    c.mg = (d > 1 && d < 65536 && max_x < 65536) ? (unsigned)((1ull << 32) / (unsigned long long)d) + 1u : 0u;
    return c;
}
__device__ __forceinline__ unsigned div_c(unsigned x, DivC c) { return c.mg ? __umulhi(x, c.mg) : (c.d == 1 ? x : x / c.d); }

// One 16-byte load per lane from global memory straight into LDS, no register in between:
// lane i's bytes land at lds_base + 16 i (lds_base wavefront-uniform, held in M0); the
// per-lane global address is free.  Completion is tracked by vmcnt like any vector load.
// Issued from inline assembly so that the wait counts stay under this file's control.
__device__ __forceinline__ void load_to_lds16(const void* gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(gptr) : "memory");
}

}  // namespace vk
