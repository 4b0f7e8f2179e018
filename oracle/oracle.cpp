// CPU oracle for the action-expert attention hot path.
//
// TEST INFRASTRUCTURE ONLY.  This file restates, in plain scalar C++, the
// arithmetic the reference (VinRobotics/vla.cpp) performs on this path through
// ggml graph ops and through its in-tree BitVLA kernels.  Only tests, the smoke
// check and the CPU-baseline leg of the benchmark may load it; the shipped
// library never links or calls it.
//
// The reference's own ggml CPU build cannot be compiled here: ggml is the
// third-party module llama.cpp @ tag b10331, fetched from the network by
// CMakeLists.txt:42-51 and not vendored.  Every function below therefore names
// the reference call site it restates, and says how it is pinned:
//
//   pinned by a reference-held vector / in-tree source  : rope pairing
//     (tests/test_rope_conventions.cpp:42-72), time embeddings
//     (tests/test_dit_common.cpp), ternary decode / pack / act-quant / GEMM
//     epilogue (src/kernels/bitvla/bitnet_kernels.h, src/models/bitvla.cpp are
//     complete in-tree definitions).
//   pinned by mathematics (closed forms, invariants, brute force, torch CPU
//     cross-checks in tests/): linear, rms/layer norm, softmax, attention,
//     concat, masks.
//   parity unpinned (exact ggml CPU last-ulp behaviour that only running ggml
//     could show): the fp32 angle evaluation inside ggml_rope_ext, the block
//     order of ggml_flash_attn_ext's online softmax and the reduction order of
//     ggml_mul_mat.  The oracle fixes these as: angles in fp64 rounded once to
//     fp32 cos/sin, exact two-pass softmax, fp64 accumulation.
//
// All matrices are row-major.  "token-major" means [token][head][head_dim],
// which is ggml's [head_dim, n_heads, n_tokens] with ne0 innermost.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

extern "C" {

// ----------------------------------------------------------------------------
// bf16 <-> f32.  Round-to-nearest-even with NaN quieting (what
// ggml_fp32_to_bf16_row and __float2bfloat16 do; the BitVLA upload helper
// src/models/bitvla.cpp:485-488 truncates instead, see orc_f32_to_bf16_trunc).
// ----------------------------------------------------------------------------
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
uint16_t orc_f32_to_bf16_trunc(float f) {  // src/models/bitvla.cpp:485-488
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t)(u >> 16);
}
float orc_bf16_to_f32(uint16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
void orc_round_bf16(const float* x, float* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = orc_bf16_to_f32(orc_f32_to_bf16(x[i]));
}
void orc_to_bf16(const float* x, uint16_t* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = orc_f32_to_bf16(x[i]);
}
void orc_from_bf16(const uint16_t* x, float* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = orc_bf16_to_f32(x[i]);
}

// ----------------------------------------------------------------------------
// RoPE, NeoX / half-split convention.
// ggml_rope_ext(x, pos, nullptr, n_dims=D, NEOX, 0, base, 1, 0, 1, 32, 1) at
// src/models/smolvla.cpp:759-766, src/models/pi0.cpp:182-189,
// src/models/bitvla.cpp:217-218, src/layers/rope.h:40-48; CUDA twin
// rope_neox_bf16_kernel src/kernels/bitvla/bitvla_lm_cuda.cu:77-98 with the
// host table of :333-342.
// theta_i = pos * base^(-2i/D), pairs (i, i + D/2).
// ----------------------------------------------------------------------------
void orc_rope_tables(const int32_t* pos, int n_tok, int D, double base, float* cos_t, float* sin_t) {
    const int half = D / 2;
    for (int s = 0; s < n_tok; ++s)
        for (int i = 0; i < half; ++i) {
            const double ang = (double)pos[s] * std::pow(base, -2.0 * (double)i / (double)D);
            cos_t[(size_t)s * half + i] = (float)std::cos(ang);
            sin_t[(size_t)s * half + i] = (float)std::sin(ang);
        }
}

// The CUDA twin's own fp32 table (bitvla_lm_cuda.cu:333-342): kept so tests can
// bound the distance between the two table definitions.
void orc_rope_tables_f32_powf(int n_tok, int D, float base, float* cos_t, float* sin_t) {
    const int half = D / 2;
    for (int s = 0; s < n_tok; ++s)
        for (int k = 0; k < half; ++k) {
            float freq = 1.0f / std::pow(base, (float)(2 * k) / (float)D);
            float ang = (float)s * freq;
            cos_t[(size_t)s * half + k] = std::cos(ang);
            sin_t[(size_t)s * half + k] = std::sin(ang);
        }
}

// x: [n_tok][n_heads][D] fp32, rotated in place.  (a,b) = (x[i], x[i+D/2]) ->
// (a c - b s, b c + a s): bitvla_lm_cuda.cu:91-96.
void orc_rope_neox(float* x, const float* cos_t, const float* sin_t, int n_tok, int n_heads, int D) {
    const int half = D / 2;
    for (int s = 0; s < n_tok; ++s)
        for (int h = 0; h < n_heads; ++h) {
            float* row = x + ((size_t)s * n_heads + h) * D;
            for (int i = 0; i < half; ++i) {
                const float c = cos_t[(size_t)s * half + i], sn = sin_t[(size_t)s * half + i];
                const float a = row[i], b = row[i + half];
                row[i] = a * c - b * sn;
                row[i + half] = b * c + a * sn;
            }
        }
}

// HuggingFace rotate_half as written in tests/test_rope_conventions.cpp:42-50;
// x*cos + rotate_half(x)*sin is the same rotation as orc_rope_neox.
void orc_rotate_half(const float* x, float* out, int D) {
    const int half = D / 2;
    for (int i = 0; i < half; ++i) {
        out[i] = -x[half + i];
        out[half + i] = x[i];
    }
}

// ----------------------------------------------------------------------------
// ggml_mul_mat(W[K,N], x[K,M]) -> [N,M]: y[m][n] = sum_k W[n][k] x[m][k]
// (+ bias), the shape rule restated at src/act_dtype.h:62-76; call sites
// src/models/smolvla.cpp:771-776,821-823, src/models/pi0.cpp:174-176,
// src/layers/linear.h:24-27.  acc64 != 0 accumulates in double.
// ----------------------------------------------------------------------------
// fp32 dot product the way a SIMD CPU kernel forms it (ggml's vec_dot keeps several vector
// accumulators): 32 independent partial sums with fused multiply-add, combined at the end.
// Used only when acc64 == 0, i.e. by the timed CPU baseline; the parity oracle accumulates
// in double.
static inline float dot_f32_lanes(const float* a, const float* b, int n) {
    float acc[32] = {0.f};
    int k = 0;
    for (; k + 32 <= n; k += 32)
        for (int j = 0; j < 32; ++j) acc[j] = __builtin_fmaf(a[k + j], b[k + j], acc[j]);
    for (; k < n; ++k) acc[k & 31] = __builtin_fmaf(a[k], b[k], acc[k & 31]);
    for (int w = 16; w > 0; w >>= 1)
        for (int j = 0; j < w; ++j) acc[j] += acc[j + w];
    return acc[0];
}

void orc_linear(const float* x, const float* W, const float* b, float* y, int M, int N, int K, int acc64) {
#pragma omp parallel for schedule(static) collapse(2)
    for (int m = 0; m < M; ++m) {
        for (int n = 0; n < N; ++n) {
            const float* xr = x + (size_t)m * K;
            const float* wr = W + (size_t)n * K;
            float out;
            if (acc64) {
                double a = 0.0;
                for (int k = 0; k < K; ++k) a += (double)wr[k] * (double)xr[k];
                out = (float)(a + (b ? (double)b[n] : 0.0));
            } else {
                out = dot_f32_lanes(wr, xr, K) + (b ? b[n] : 0.f);
            }
            y[(size_t)m * N + n] = out;
        }
    }
}

// ----------------------------------------------------------------------------
// ggml_mul(ggml_rms_norm(x, eps), w): src/models/smolvla.cpp:820,
// src/models/pi0.cpp:170, src/layers/norm.h:31-34.  w may be NULL.
// ----------------------------------------------------------------------------
void orc_rms_norm(const float* x, const float* w, float* y, int M, int K, float eps) {
    for (int m = 0; m < M; ++m) {
        const float* xr = x + (size_t)m * K;
        double ss = 0.0;
        for (int k = 0; k < K; ++k) ss += (double)xr[k] * (double)xr[k];
        const float scale = (float)(1.0 / std::sqrt(ss / (double)K + (double)eps));
        for (int k = 0; k < K; ++k) y[(size_t)m * K + k] = xr[k] * scale * (w ? w[k] : 1.f);
    }
}

// ggml_norm(x, eps): (x - mean) / sqrt(var + eps); optional affine
// (src/layers/norm.h:27-29).
void orc_layer_norm(const float* x, const float* w, const float* b, float* y, int M, int K, float eps) {
    for (int m = 0; m < M; ++m) {
        const float* xr = x + (size_t)m * K;
        double mean = 0.0;
        for (int k = 0; k < K; ++k) mean += xr[k];
        mean /= K;
        double var = 0.0;
        for (int k = 0; k < K; ++k) var += ((double)xr[k] - mean) * ((double)xr[k] - mean);
        var /= K;
        const double inv = 1.0 / std::sqrt(var + (double)eps);
        for (int k = 0; k < K; ++k) {
            float v = (float)(((double)xr[k] - mean) * inv);
            if (w) v *= w[k];
            if (b) v += b[k];
            y[(size_t)m * K + k] = v;
        }
    }
}

// adaLN with (scale, shift) conditioning: xn + xn*sc + sh, one (sc, sh) pair of
// length K for all rows (src/layers/norm.h:37-46; used by DitHead::block at
// src/modules/dit_head.cpp:111).
void orc_adaln(const float* x, const float* sc, const float* sh, float* y, int M, int K, float eps) {
    orc_layer_norm(x, nullptr, nullptr, y, M, K, eps);
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            float xn = y[(size_t)m * K + k];
            y[(size_t)m * K + k] = xn + xn * sc[k] + sh[k];
        }
}

float orc_silu(float x) { return x / (1.f + std::exp(-x)); }

// ----------------------------------------------------------------------------
// ggml_concat(cached, suffix, 2) on token-major tensors: a fresh buffer holding
// the P cached token rows followed by the S suffix rows
// (src/models/smolvla.cpp:832-833, src/models/pi0.cpp:198-201).  Byte copy, so
// valid for any element type: `row_bytes` is n_kv_heads*head_dim*elem_size.
// ----------------------------------------------------------------------------
void orc_kv_concat(const void* cache, int64_t P, const void* suffix, int64_t S, int64_t row_bytes, void* out) {
    std::memcpy(out, cache, (size_t)(P * row_bytes));
    std::memcpy((char*)out + P * row_bytes, suffix, (size_t)(S * row_bytes));
}

// ----------------------------------------------------------------------------
// ggml_soft_max_ext(kq, mask, scale, 0): row-wise softmax(scale*kq + mask)
// (src/layers/attn.h:43, src/models/pi0.cpp:219).  In place on kq [rows][T];
// mask [rows][T] additive (0 / -inf) or NULL.
// ----------------------------------------------------------------------------
void orc_softmax_ext(float* kq, const float* mask, float scale, int rows, int T) {
    for (int r = 0; r < rows; ++r) {
        float* row = kq + (size_t)r * T;
        float mx = -std::numeric_limits<float>::infinity();
        for (int t = 0; t < T; ++t) {
            row[t] = row[t] * scale + (mask ? mask[(size_t)r * T + t] : 0.f);
            mx = std::max(mx, row[t]);
        }
        double sum = 0.0;
        for (int t = 0; t < T; ++t) {
            row[t] = std::exp(row[t] - mx);
            sum += row[t];
        }
        const float inv = (float)(1.0 / sum);
        for (int t = 0; t < T; ++t) row[t] *= inv;
    }
}

// The BitVLA CUDA softmax (bitvla_lm_cuda.cu:100-159): no mask, input and
// output bf16, fp32 inside.
void orc_softmax_scaled_bf16(uint16_t* inout, float scale, int rows, int S) {
    std::vector<float> tmp(S);
    for (int r = 0; r < rows; ++r) {
        uint16_t* row = inout + (size_t)r * S;
        float mx = -std::numeric_limits<float>::infinity();
        for (int i = 0; i < S; ++i) {
            tmp[i] = orc_bf16_to_f32(row[i]) * scale;
            mx = std::max(mx, tmp[i]);
        }
        double sum = 0.0;
        for (int i = 0; i < S; ++i) {
            tmp[i] = std::exp(tmp[i] - mx);
            sum += tmp[i];
        }
        const float inv = 1.0f / (float)sum;
        for (int i = 0; i < S; ++i) row[i] = orc_f32_to_bf16(tmp[i] * inv);
    }
}

// ----------------------------------------------------------------------------
// Explicit attention: mul_mat(K,Q) -> soft_max_ext(mask, scale) -> mul_mat(V,.)
// (src/layers/attn.h:38-46, src/models/pi0.cpp:215-223); the flash variant
// (src/models/smolvla.cpp:835-842) is the same mathematics.
// Q [S][Hq][D], K/V [T][Hkv][D] token-major; mask [S][T] or NULL;
// out [S][Hq*D].  GQA by broadcast: kv head = h / (Hq/Hkv), as ggml_mul_mat
// broadcasts and as repeat_kv_bf16_kernel copies (bitvla_lm_cuda.cu:181-190).
// ----------------------------------------------------------------------------
void orc_attention(const float* Q, const float* K, const float* V, const float* mask, float scale,
                   int S, int T, int Hq, int Hkv, int D, float* out, int acc64) {
    const int g = Hq / Hkv;
#pragma omp parallel for schedule(static)
    for (int h = 0; h < Hq; ++h) {
        const int hk = h / g;
        std::vector<float> sc(T);
        for (int s = 0; s < S; ++s) {
            const float* q = Q + ((size_t)s * Hq + h) * D;
            for (int t = 0; t < T; ++t) {
                const float* k = K + ((size_t)t * Hkv + hk) * D;
                if (acc64) {
                    double a = 0.0;
                    for (int d = 0; d < D; ++d) a += (double)q[d] * (double)k[d];
                    sc[t] = (float)a;
                } else {
                    sc[t] = dot_f32_lanes(q, k, D);
                }
            }
            orc_softmax_ext(sc.data(), mask ? mask + (size_t)s * T : nullptr, scale, 1, T);
            float* o = out + ((size_t)s * Hq + h) * D;
            if (acc64) {
                for (int d = 0; d < D; ++d) {
                    double a = 0.0;
                    for (int t = 0; t < T; ++t) a += (double)sc[t] * (double)V[((size_t)t * Hkv + hk) * D + d];
                    o[d] = (float)a;
                }
            } else {  // keys outermost: every V row is read once, contiguously
                for (int d = 0; d < D; ++d) o[d] = 0.f;
                for (int t = 0; t < T; ++t) {
                    const float* v = V + ((size_t)t * Hkv + hk) * D;
                    const float p = sc[t];
                    for (int d = 0; d < D; ++d) o[d] = __builtin_fmaf(p, v[d], o[d]);
                }
            }
        }
    }
}

// ----------------------------------------------------------------------------
// Masks and positions built on the host by the reference.
// ----------------------------------------------------------------------------
static const float NEG_INF = -std::numeric_limits<float>::infinity();

// SmolVLA mask_full [S][P+S] (src/models/smolvla.cpp:1651-1664): prefix columns
// blocked inside the padded-language range, suffix block causal.
void orc_mask_smolvla_full(int P, int S, int pad_start, int pad_end, float* mask) {
    const int T = P + S;
    for (int i = 0; i < S; ++i)
        for (int j = 0; j < T; ++j) {
            bool blocked;
            if (j < P) blocked = (j >= pad_start && j < pad_end);
            else blocked = ((j - P) > i);
            mask[(size_t)i * T + j] = blocked ? NEG_INF : 0.f;
        }
}
// SmolVLA mask_prefix_only [S][P] (smolvla.cpp:1665-1669).
void orc_mask_smolvla_prefix_only(int P, int S, int pad_start, int pad_end, float* mask) {
    for (int i = 0; i < S; ++i)
        for (int j = 0; j < P; ++j)
            mask[(size_t)i * P + j] = (j >= pad_start && j < pad_end) ? NEG_INF : 0.f;
}
// SmolVLA prefill mask [P][P] and positions (smolvla.cpp:1633-1649): only the
// state token (last) sees the state token; padded language blocked; the state
// token's position is right after the real text.
void orc_mask_smolvla_prefill(int P, int pad_start, int pad_end, int state_pos, float* mask, int32_t* pos) {
    for (int i = 0; i < P; ++i) {
        for (int j = 0; j < P; ++j) {
            bool blocked = false;
            if (i < P - 1 && j == P - 1) blocked = true;
            if (j >= pad_start && j < pad_end) blocked = true;
            mask[(size_t)i * P + j] = blocked ? NEG_INF : 0.f;
        }
        pos[i] = (i == P - 1) ? state_pos : i;
    }
}
// pi0 full mask [S][P+S] (src/models/pi0.cpp:638-653): prefix open; row 0 (the
// state token) sees suffix column 0 only; other rows see the whole suffix.
void orc_mask_pi0_full(int P, int S, float* mask) {
    const int T = P + S;
    for (int i = 0; i < S; ++i)
        for (int j = 0; j < T; ++j) {
            bool allowed;
            if (j < P) allowed = true;
            else {
                const int s = j - P;
                allowed = (i == 0) ? (s == 0) : true;
            }
            mask[(size_t)i * T + j] = allowed ? 0.f : NEG_INF;
        }
}
// src/layers/embed.h:75-81.
void orc_mask_causal(int seq, float* mask) {
    for (int q = 0; q < seq; ++q)
        for (int kv = 0; kv < seq; ++kv) mask[(size_t)q * seq + kv] = kv > q ? NEG_INF : 0.f;
}

// ----------------------------------------------------------------------------
// Time embeddings (src/layers/embed.h:32-73; pinned by
// tests/test_dit_common.cpp).
// ----------------------------------------------------------------------------
void orc_timesteps_proj(int64_t bucket, float* out256) {  // cos first, then sin
    const int half = 128;
    const float lm = std::log(10000.0f);
    const float t = (float)bucket;
    for (int i = 0; i < half; ++i) {
        const float emb = t * std::exp(-lm * (float)i / (float)(half - 1));
        out256[i] = std::cos(emb);
        out256[half + i] = std::sin(emb);
    }
}
void orc_action_sinusoid(int64_t bucket, int64_t dim, int64_t T, float* out) {  // sin first
    const int64_t half = dim / 2;
    const float step = std::log(10000.0f) / (float)half;
    const float t = (float)bucket;
    for (int64_t tk = 0; tk < T; ++tk)
        for (int64_t i = 0; i < half; ++i) {
            const float emb = t * std::exp(-(float)i * step);
            out[tk * dim + i] = std::sin(emb);
            out[tk * dim + half + i] = std::cos(emb);
        }
}
void orc_sinusoidal_time_emb(double t, int64_t dim, double min_p, double max_p, float* out) {
    const int64_t half = dim / 2;
    for (int64_t i = 0; i < half; ++i) {
        const double frac = (half == 1) ? 0.0 : double(i) / double(half - 1);
        const double period = min_p * std::pow(max_p / min_p, frac);
        const double s = (2.0 * M_PI / period) * t;
        out[i] = (float)std::sin(s);
        out[half + i] = (float)std::cos(s);
    }
}

// ----------------------------------------------------------------------------
// BitVLA ternary path.
// ----------------------------------------------------------------------------

// recover_ternary_and_scale (src/models/bitvla.cpp:430-451) ==
// weight_quant_to_ternary (scripts/convert_bitvla_to_gguf.py:95-101).
void orc_weight_quant_ternary(const float* W, int64_t n, int8_t* ternary, float* absmean) {
    double s = 0.0;
    for (int64_t i = 0; i < n; ++i) s += std::fabs((double)W[i]);
    float mean = n > 0 ? (float)(s / (double)n) : 0.0f;
    if (mean < 1e-5f) mean = 1e-5f;
    *absmean = mean;
    const float inv = 1.0f / mean;
    for (int64_t i = 0; i < n; ++i) {
        float q = std::nearbyintf(W[i] * inv);
        if (q > 1.0f) q = 1.0f;
        if (q < -1.0f) q = -1.0f;
        ternary[i] = (int8_t)q;
    }
}

// pack_ladder_int2 (src/models/bitvla.cpp:453-483): 4 codes per byte,
// code = t + 2, byte b of a 16-value slot holds values b + 4j at bits 2j.
void orc_pack_ladder_int2(const int8_t* W, int64_t N, int64_t K, uint8_t* out) {
    const int64_t n_slots = N * K / 16;
    const int64_t slots_per_block = (16 * K) / 16;
    for (int64_t s = 0; s < n_slots; ++s) {
        const int64_t n_block = s / slots_per_block, in_block = s % slots_per_block;
        const int64_t k_0 = in_block / 128, in_k0 = in_block % 128;
        const int64_t major_k = in_k0 / 32, in_major = in_k0 % 32;
        const int64_t y_half = in_major / 16, in_yhalf = in_major % 16;
        const int64_t sub_k = in_yhalf / 8, y_in_h = in_yhalf % 8;
        const int64_t n_global = n_block * 16 + y_half * 8 + y_in_h;
        const int64_t k_sub = k_0 * 128 + major_k * 32 + sub_k * 16;
        for (int byte_i = 0; byte_i < 4; ++byte_i) {
            uint8_t b = 0;
            for (int j = 0; j < 4; ++j) {
                const int t = (int)W[n_global * K + (k_sub + byte_i + 4 * j)];
                b |= (uint8_t)(((uint8_t)(t + 2) & 0x3) << (2 * j));
            }
            out[s * 4 + byte_i] = b;
        }
    }
}

// decode_i2s_to_i8s (src/kernels/bitvla/bitnet_kernels.h:71-90): output word i
// is ((i2s >> 2i) & 0x03030303) with 2 subtracted from every byte (saturating,
// never reached), so byte b of word i is value b + 4i... laid out as 16
// consecutive int8.
void orc_decode_i2s_to_i8s(uint32_t i2s, int8_t* out16) {
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = (i2s >> (2 * i)) & 0x03030303u;
        for (int b = 0; b < 4; ++b) out16[4 * i + b] = (int8_t)((int)((w >> (8 * b)) & 0xff) - 2);
    }
}

// Unpack by walking the GEMV kernel's own addressing
// (ladder_int8xint2_kernel, bitnet_kernels.h:108-145): thread (tx 0..7,
// ty 0..15) of block bx at iteration k_0 reads one 32-bit word and multiplies
// its 16 decoded values with A[k_0*128 + tx*16 .. +16) for output column
// bx*16 + ty.  Independent of orc_pack_ladder_int2, so pack -> unpack == id
// pins both.
void orc_unpack_ladder_int2(const uint8_t* B, int64_t N, int64_t K, int8_t* W) {
    for (int64_t bx = 0; bx < N / 16; ++bx)
        for (int64_t k_0 = 0; k_0 < K / 128; ++k_0)
            for (int ty = 0; ty < 16; ++ty)
                for (int tx = 0; tx < 8; ++tx) {
                    const int64_t off = bx * 16 * K / 4 + k_0 * 8 * 16 * 16 / 4 + (tx >> 1) * 32 * 16 / 4 +
                                        (ty >> 3) * (32 * 16 / 2) / 4 + (tx & 1) * (32 * 16 / 4) / 4 +
                                        (ty & 7) * (32 / 2) / 4;
                    uint32_t word;
                    std::memcpy(&word, B + off, 4);
                    int8_t v[16];
                    orc_decode_i2s_to_i8s(word, v);
                    const int64_t n = bx * 16 + ty, k = k_0 * 128 + tx * 16;
                    for (int i = 0; i < 16; ++i) W[n * K + k + i] = v[i];
                }
}

// act_quant_kernel (bitnet_kernels.h:465-521): per row amax = max(max|x|, 1e-5),
// scale = 127/amax, q = clamp(nearbyint(x*scale), -128, 127); scales[m] = scale.
// Input is whatever the caller holds in fp32 (bf16 values widened exactly for
// the CUDA twin, fp32 for the CPU twin src/models/bitvla.cpp:69-96).
void orc_act_quant(const float* x, int M, int K, int8_t* q, float* scales) {
    for (int m = 0; m < M; ++m) {
        const float* row = x + (size_t)m * K;
        float amax = 0.f;
        for (int k = 0; k < K; ++k) amax = std::max(amax, std::fabs(row[k]));
        if (amax < 1e-5f) amax = 1e-5f;
        const float s = 127.0f / amax;
        scales[m] = s;
        for (int k = 0; k < K; ++k) {
            float v = std::nearbyintf(row[k] * s);
            if (v > 127.0f) v = 127.0f;
            if (v < -128.0f) v = -128.0f;
            q[(size_t)m * K + k] = (int8_t)v;
        }
    }
}
// The CPU twin's fake-quant output q * (1/s) (src/models/bitvla.cpp:69-96).
void orc_act_fake_quant(const float* x, int M, int K, float* out) {
    for (int m = 0; m < M; ++m) {
        const float* row = x + (size_t)m * K;
        float amax = 0.f;
        for (int k = 0; k < K; ++k) amax = std::max(amax, std::fabs(row[k]));
        if (amax < 1e-5f) amax = 1e-5f;
        const float s = 127.0f / amax, inv_s = 1.0f / s;
        for (int k = 0; k < K; ++k) {
            float v = std::nearbyintf(row[k] * s);
            if (v > 127.0f) v = 127.0f;
            if (v < -128.0f) v = -128.0f;
            out[(size_t)m * K + k] = v * inv_s;
        }
    }
}

// acc[m][n] = sum_k A[m][k] * Wt[n][k], exact in int32 (bitnet_kernels.h:165-247;
// K <= 2^17 keeps |acc| < 2^31 for |A| <= 128, |Wt| <= 2).
void orc_ternary_gemm_i32(const int8_t* A, const int8_t* Wt, int M, int N, int K, int32_t* acc) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            int32_t a = 0;
            const int8_t* ar = A + (size_t)m * K;
            const int8_t* wr = Wt + (size_t)n * K;
            for (int k = 0; k < K; ++k) a += (int32_t)ar[k] * (int32_t)wr[k];
            acc[(size_t)m * N + n] = a;
        }
}

// Epilogue out = bf16(float(acc) / s[m] * ws[n / (N/ws_num)])
// (bitnet_kernels.h:239-245, 400-406).  IEEE division; the reference's CUDA
// build passes --use_fast_math (CMakeLists.txt:135), so its own division is
// approximate and this is the exact form of it.
void orc_ternary_epilogue(const int32_t* acc, const float* s, const float* ws, int M, int N, int ws_num,
                          uint16_t* out) {
    const int group = N / ws_num;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
            out[(size_t)m * N + n] = orc_f32_to_bf16((float)acc[(size_t)m * N + n] / s[m] * ws[n / group]);
}

// bitlinear on the CPU path: ggml_mul_mat(W_dequant, act_quant(x))
// (src/models/bitvla.cpp:173-176): y[m][n] = sum_k (t[n][k]*absmean) * (q/s).
void orc_bit_linear_f32(const float* x, const int8_t* Wt, float absmean, float* y, int M, int N, int K) {
    std::vector<float> fq((size_t)M * K);
    orc_act_fake_quant(x, M, K, fq.data());
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double a = 0.0;
            for (int k = 0; k < K; ++k) a += (double)((float)Wt[(size_t)n * K + k] * absmean) * (double)fq[(size_t)m * K + k];
            y[(size_t)m * N + n] = (float)a;
        }
}

// Layout helpers of the BitVLA CUDA forward (bitvla_lm_cuda.cu:181-224).
void orc_repeat_kv_u16(const uint16_t* in, uint16_t* out, int n_q, int n_kv, int seq, int hd) {
    for (int qh = 0; qh < n_q; ++qh) {
        const int kvh = qh * n_kv / n_q;
        std::memcpy(out + (size_t)qh * seq * hd, in + (size_t)kvh * seq * hd, (size_t)seq * hd * 2);
    }
}
void orc_transpose_sHd_to_Hsd_u16(const uint16_t* in, uint16_t* out, int S, int H, int hd) {
    for (int s = 0; s < S; ++s)
        for (int h = 0; h < H; ++h)
            std::memcpy(out + ((size_t)h * S + s) * hd, in + ((size_t)s * H + h) * hd, (size_t)hd * 2);
}
void orc_transpose_Hsd_to_sHd_u16(const uint16_t* in, uint16_t* out, int H, int S, int hd) {
    for (int s = 0; s < S; ++s)
        for (int h = 0; h < H; ++h)
            std::memcpy(out + ((size_t)s * H + h) * hd, in + ((size_t)h * S + s) * hd, (size_t)hd * 2);
}
void orc_gather_rows_u16(const uint16_t* in, uint16_t* out, const int32_t* ids, int n_rows, int K) {
    for (int m = 0; m < n_rows; ++m) std::memcpy(out + (size_t)m * K, in + (size_t)ids[m] * K, (size_t)K * 2);
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

}  // extern "C"
