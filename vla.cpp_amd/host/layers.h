// Host-side op fragments with the names and argument order of the reference's
// src/layers (attn.h:27-58, rope.h:28-48, linear.h:24-27, norm.h:27-46,
// embed.h:61-73).  The reference's versions record ggml graph nodes on
// ggml_tensor*; these run eagerly on a HIP stream over a light tensor view and
// the resident KV cache, by calling the kernel C ABI (include/vla_kernels.h)
// and nothing else.
#pragma once

#include <cmath>
#include <cstdint>
#include <vector>

#include "device.h"
#include "vla_kernels.h"

namespace vla {

// ne[0] is the innermost dimension, as in ggml.
struct Tensor {
    void* data = nullptr;
    int dtype = VLA_DT_F32;
    int64_t ne[4] = {1, 1, 1, 1};
    int64_t rows() const { return ne[1] * ne[2] * ne[3]; }
};

inline Tensor tensor_2d(void* data, int dtype, int64_t ne0, int64_t ne1) {
    Tensor t;
    t.data = data;
    t.dtype = dtype;
    t.ne[0] = ne0;
    t.ne[1] = ne1;
    return t;
}

// Execution context in place of ggml_context: the stream every op is queued on.
struct Ctx {
    hipStream_t stream = nullptr;
};

// rope.h:28-38 without the fields this path never varies (NeoX only, freq_scale
// 1, no YaRN).  The angle tables are built once per observation on the host.
struct RopeSpec {
    int n_dims = 0;
    float freq_base = 10000.0f;
};

struct RopeTable {
    DevBuf cos, sin;
    int rows = 0;
    void build(const RopeSpec& r, const std::vector<int32_t>& pos) {
        rows = (int)pos.size();
        const size_t n = pos.size() * (size_t)(r.n_dims / 2);
        std::vector<float> c(n), s(n);
        VLA_K(vla_rope_tables_host(pos.data(), rows, r.n_dims, (double)r.freq_base, c.data(), s.data()));
        cos.upload(c.data(), n * sizeof(float));
        sin.upload(s.data(), n * sizeof(float));
    }
};

// One layer's resident cache: K [B][Hkv][t_max][D], V^T [B][Hkv][D][t_max].
struct KVLayer {
    DevBuf k, vt;
    int dtype = VLA_DT_F32, batch = 0, n_kv_heads = 0, head_dim = 0, t_max = 0;
    int n_prefix = 0;  // tokens [0, n_prefix) are the observation's prefix
    void create(int dt, int B, int Hkv, int D, int tmax) {
        dtype = dt; batch = B; n_kv_heads = Hkv; head_dim = D; t_max = tmax;
        const size_t bytes = (size_t)B * Hkv * D * tmax * dtype_size(dt);
        k.alloc(bytes);
        vt.alloc(bytes);
        k.zero();
        vt.zero();
    }
};

// Scratch memory of a handle's attention launches (key-slice partials and arrival counters):
// owned by the handle, so that handles never share any -- the reference's contract is one
// call at a time per handle (include/vla.h:18-19), not per process.  plan() every shape the
// handle will launch, then commit() (allocates and zero-fills; invalidates captured graphs
// that hold the old block, so the owner bumps its launch key).
struct AttnWorkspace {
    DevBuf buf;
    size_t need = 0;
    void reset() { need = 0; }
    void plan(int dtype, int batch, int S, int Hq, int Hkv, int D, int n_keys) {
        const size_t b = vla_attn_workspace_bytes(dtype, batch, S, Hq, Hkv, D, n_keys);
        if (b == VLA_ATTN_WORKSPACE_UNSUPPORTED) throw std::invalid_argument("vla: no attention kernel takes this head geometry");
        if (b > need) need = b;
    }
    void commit() {
        buf.alloc(need);
        buf.zero();
    }
    // The part launches count in, back at zero: once per launch sequence, so that a sequence cut
    // short by a device fault cannot poison the next one.
    void begin(hipStream_t stream) {
        if (buf.bytes()) VLA_K(vla_attn_workspace_reset(buf.get(), buf.bytes(), stream));
    }
};

// Mask as the attention kernel generates it (masks are data in the reference:
// src/models/smolvla.cpp:1651-1669, src/models/pi0.cpp:638-653).
struct MaskSpec {
    int kind = VLA_MASK_NONE;
    int pad_start = 0, pad_end = 0;
};

// linear.h:24-27: y = W x + b, optionally fused with the residual add that
// follows it in every layer (h1 = x_in + Wo att).
inline void linear(Ctx& C, const Tensor& W, const float* b, const Tensor& x, const void* residual, Tensor& y) {
    VLA_K(vla_linear(x.data, W.data, b, residual, y.data, x.dtype, y.dtype, (int)x.rows(), (int)W.ne[1], (int)W.ne[0],
                     C.stream));
}

// The same projection (bf16 rows, bf16 output) that also leaves (sum of squares, sum) of what it wrote per
// (row, 64-column tile) in row_stats [rows][W rows / 64][2], for the launch that takes the next LayerNorm inside.
inline void linear_row_stats(Ctx& C, const Tensor& W, const float* b, const Tensor& x, const void* residual, Tensor& y,
                             float* row_stats) {
    VLA_K(vla_linear_row_stats(x.data, W.data, b, residual, y.data, row_stats, x.dtype, (int)x.rows(), (int)W.ne[1], (int)W.ne[0],
                               C.stream));
}

// ffn.h:24-27 (ffn_gelu) with the residual add that follows it in DitHead::block
// (src/modules/dit_head.cpp:133): y = residual + W2 gelu(W1 x + b1) + b2.  `mid` is scratch
// for the activated intermediate [rows][W1 rows].
inline void ffn_gelu(Ctx& C, const Tensor& W1, const float* b1, const Tensor& W2, const float* b2, const Tensor& x,
                     const void* residual, Tensor& mid, Tensor& y) {
    VLA_K(vla_linear_act(x.data, W1.data, b1, nullptr, mid.data, x.dtype, mid.dtype, (int)x.rows(), (int)W1.ne[1],
                         (int)W1.ne[0], VLA_ACT_GELU, C.stream));
    VLA_K(vla_linear(mid.data, W2.data, b2, residual, y.data, mid.dtype, y.dtype, (int)mid.rows(), (int)W2.ne[1],
                     (int)W2.ne[0], C.stream));
}

// ffn.h:35-40 (ffn_swiglu) generalised over the gate activation (ggml_silu in the SmolVLA
// expert, ggml_gelu in the Gemma expert), without biases, with the residual add that follows:
// y = residual + Wd (act(Wg x) * (Wu x)).  Wgu holds the gate rows, then the up rows.  With
// rms_eps >= 0, x is the un-normalised stream and Wgu carries the post-attention norm
// weight (vla_fold_norm_weight_host); returns false, launching nothing, when the shapes do
// not fit that fused launch.
inline bool ffn_glu(Ctx& C, const Tensor& Wgu, int act, const Tensor& Wd, const Tensor& x, float rms_eps,
                    const void* residual, Tensor& mid, Tensor& y) {
    const int rc = vla_glu_linear(x.data, Wgu.data, nullptr, mid.data, x.dtype, mid.dtype, (int)x.rows(),
                                  (int)(Wgu.ne[1] / 2), (int)Wgu.ne[0], act, rms_eps, C.stream);
    if (rc == VLA_K_ERR_SHAPE && rms_eps >= 0.f) return false;
    VLA_K(rc);
    VLA_K(vla_linear(mid.data, Wd.data, nullptr, residual, y.data, mid.dtype, y.dtype, (int)mid.rows(), (int)Wd.ne[1],
                     (int)Wd.ne[0], C.stream));
    return true;
}

// norm.h:31-34.
inline void rms_norm(Ctx& C, const Tensor& x, const void* w, float eps, Tensor& y) {
    VLA_K(vla_rms_norm(x.data, w, y.data, x.dtype, (int)x.rows(), (int)x.ne[0], eps, C.stream));
}

// norm.h:37-46 with the (scale, shift) pair already evaluated for this step.
inline void adaln(Ctx& C, const Tensor& x, const float* sc, const float* sh, float eps, Tensor& y) {
    VLA_K(vla_adaln(x.data, sc, sh, y.data, x.dtype, (int)x.rows(), (int)x.ne[0], eps, C.stream));
}

// rope.h:40-48 on a token-major tensor [D, H, rows].
inline void rope(Ctx& C, const RopeTable& tab, Tensor& x) {
    VLA_K(vla_rope_neox(x.data, tab.cos.as<float>(), tab.sin.as<float>(), x.dtype, (int)(x.ne[2] * x.ne[3]), tab.rows,
                        (int)x.ne[1], (int)x.ne[0], C.stream));
}

// The QKV projections, head split, rotation and ggml_concat of a layer
// (src/models/smolvla.cpp:821-833) as one launch.  `S` rows per observation land
// at tokens [kv.n_prefix, kv.n_prefix + S) of the cache unless tok_offset >= 0.
inline void qkv_rope_append(Ctx& C, const Tensor& x, const Tensor& W, const float* bias, int S, int n_q_heads,
                            bool has_k, bool has_v, const RopeTable* tab, void* q_out, KVLayer& kv, int tok_offset) {
    VLA_K(vla_attn_qkv_rope(x.data, W.data, bias, x.dtype, (int)x.rows(), (int)x.ne[0], S, n_q_heads, kv.n_kv_heads,
                            has_k ? 1 : 0, has_v ? 1 : 0, kv.head_dim, tab ? tab->cos.as<float>() : nullptr,
                            tab ? tab->sin.as<float>() : nullptr, q_out, kv.k.get(), kv.vt.get(), kv.t_max, tok_offset,
                            C.stream));
}

// The pre-norm of the layer (norm.h:31-34) and the launch above as one: x is the
// un-normalised stream and W carries the norm weight (vla_fold_norm_weight_host).
// Returns false when the shapes do not fit the fused kernel; nothing was launched then.
inline bool rmsnorm_qkv_rope_append(Ctx& C, const Tensor& x, const Tensor& W_folded, const float* bias, float eps, int S,
                                    int n_q_heads, bool has_k, bool has_v, const RopeTable* tab, void* q_out, KVLayer& kv,
                                    int tok_offset) {
    const int rc = vla_rmsnorm_attn_qkv_rope(x.data, W_folded.data, bias, x.dtype, (int)x.rows(), (int)x.ne[0], S, n_q_heads,
                                             kv.n_kv_heads, has_k ? 1 : 0, has_v ? 1 : 0, kv.head_dim,
                                             tab ? tab->cos.as<float>() : nullptr, tab ? tab->sin.as<float>() : nullptr,
                                             q_out, kv.k.get(), kv.vt.get(), kv.t_max, tok_offset, eps, C.stream);
    if (rc == VLA_K_ERR_SHAPE) return false;
    VLA_K(rc);
    return true;
}

// A DiT block's modulated LayerNorm (norm.h:37-46) and the projection launch as one: x is
// the un-normalised stream; W_folded, colsum and bias carry this step's (scale, shift)
// (vla_fold_adaln_weight_host).  Returns false when the shapes do not fit the fused kernel.
// row_stats: the rows' sums as the launch that wrote x left them (linear_row_stats), or null.
inline bool layernorm_qkv_rope_append(Ctx& C, const Tensor& x, const Tensor& W_folded, const float* colsum, const float* bias,
                                      float eps, int S, int n_q_heads, bool has_k, bool has_v, const RopeTable* tab, void* q_out,
                                      KVLayer& kv, int tok_offset, const float* row_stats = nullptr) {
    const float* ct = tab ? tab->cos.as<float>() : nullptr;
    const float* st = tab ? tab->sin.as<float>() : nullptr;
    const int rc = row_stats
        ? vla_layernorm_attn_qkv_rope_stats(x.data, W_folded.data, colsum, bias, row_stats, (int)x.ne[0] / 64, x.dtype, (int)x.rows(),
                                            (int)x.ne[0], S, n_q_heads, kv.n_kv_heads, has_k ? 1 : 0, has_v ? 1 : 0, kv.head_dim, ct, st,
                                            q_out, kv.k.get(), kv.vt.get(), kv.t_max, tok_offset, eps, C.stream)
        : vla_layernorm_attn_qkv_rope(x.data, W_folded.data, colsum, bias, x.dtype, (int)x.rows(), (int)x.ne[0], S, n_q_heads,
                                      kv.n_kv_heads, has_k ? 1 : 0, has_v ? 1 : 0, kv.head_dim, ct, st, q_out, kv.k.get(),
                                      kv.vt.get(), kv.t_max, tok_offset, eps, C.stream);
    if (rc == VLA_K_ERR_SHAPE) return false;
    VLA_K(rc);
    return true;
}

// A DiT self block's adaLN, Q / K / V projections and the attention of each observation's S
// tokens over themselves as one launch (dit_head.cpp:111-125 with enc = nullptr); the block's K
// and V stay on the chip.  Returns false when the shapes do not fit the fused kernel.
inline bool layernorm_qkv_self_attention(Ctx& C, const Tensor& x, const Tensor& W_folded, const float* colsum, const float* bias,
                                         float eps, int S, int n_heads, int head_dim, float scale, Tensor& out,
                                         const float* row_stats = nullptr) {
    const int rc = row_stats
        ? vla_layernorm_qkv_self_attention_stats(x.data, W_folded.data, colsum, bias, row_stats, (int)x.ne[0] / 64, x.dtype,
                                                 (int)x.rows(), (int)x.ne[0], S, n_heads, head_dim, scale, eps, out.data, C.stream)
        : vla_layernorm_qkv_self_attention(x.data, W_folded.data, colsum, bias, x.dtype, (int)x.rows(), (int)x.ne[0], S, n_heads,
                                           head_dim, scale, eps, out.data, C.stream);
    if (rc == VLA_K_ERR_SHAPE) return false;
    VLA_K(rc);
    return true;
}

// attn.h:48-58 (flash_attention) over the resident cache: Q [D, Hq, S, B]
// token-major, keys [0, n_keys).
inline void flash_attention(Ctx& C, const Tensor& Q, const KVLayer& kv, int n_keys, const MaskSpec& mask, float scale,
                            Tensor& out, const AttnWorkspace& ws) {
    VLA_K(vla_attn_prefix_suffix_ws(Q.data, kv.k.get(), kv.vt.get(), out.data, Q.dtype, (int)Q.ne[3], (int)Q.ne[2],
                                    (int)Q.ne[1], kv.n_kv_heads, (int)Q.ne[0], kv.t_max, n_keys, scale, mask.kind,
                                    kv.n_prefix, mask.pad_start, mask.pad_end, nullptr, ws.buf.get(), ws.buf.bytes(),
                                    C.stream));
}

// embed.h:61-73, log-spaced periods, sin first.
inline std::vector<float> sinusoidal_time_emb(double t, int64_t dim, double min_p, double max_p) {
    const int64_t half = dim / 2;
    std::vector<float> out((size_t)dim);
    for (int64_t i = 0; i < half; ++i) {
        const double frac = (half == 1) ? 0.0 : double(i) / double(half - 1);
        const double period = min_p * std::pow(max_p / min_p, frac);
        const double s = (2.0 * 3.14159265358979323846 / period) * t;
        out[i] = (float)std::sin(s);
        out[half + i] = (float)std::cos(s);
    }
    return out;
}

// embed.h:32-44, cos first.
inline void timesteps_proj(int64_t bucket, std::vector<float>& out) {
    const int64_t half = 128;
    const float lm = std::log(10000.0f);
    const float t = (float)bucket;
    out.assign(256, 0.0f);
    for (int64_t i = 0; i < half; ++i) {
        const float emb = t * std::exp(-lm * (float)i / (float)(half - 1));
        out[i] = std::cos(emb);
        out[half + i] = std::sin(emb);
    }
}

}  // namespace vla
