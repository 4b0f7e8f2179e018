// The context form of the BitVLA language model: bitvla_lm_cuda_{init, set_layer,
// set_output_norm, forward, free} of src/kernels/bitvla/bitvla_lm_cuda.h:247-286 and the
// layer sequence of run_layer (src/kernels/bitvla/bitvla_lm_cuda.cu:395-522), on this
// library's kernels.  The caller owns every weight pointer; the context owns the workspace.
//
// Per layer: RMSNorm + int8 quantisation (one launch) -> Q, K, V ternary GEMMs -> NeoX RoPE on
// Q and K (token-major, positions 0..seq-1) -> K / V into a [Hkv][seq][D] / [Hkv][D][seq]
// workspace -> attention over all seq keys -> sub-norm + quantisation -> O GEMM + residual ->
// FFN norm + quantisation -> fused gate|up GEMM -> relu(gate)^2 * up -> FFN sub-norm +
// quantisation -> down GEMM + residual.  Then the output RMSNorm into d_out.

#include <cmath>
#include <cstdio>
#include <exception>
#include <new>
#include <vector>

#include "device.h"
#include "vla_kernels.h"

struct bitvla_lm_hip_ctx {
    int hidden = 0, n_q = 0, n_kv = 0, hd = 0, ffn = 0, n_layers = 0, max_seq = 0, t_max = 0;
    float rms_eps = 0.f;
    std::vector<bitvla_lm_layer_hip> layers;
    std::vector<char> bound;
    const uint16_t* out_norm = nullptr;
    vla::DevBuf cos, sin, h, q8, s, rowsum, q, k, v, kc, vtc, att, gate_up, act, attn_ws;
};

namespace {

// fprintf + -1 instead of an exception: nothing may unwind through the C boundary
int run(bitvla_lm_hip_ctx* c, const uint16_t* d_in, uint16_t* d_out, int seq, hipStream_t st) {
    const int H = c->hidden, hq = c->n_q * c->hd, hkv = c->n_kv * c->hd, F = c->ffn;
    uint16_t* h = c->h.as<uint16_t>();
    int8_t* q8 = c->q8.as<int8_t>();
    float* s = c->s.as<float>();
    int32_t* rs = c->rowsum.as<int32_t>();
    const float scale = 1.0f / std::sqrt((float)c->hd);
    VLA_HIP(hipMemcpyAsync(h, d_in, (size_t)seq * H * 2, hipMemcpyDeviceToDevice, st));
    for (int L = 0; L < c->n_layers; ++L) {
        const bitvla_lm_layer_hip& w = c->layers[L];
        VLA_K(vla_rmsnorm_act_quant_bf16(h, w.attn_norm_w, q8, s, rs, c->rms_eps, seq, H, st));
        VLA_K(vla_ternary_gemm(q8, (const uint32_t*)w.q_packed, c->q.as<uint16_t>(), nullptr, s, rs, w.q_ws, 1, seq, hq, H, st));
        VLA_K(vla_ternary_gemm(q8, (const uint32_t*)w.k_packed, c->k.as<uint16_t>(), nullptr, s, rs, w.k_ws, 1, seq, hkv, H, st));
        VLA_K(vla_ternary_gemm(q8, (const uint32_t*)w.v_packed, c->v.as<uint16_t>(), nullptr, s, rs, w.v_ws, 1, seq, hkv, H, st));
        VLA_K(vla_rope_neox(c->q.get(), c->cos.as<float>(), c->sin.as<float>(), VLA_DT_BF16, seq, seq, c->n_q, c->hd, st));
        VLA_K(vla_rope_neox(c->k.get(), c->cos.as<float>(), c->sin.as<float>(), VLA_DT_BF16, seq, seq, c->n_kv, c->hd, st));
        VLA_K(vla_kv_append(c->kc.get(), c->vtc.get(), c->k.get(), c->v.get(), VLA_DT_BF16, 1, c->n_kv, c->hd, c->t_max, 0, seq, st));
        VLA_K(vla_attn_prefix_suffix_ws(c->q.get(), c->kc.get(), c->vtc.get(), c->att.get(), VLA_DT_BF16_P2, 1, seq, c->n_q, c->n_kv,
                                        c->hd, c->t_max, seq, scale, VLA_MASK_NONE, seq, 0, 0, nullptr, c->attn_ws.get(),
                                        c->attn_ws.bytes(), st));
        VLA_K(vla_rmsnorm_act_quant_bf16(c->att.as<uint16_t>(), w.attn_sub_norm_w, q8, s, rs, c->rms_eps, seq, hq, st));
        VLA_K(vla_ternary_gemm_add(q8, (const uint32_t*)w.o_packed, h, h, s, rs, w.o_ws, 1, seq, H, hq, st));
        VLA_K(vla_rmsnorm_act_quant_bf16(h, w.ffn_norm_w, q8, s, rs, c->rms_eps, seq, H, st));
        VLA_K(vla_ternary_gemm(q8, (const uint32_t*)w.gate_up_packed, c->gate_up.as<uint16_t>(), nullptr, s, rs, w.gate_up_ws, 2, seq,
                               2 * F, H, st));
        // activation, sub-norm and quantisation in one launch (same bits as the two below it)
        const int rc = vla_sqrelu_rmsnorm_act_quant_bf16(c->gate_up.as<uint16_t>(), w.ffn_sub_norm_w, q8, s, rs, c->rms_eps, seq, F, st);
        if (rc != VLA_K_ERR_SHAPE) VLA_K(rc);
        else {
            VLA_K(gate_up_fused_sqrelu_mul_bf16(c->gate_up.as<uint16_t>(), c->act.as<uint16_t>(), seq, F, st));
            VLA_K(vla_rmsnorm_act_quant_bf16(c->act.as<uint16_t>(), w.ffn_sub_norm_w, q8, s, rs, c->rms_eps, seq, F, st));
        }
        VLA_K(vla_ternary_gemm_add(q8, (const uint32_t*)w.down_packed, h, h, s, rs, w.down_ws, 1, seq, H, F, st));
    }
    VLA_K(bitvla_rmsnorm_bf16(h, c->out_norm, d_out, c->rms_eps, seq, H, st));
    return 0;
}

}  // namespace

extern "C" {

bitvla_lm_hip_ctx* bitvla_lm_hip_init(int hidden, int n_q, int n_kv, int head_dim, int ffn, int n_layers, float rope_base,
                                      float rms_eps, int max_seq) {
    if (hidden <= 0 || n_q <= 0 || n_kv <= 0 || head_dim <= 0 || (head_dim & 1) || ffn <= 0 || n_layers <= 0 || max_seq <= 0 ||
        n_q % n_kv || hidden % 128 || (n_q * head_dim) % 128 || ffn % 128) {
        std::fprintf(stderr, "vla(bitvla_lm_hip): unsupported geometry (K of every ternary GEMM must be a multiple of 128)\n");
        return nullptr;
    }
    bitvla_lm_hip_ctx* c = new (std::nothrow) bitvla_lm_hip_ctx();
    if (!c) return nullptr;
    try {
        c->hidden = hidden; c->n_q = n_q; c->n_kv = n_kv; c->hd = head_dim; c->ffn = ffn; c->n_layers = n_layers;
        c->rms_eps = rms_eps; c->max_seq = max_seq; c->t_max = (max_seq + 63) / 64 * 64;
        c->layers.resize((size_t)n_layers);
        c->bound.assign((size_t)n_layers, 0);
        const int half = head_dim / 2, hq = n_q * head_dim, hkv = n_kv * head_dim;
        std::vector<int32_t> pos((size_t)max_seq);
        for (int i = 0; i < max_seq; ++i) pos[i] = i;
        std::vector<float> cs((size_t)max_seq * half), sn((size_t)max_seq * half);
        VLA_K(vla_rope_tables_host(pos.data(), max_seq, head_dim, (double)rope_base, cs.data(), sn.data()));
        c->cos.upload(cs.data(), cs.size() * 4);
        c->sin.upload(sn.data(), sn.size() * 4);
        const size_t S = (size_t)max_seq, widest = (size_t)(hidden > ffn ? (hidden > hq ? hidden : hq) : (ffn > hq ? ffn : hq));
        c->h.alloc(S * hidden * 2);
        c->q8.alloc(S * widest);
        c->s.alloc(S * 4);
        c->rowsum.alloc(S * 4);
        c->q.alloc(S * hq * 2);
        c->k.alloc(S * hkv * 2);
        c->v.alloc(S * hkv * 2);
        c->kc.alloc((size_t)c->t_max * hkv * 2);
        c->vtc.alloc((size_t)c->t_max * hkv * 2);
        c->kc.zero();
        c->vtc.zero();
        c->att.alloc(S * hq * 2);
        c->gate_up.alloc(S * 2 * ffn * 2);
        c->act.alloc(S * ffn * 2);
        // attention scratch for the most demanding sequence length, so forward() never allocates
        size_t ws = 0;
        for (int seq = 1; seq <= max_seq; ++seq) {
            const size_t b = vla_attn_workspace_bytes(VLA_DT_BF16_P2, 1, seq, n_q, n_kv, head_dim, seq);
            if (b == VLA_ATTN_WORKSPACE_UNSUPPORTED) throw std::invalid_argument("no attention kernel takes this head geometry");
            if (b > ws) ws = b;
        }
        c->attn_ws.alloc(ws);
        c->attn_ws.zero();
        return c;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla(bitvla_lm_hip): init failed: %s\n", e.what());
        delete c;
        return nullptr;
    }
}

void bitvla_lm_hip_free(bitvla_lm_hip_ctx* ctx) { delete ctx; }

void bitvla_lm_hip_set_layer(bitvla_lm_hip_ctx* ctx, int L, const bitvla_lm_layer_hip* layer) {
    if (!ctx || !layer || L < 0 || L >= ctx->n_layers) return;
    ctx->layers[(size_t)L] = *layer;
    const bitvla_lm_layer_hip& w = *layer;
    ctx->bound[(size_t)L] = w.attn_norm_w && w.attn_sub_norm_w && w.ffn_norm_w && w.ffn_sub_norm_w && w.q_packed && w.q_ws &&
                            w.k_packed && w.k_ws && w.v_packed && w.v_ws && w.o_packed && w.o_ws && w.gate_up_packed &&
                            w.gate_up_ws && w.down_packed && w.down_ws;
}

void bitvla_lm_hip_set_output_norm(bitvla_lm_hip_ctx* ctx, const uint16_t* w) {
    if (ctx) ctx->out_norm = w;
}

int bitvla_lm_hip_forward(bitvla_lm_hip_ctx* ctx, const uint16_t* d_in, uint16_t* d_out, int seq, vla_stream_t stream) {
    if (!ctx || !d_in || !d_out || seq <= 0) return -1;
    if (seq > ctx->max_seq) {
        std::fprintf(stderr, "vla(bitvla_lm_hip): seq=%d > max_seq=%d\n", seq, ctx->max_seq);
        return -1;
    }
    if (!ctx->out_norm) {
        std::fprintf(stderr, "vla(bitvla_lm_hip): output norm not bound\n");
        return -1;
    }
    for (int L = 0; L < ctx->n_layers; ++L)
        if (!ctx->bound[(size_t)L]) {
            std::fprintf(stderr, "vla(bitvla_lm_hip): layer %d not bound\n", L);
            return -1;
        }
    try {
        return run(ctx, d_in, d_out, seq, (hipStream_t)stream);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla(bitvla_lm_hip): forward failed: %s\n", e.what());
        return -1;
    }
}

}  // extern "C"
