// BitVLA-shape ternary (b1.58) attention path with a resident KV cache.
//
// Arithmetic of one layer follows the reference's CUDA forward, run_layer
// (src/kernels/bitvla/bitvla_lm_cuda.cu:422-486): bf16 RMSNorm -> per-token
// int8 act-quant -> ternary QKV GEMM (int32 accumulate, bf16 out) -> NeoX RoPE
// on Q and K -> attention -> bf16 sub-norm -> act-quant -> ternary O GEMM ->
// bf16 residual add.  Differences, all by design: Q|K|V is one fused GEMM
// (N = 3840, the shape bitnet_kernels.cu:112 registers as "head.qkv"); K/V are
// written into the resident cache instead of being expanded by repeat_kv; the
// attention is one fused kernel with fp32 scores instead of two cuBLAS GEMMs
// around a bf16 score buffer; the FFN half of the layer is not on this path.
//
// The reference runs one bidirectional pass with no cache
// (src/models/bitvla.cpp:205-238).  Here the prefix (image + text tokens) is
// prefilled once, then action tokens are appended one at a time, each
// attending to the prefix and to the tokens appended before it.
//
// Weight preparation at load restates recover_ternary_and_scale and the
// per-source scales of pack_and_upload_fused (src/models/bitvla.cpp:430-451,
// 523-543); ladder-packed tensors ("*.i2") are re-ordered word by word into the
// gfx950 layout.

#include <algorithm>
#include <cmath>
#include <random>

#include "checkpoint.h"
#include "layers.h"
#include "model.h"

namespace vla {
namespace {

int round_up(int x, int m) { return (x + m - 1) / m * m; }

struct TernaryW {
    DevBuf packed;  // [N][K/16] words
    DevBuf paired;  // fused QKV only: the same words with rotation pairs in one 32-row block (decode launch)
    DevBuf ws;      // fp32 [ws_num]
    int N = 0, K = 0, ws_num = 1;
};

// `parts` = row counts of the tensors fused into `name` (one absmean each).
// pair_q / pair_kv / pair_d > 0: also keep the row order of vla_ternary_pair_rope_rows_host.
TernaryW load_ternary(const Checkpoint& ck, const std::string& name, const std::vector<int>& parts, int K, int ws_group,
                      int pair_q = 0, int pair_kv = 0, int pair_d = 0) {
    TernaryW w;
    w.K = K;
    for (int n : parts) w.N += n;
    std::vector<uint32_t> packed((size_t)vla_ternary_packed_words(w.N, K));
    std::vector<float> scales;
    if (ck.has(name + ".i2")) {
        if (ck.info(name + ".i2").nbytes != (size_t)w.N * K / 4 || w.N % 16 || K % 128)
            throw std::runtime_error("vla: " + name + ".i2 does not hold " + std::to_string(w.N) + " x " + std::to_string(K) + " ladder-packed weights");
        VLA_K(vla_ternary_repack_ladder_host((const uint8_t*)ck.data(name + ".i2"), w.N, K, packed.data()));
        scales = ck.f32(name + ".ws");
        if (scales.size() != parts.size()) throw std::runtime_error("vla: " + name + ".ws has the wrong length");
    } else if (ck.has(name + ".p2")) {  // already in the gfx950 word order
        if (ck.info(name + ".p2").nbytes != packed.size() * 4) throw std::runtime_error("vla: " + name + ".p2 has the wrong size");
        std::memcpy(packed.data(), ck.data(name + ".p2"), packed.size() * 4);
        scales = ck.f32(name + ".ws");
        if (scales.size() != parts.size()) throw std::runtime_error("vla: " + name + ".ws has the wrong length");
    } else {
        ck.expect(name, {(int64_t)w.N, (int64_t)K});
        const std::vector<float> W = ck.f32(name);
        std::vector<int8_t> tern((size_t)w.N * K);
        size_t row = 0;
        for (int n : parts) {
            float am = 0.f;
            VLA_K(vla_ternary_quant_host(W.data() + row * K, (int64_t)n * K, tern.data() + row * K, &am));
            scales.push_back(am);
            row += n;
        }
        VLA_K(vla_ternary_pack_host(tern.data(), w.N, K, packed.data()));
    }
    // The epilogue indexes scales by n / (N / ws_num): expand to equal groups.
    std::vector<float> ws;
    for (size_t p = 0; p < parts.size(); ++p)
        for (int g = 0; g < parts[p] / ws_group; ++g) ws.push_back(scales[p]);
    w.ws_num = (int)ws.size();
    w.packed.upload(packed.data(), packed.size() * 4);
    w.ws.upload(ws.data(), ws.size() * 4);
    if (pair_d > 0 && pair_d % 32 == 0 && K % 32 == 0 && ws_group % pair_d == 0 && w.N == (pair_q + 2 * pair_kv) * pair_d) {
        std::vector<uint32_t> paired(packed.size());
        VLA_K(vla_ternary_pair_rope_rows_host(packed.data(), pair_q, pair_kv, pair_d, K, paired.data()));
        w.paired.upload(paired.data(), paired.size() * 4);
    }
    return w;
}

struct LmLayer {
    DevBuf attn_norm, sub_norm;
    TernaryW Wqkv, Wo;
    DevBuf ffn_norm, ffn_sub_norm;  // the GLU half, present when the checkpoint carries ffn_dim
    TernaryW Wgu, Wd;
    KVLayer kv;
};

class BitvlaLm : public ModelArch {
  public:
    explicit BitvlaLm(const Checkpoint& ck);
    void prefill(const Inputs* in, int batch) override;
    int steps_per_chunk() const override { return n_act_; }
    std::vector<float> fetch() override;
    int64_t n_actions() const override { return n_act_; }

  protected:
    void run_steps(int n_steps, void* stream) override;
    uint64_t launch_key() const override { return ((uint64_t)alloc_gen_ << 32) ^ (uint64_t)B_; }

  private:
    uint32_t alloc_gen_ = 0;
    int tuning_gen_ = -1;
    DevBuf zeros_;
    // last_out: where the last layer's closing projection writes the hidden rows (nullptr: in
    // place); honoured on the few-row decode path only, returns whether it was.  first_in: the
    // rows entering the first layer when they are not in h_ yet (decode path only, as last_out).
    bool run_layers(Ctx& C, int M, int S, int tok_offset, int n_keys, uint16_t* last_out = nullptr,
                    const uint16_t* first_in = nullptr);
    // a handful of rows (token-by-token decode): norm, quantisation and projection in one launch
    bool few_rows(int M) const { return M <= 8 && H_ <= 4096 && H_ % 128 == 0; }
    int L_, Hq_, Hkv_, D_, H_, A_, n_act_, n_img_, n_lang_, vocab_, F_ = 0, P_ = 0, B_ = 0;
    float eps_;
    std::vector<LmLayer> layers_;
    std::vector<float> E_lang_, act_emb_;
    std::shared_ptr<RowSource> lang_rows_;
    DevBuf out_norm_, W_out_, b_out_;
    RopeTable rope_;
    AttnWorkspace attn_ws_;
    DevBuf h_, hn_, q8_, s_, rowsum_, qkv_, q_, att_, o_, emb_bcast_, hfin_, x_, gu_, act_;
    hipStream_t last_stream_ = nullptr;
};

BitvlaLm::BitvlaLm(const Checkpoint& ck) {
    L_ = (int)ck.i64("n_layers");
    Hq_ = (int)ck.i64("n_q_heads");
    Hkv_ = (int)ck.i64("n_kv_heads");
    D_ = (int)ck.i64("head_dim");
    H_ = (int)ck.i64("hidden");
    A_ = (int)ck.i64("max_action_dim");
    n_act_ = (int)ck.i64("n_suffix");
    n_img_ = (int)ck.i64("n_img");
    n_lang_ = (int)ck.i64("n_lang");
    vocab_ = (int)ck.i64("vocab");
    eps_ = (float)ck.f64("rms_eps", 1e-5);
    F_ = (int)ck.i64("ffn_dim", 0);
    if (F_ % 128) throw std::runtime_error("vla(bitvla): ffn_dim must be a multiple of 128");
    if (Hq_ * D_ != H_) throw std::runtime_error("vla(bitvla): n_q_heads * head_dim must equal hidden");
    cfg.n_img = n_img_; cfg.n_lang = n_lang_; cfg.n_prefix = n_img_ + n_lang_; cfg.n_suffix = n_act_;
    cfg.n_full = cfg.n_prefix + n_act_;
    cfg.hidden = H_; cfg.expert_h = H_; cfg.n_q_heads = Hq_; cfg.n_kv_heads = Hkv_; cfg.head_dim = D_;
    cfg.q_full_dim = H_; cfg.kv_full_dim = (int64_t)Hkv_ * D_; cfg.n_layers = L_;
    cfg.max_action_dim = A_; cfg.real_action_dim = ck.i64("real_action_dim", A_);
    cfg.max_state_dim = 0; cfg.real_state_dim = 0;
    cfg.num_steps = n_act_; cfg.rms_eps = eps_; cfg.rope_n_dims = D_;
    cfg.rope_freq_base = (float)ck.f64("rope_freq_base", 500000.0);

    lang_rows_ = ck.row_source("prefix.E_lang");  // a large vocabulary stays on disk
    if (lang_rows_) {
        if (lang_rows_->rows != vocab_ || lang_rows_->cols != H_) throw std::runtime_error("vla: token embedding matrix does not match vocab x hidden");
    } else {
        ck.expect("prefix.E_lang", {(int64_t)vocab_, (int64_t)H_});
        E_lang_ = ck.f32("prefix.E_lang");
    }
    ck.expect("act.emb", {(int64_t)n_act_, (int64_t)H_});
    ck.expect("act.norm", {(int64_t)H_});
    ck.expect("act.W_out", {(int64_t)A_, (int64_t)H_});
    ck.expect("act.b_out", {(int64_t)A_});
    act_emb_ = ck.f32("act.emb");
    std::vector<float> nf = ck.f32("act.norm");
    upload_as(out_norm_, nf.data(), nf.size(), VLA_DT_BF16);
    { std::vector<float> t = ck.f32("act.W_out"); W_out_.upload(t.data(), t.size() * 4); }
    { std::vector<float> t = ck.f32("act.b_out"); b_out_.upload(t.data(), t.size() * 4); }
    const int kvd = Hkv_ * D_;
    layers_.resize(L_);
    for (int l = 0; l < L_; ++l) {
        const std::string p = "lm." + std::to_string(l) + ".";
        LmLayer& w = layers_[l];
        ck.expect(p + "attn_norm", {(int64_t)H_});
        ck.expect(p + "sub_norm", {(int64_t)H_});
        std::vector<float> a = ck.f32(p + "attn_norm"), s = ck.f32(p + "sub_norm");
        upload_as(w.attn_norm, a.data(), a.size(), VLA_DT_BF16);
        upload_as(w.sub_norm, s.data(), s.size(), VLA_DT_BF16);
        w.Wqkv = load_ternary(ck, p + "Wqkv", {H_, kvd, kvd}, H_, kvd, Hq_, Hkv_, D_);
        w.Wo = load_ternary(ck, p + "Wo", {H_}, H_, H_);
        if (F_ > 0) {
            ck.expect(p + "ffn_norm", {(int64_t)H_});
            ck.expect(p + "ffn_sub_norm", {(int64_t)F_});
            std::vector<float> fn = ck.f32(p + "ffn_norm"), fs = ck.f32(p + "ffn_sub_norm");
            upload_as(w.ffn_norm, fn.data(), fn.size(), VLA_DT_BF16);
            upload_as(w.ffn_sub_norm, fs.data(), fs.size(), VLA_DT_BF16);
            w.Wgu = load_ternary(ck, p + "Wgu", {F_, F_}, H_, F_);
            w.Wd = load_ternary(ck, p + "Wd", {H_}, F_, H_);
        }
    }
}

void BitvlaLm::prefill(const Inputs* in, int batch) {
    if (!in || batch <= 0) throw std::invalid_argument("vla: prefill needs at least one observation");
    const int P = n_img_ + n_lang_, B = batch;
    for (int b = 0; b < B; ++b) {
        if (!in[b].precomputed_img_emb || in[b].n_img_views != 1) throw std::invalid_argument("vla(bitvla): one view of precomputed_img_emb is required");
        if (in[b].n_lang != n_lang_ || !in[b].lang_tokens) throw std::invalid_argument("vla(bitvla): n_lang must equal the configured text length");
        for (int i = 0; i < n_lang_; ++i)
            if (in[b].lang_tokens[i] < 0 || in[b].lang_tokens[i] >= vocab_) throw std::invalid_argument("vla: language token outside the vocabulary");
    }
    const int t_max = round_up(P + n_act_, 64);
    const int tuning_gen = vla_kernels_tuning_generation();  // the attention workspace is planned under the tuning overrides
    if (B != B_ || P != P_ || tuning_gen != tuning_gen_) {
        tuning_gen_ = tuning_gen;
        B_ = B;
        P_ = P;
        const size_t M = (size_t)B * P;
        for (LmLayer& w : layers_) {
            w.kv.create(VLA_DT_BF16, B, Hkv_, D_, t_max);
            w.kv.n_prefix = P;
        }
        h_.alloc(M * H_ * 2); hn_.alloc(M * H_ * 2); q8_.alloc(M * (size_t)(F_ > H_ ? F_ : H_)); s_.alloc(M * 4); rowsum_.alloc(M * 4);
        if (F_ > 0) { gu_.alloc(M * 2 * F_ * 2); act_.alloc(M * F_ * 2); }
        qkv_.alloc(M * (H_ + 2 * Hkv_ * D_) * 2); q_.alloc(M * H_ * 2); att_.alloc(M * H_ * 2); o_.alloc(M * H_ * 2);
        hfin_.alloc((size_t)n_act_ * B * H_ * 2);
        x_.alloc((size_t)n_act_ * B * A_ * 4);
        zeros_.alloc((size_t)n_act_ * B * A_ * 4);
        zeros_.zero();
        attn_ws_.reset();
        attn_ws_.plan(VLA_DT_BF16_P2, B, P, Hq_, Hkv_, D_, P);  // prefill
        for (int t = 0; t < n_act_; ++t) attn_ws_.plan(VLA_DT_BF16_P2, B, 1, Hq_, Hkv_, D_, P + t + 1);  // appended tokens
        attn_ws_.commit();
        ++alloc_gen_;
        std::vector<int32_t> pos(P + n_act_);
        for (int i = 0; i < P + n_act_; ++i) pos[i] = i;  // src/models/bitvla.cpp positions 0..seq-1
        rope_.build(RopeSpec{D_, cfg.rope_freq_base}, pos);
        std::vector<uint16_t> eb((size_t)n_act_ * B * H_);
        for (int t = 0; t < n_act_; ++t)
            for (int b = 0; b < B; ++b)
                for (int c = 0; c < H_; ++c) eb[((size_t)t * B + b) * H_ + c] = f32_to_bf16(act_emb_[(size_t)t * H_ + c]);
        emb_bcast_.upload(eb.data(), eb.size() * 2);
    }
    std::vector<uint16_t> emb((size_t)B * P * H_);
    for (int b = 0; b < B; ++b) {
        uint16_t* dst = emb.data() + (size_t)b * P * H_;
        for (size_t i = 0; i < (size_t)n_img_ * H_; ++i) dst[i] = f32_to_bf16(in[b].precomputed_img_emb[i]);
        std::vector<float> fetched;
        if (lang_rows_) {
            fetched.resize((size_t)n_lang_ * H_);
            const std::vector<int32_t> ids(in[b].lang_tokens, in[b].lang_tokens + n_lang_);
            if (n_lang_ > 0 && !lang_rows_->fetch_locked(ids, fetched.data())) throw std::runtime_error("vla: cannot read token embedding rows");
        }
        for (int i = 0; i < n_lang_; ++i) {
            const float* e = lang_rows_ ? fetched.data() + (size_t)i * H_ : E_lang_.data() + (size_t)in[b].lang_tokens[i] * H_;
            for (int c = 0; c < H_; ++c) dst[(size_t)(n_img_ + i) * H_ + c] = f32_to_bf16(e[c]);
        }
    }
    h_.upload(emb.data(), emb.size() * 2);
    Ctx C;
    prof_start("prefill", C.stream);
    run_layers(C, B * P, P, 0, P);
    VLA_HIP(hipDeviceSynchronize());
}

// One pass of all layers over M = B*S rows sitting in h_ (S consecutive tokens
// per observation starting at cache slot tok_offset, attending to n_keys keys).
bool BitvlaLm::run_layers(Ctx& C, int M, int S, int tok_offset, int n_keys, uint16_t* last_out, const uint16_t* first_in) {
    const int kvd = Hkv_ * D_, Nqkv = H_ + 2 * kvd;
    const int half = D_ / 2;
    const float scale = 1.0f / std::sqrt((float)D_);
    const float* cos_t = rope_.cos.as<float>() + (size_t)tok_offset * half;
    const float* sin_t = rope_.sin.as<float>() + (size_t)tok_offset * half;
    const bool fused = few_rows(M);
    const bool redirect = last_out && fused && F_ <= 4096;
    for (LmLayer& w : layers_) {
        const bool last = &w == &layers_.back();
        // the hidden rows as this layer finds them: h_, except in front of the first layer
        const uint16_t* hin = (redirect && first_in && &w == &layers_.front()) ? first_in : h_.as<uint16_t>();
        if (fused && S == 1 && w.Wqkv.paired.get()) {
            // ... and the split, rotation and cache append as well
            VLA_K(vla_rmsnorm_ternary_gemv_rope_append(hin, w.attn_norm.as<uint16_t>(), eps_,
                                                       w.Wqkv.paired.as<uint32_t>(), w.Wqkv.ws.as<float>(), w.Wqkv.ws_num,
                                                       cos_t, sin_t, q_.as<uint16_t>(), w.kv.k.as<uint16_t>(),
                                                       w.kv.vt.as<uint16_t>(), M, Hq_, Hkv_, D_, H_, w.kv.t_max, tok_offset,
                                                       C.stream));
            prof_mark("norm_quant_qkv_gemv_rope_append");
        } else if (fused) {
            VLA_K(vla_rmsnorm_ternary_gemv(hin, w.attn_norm.as<uint16_t>(), eps_, w.Wqkv.packed.as<uint32_t>(),
                                           qkv_.as<uint16_t>(), nullptr, w.Wqkv.ws.as<float>(), w.Wqkv.ws_num, M, Nqkv, H_,
                                           C.stream));
            prof_mark("norm_quant_qkv_gemv");
        } else {
            VLA_K(vla_rmsnorm_act_quant_bf16(h_.as<uint16_t>(), w.attn_norm.as<uint16_t>(), q8_.as<int8_t>(), s_.as<float>(),
                                             rowsum_.as<int32_t>(), eps_, M, H_, C.stream));
            prof_mark("norm_quant");
            VLA_K(vla_ternary_gemm(q8_.as<int8_t>(), w.Wqkv.packed.as<uint32_t>(), qkv_.as<uint16_t>(), nullptr,
                                   s_.as<float>(), rowsum_.as<int32_t>(), w.Wqkv.ws.as<float>(), w.Wqkv.ws_num, M, Nqkv, H_,
                                   C.stream));
            prof_mark("ternary_qkv_gemm");
        }
        if (!(fused && S == 1 && w.Wqkv.paired.get())) {
            VLA_K(vla_qkv_split_rope_append(qkv_.get(), cos_t, sin_t, q_.get(), w.kv.k.get(), w.kv.vt.get(), VLA_DT_BF16, M, S,
                                            Hq_, Hkv_, D_, w.kv.t_max, tok_offset, C.stream));
            prof_mark("qkv_split_rope_append");
        }
        VLA_K(vla_attn_prefix_suffix_ws(q_.get(), w.kv.k.get(), w.kv.vt.get(), att_.get(), VLA_DT_BF16_P2, M / S, S, Hq_, Hkv_,
                                        D_, w.kv.t_max, n_keys, scale, VLA_MASK_NONE, n_keys, 0, 0, nullptr, attn_ws_.buf.get(),
                                        attn_ws_.buf.bytes(), C.stream));
        prof_mark("attention");
        // O projection and the residual add of the hidden stream in one launch
        if (fused) {
            VLA_K(vla_rmsnorm_ternary_gemv(att_.as<uint16_t>(), w.sub_norm.as<uint16_t>(), eps_, w.Wo.packed.as<uint32_t>(),
                                           redirect && last && F_ == 0 ? last_out : h_.as<uint16_t>(), hin,
                                           w.Wo.ws.as<float>(), w.Wo.ws_num, M, H_, H_, C.stream));
            prof_mark("norm_quant_o_gemv_add");
        } else {
            VLA_K(vla_rmsnorm_act_quant_bf16(att_.as<uint16_t>(), w.sub_norm.as<uint16_t>(), q8_.as<int8_t>(), s_.as<float>(),
                                             rowsum_.as<int32_t>(), eps_, M, H_, C.stream));
            prof_mark("norm_quant");
            VLA_K(vla_ternary_gemm_add(q8_.as<int8_t>(), w.Wo.packed.as<uint32_t>(), h_.as<uint16_t>(), h_.as<uint16_t>(),
                                       s_.as<float>(), rowsum_.as<int32_t>(), w.Wo.ws.as<float>(), w.Wo.ws_num, M, H_, H_,
                                       C.stream));
            prof_mark("ternary_o_gemm_add");
        }
        if (F_ == 0) continue;
        // the GLU half: ffn norm -> [gate | up] -> relu(gate)^2 * up -> sub-norm -> down + residual
        if (fused) {
            VLA_K(vla_rmsnorm_ternary_gemv(h_.as<uint16_t>(), w.ffn_norm.as<uint16_t>(), eps_, w.Wgu.packed.as<uint32_t>(),
                                           gu_.as<uint16_t>(), nullptr, w.Wgu.ws.as<float>(), w.Wgu.ws_num, M, 2 * F_, H_,
                                           C.stream));
            prof_mark("norm_quant_gate_up_gemv");
        } else {
            VLA_K(vla_rmsnorm_act_quant_bf16(h_.as<uint16_t>(), w.ffn_norm.as<uint16_t>(), q8_.as<int8_t>(), s_.as<float>(),
                                             rowsum_.as<int32_t>(), eps_, M, H_, C.stream));
            prof_mark("norm_quant");
            VLA_K(vla_ternary_gemm(q8_.as<int8_t>(), w.Wgu.packed.as<uint32_t>(), gu_.as<uint16_t>(), nullptr, s_.as<float>(),
                                   rowsum_.as<int32_t>(), w.Wgu.ws.as<float>(), w.Wgu.ws_num, M, 2 * F_, H_, C.stream));
            prof_mark("ternary_gate_up_gemm");
        }
        if (fused && F_ <= 4096) {  // activation, sub-norm, quantisation and down projection in one launch
            VLA_K(vla_sqrelu_rmsnorm_ternary_gemv(gu_.as<uint16_t>(), w.ffn_sub_norm.as<uint16_t>(), eps_,
                                                  w.Wd.packed.as<uint32_t>(), redirect && last ? last_out : h_.as<uint16_t>(),
                                                  h_.as<uint16_t>(), w.Wd.ws.as<float>(), w.Wd.ws_num, M, H_, F_, C.stream));
            prof_mark("sqrelu_norm_quant_down_gemv_add");
            continue;
        }
        // Longer rows (the model's 6912): every 32-column workgroup of the one-launch form would
        // repeat the rows' activation and norm, which costs more than a launch; the activation
        // still stays on chip, inside the norm + quantisation launch.
        const int rc = vla_sqrelu_rmsnorm_act_quant_bf16(gu_.as<uint16_t>(), w.ffn_sub_norm.as<uint16_t>(), q8_.as<int8_t>(),
                                                         s_.as<float>(), rowsum_.as<int32_t>(), eps_, M, F_, C.stream);
        if (rc != VLA_K_ERR_SHAPE) VLA_K(rc);
        else {  // rows the one-wavefront kernel does not hold
            VLA_K(gate_up_fused_sqrelu_mul_bf16(gu_.as<uint16_t>(), act_.as<uint16_t>(), M, F_, C.stream));
            VLA_K(vla_rmsnorm_act_quant_bf16(act_.as<uint16_t>(), w.ffn_sub_norm.as<uint16_t>(), q8_.as<int8_t>(), s_.as<float>(),
                                             rowsum_.as<int32_t>(), eps_, M, F_, C.stream));
        }
        prof_mark("sqrelu_norm_quant");
        VLA_K(vla_ternary_gemm_add(q8_.as<int8_t>(), w.Wd.packed.as<uint32_t>(), h_.as<uint16_t>(), h_.as<uint16_t>(),
                                   s_.as<float>(), rowsum_.as<int32_t>(), w.Wd.ws.as<float>(), w.Wd.ws_num, M, H_, F_,
                                   C.stream));
        prof_mark("ternary_down_gemm_add");
    }
    return redirect;
}

void BitvlaLm::run_steps(int n_steps, void* stream) {
    if (B_ == 0) throw std::logic_error("vla: denoise before prefill");
    Ctx C;
    C.stream = (hipStream_t)stream;
    last_stream_ = C.stream;
    const int B = B_;
    const size_t row = (size_t)B * H_;
    // one step = one appended action token through every layer; the action head runs
    // when the last token of a chunk is done
    prof_start("step", C.stream);
    for (int it = 0; it < n_steps; ++it) {
        const int t = it % n_act_;
        if (t == 0) attn_ws_.begin(C.stream);
        // Where the few-row launches apply (`direct`, a matter of shapes only), the first layer reads
        // token t's embedding rows where they lie and the last layer leaves its rows in hfin_: no
        // copy in front, and one final norm over all tokens' rows in front of the action head.
        const uint16_t* emb = emb_bcast_.as<uint16_t>() + (size_t)t * row;
        uint16_t* hf = hfin_.as<uint16_t>() + (size_t)t * row;
        const bool direct = few_rows(B) && F_ <= 4096;
        if (!direct) {
            VLA_HIP(hipMemcpyAsync(h_.get(), emb, row * 2, hipMemcpyDeviceToDevice, C.stream));
            prof_mark("token_embedding");
        }
        const bool raw = run_layers(C, B, 1, P_ + t, P_ + t + 1, hf, emb);
        if (!raw) {
            VLA_K(bitvla_rmsnorm_bf16(h_.as<uint16_t>(), out_norm_.as<uint16_t>(), hf, eps_, B, H_, C.stream));
            prof_mark("final_norm");
        }
        if (t == n_act_ - 1) {
            // cleared by a copy node: memset nodes are kept out of captured graphs
            VLA_HIP(hipMemcpyAsync(x_.get(), zeros_.get(), (size_t)n_act_ * B * A_ * 4, hipMemcpyDeviceToDevice, C.stream));
            // x[t][b] = W_out . norm(h[t][b]) + b_out (batch' = n_act, rows = B, unit step)
            if (raw)  // every token's rows at once, in place
                VLA_K(bitvla_rmsnorm_bf16(hfin_.as<uint16_t>(), out_norm_.as<uint16_t>(), hfin_.as<uint16_t>(), eps_, n_act_ * B, H_,
                                          C.stream));
            VLA_K(vla_euler_step(x_.as<float>(), hfin_.get(), W_out_.as<float>(), b_out_.as<float>(), VLA_DT_BF16, n_act_, B, 0,
                                 A_, H_, 1.0f, C.stream));
            prof_mark("action_head");
        }
    }
}

std::vector<float> BitvlaLm::fetch() {
    VLA_HIP(hipDeviceSynchronize());
    std::vector<float> tb((size_t)n_act_ * B_ * A_), out(tb.size());
    x_.download(tb.data(), tb.size() * 4);
    for (int t = 0; t < n_act_; ++t)
        for (int b = 0; b < B_; ++b)
            for (int j = 0; j < A_; ++j)
                out[((size_t)b * n_act_ + t) * A_ + j] = j < cfg.real_action_dim ? tb[((size_t)t * B_ + b) * A_ + j] : 0.f;
    return out;
}

}  // namespace

ModelArch* bitvla_create(const Checkpoint& ck) { return new BitvlaLm(ck); }

}  // namespace vla
