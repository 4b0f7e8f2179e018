// Flow-matching / DiT action experts on the resident-KV attention path:
// SmolVLA, pi0 and GR00T N1.5 schedules over the same kernels.
//
// What is restated from the reference (graph builders that record ggml nodes
// there, eager launches here):
//   SmolVLA  build_vlm_layer's K/V outputs, expert_cross_kv,
//            build_expert_self_attn_layer, build_expert_cross_attn_layer and
//            the denoise loop of build_compute_graph
//            (src/models/smolvla.cpp:778-888, 1376-1419), masks and positions
//            of predict (1608-1672)
//   pi0      build_gemma_layer prefix / suffix passes, build_embed_suffix, the
//            step loop and the full mask (src/models/pi0.cpp:159-248, 536-661)
//   GR00T    DitHead::kv hoisted out of the solver loop, DitHead::block's
//            adaLN -> Q(KV) -> attention -> Wo, the Euler loop
//            (src/modules/dit_head.cpp:87-133, src/models/gr00tn1d5.cpp:359-381)
// The FFN half of each layer, the VLM backbone between prefix layers and the
// vision towers are not part of this path: every prefix layer projects the same
// prefix embeddings, and a layer is pre-norm -> QKV(+RoPE, +append) ->
// attention -> Wo + residual.
//
// The prefix K/V of every layer is written once per observation and stays in
// HBM; each denoise step overwrites only the S suffix slots behind it.

#include <algorithm>
#include <chrono>
#include <cmath>
#include <random>
#include <thread>

#include "checkpoint.h"
#include "layers.h"
#include "model.h"

namespace vla {
namespace {

enum class Arch { SMOLVLA, PI0, GR00T };

int round_up(int x, int m) { return (x + m - 1) / m * m; }

// Every load names the shape the configuration implies: a file whose tensors do not match its
// own keys fails here, not as a device read past a buffer.
using Shape = std::vector<int64_t>;
DevBuf load_w(const Checkpoint& ck, const std::string& name, int dtype, const Shape& shape) {
    const CkptTensor& t = ck.expect(name, shape);
    DevBuf b;
    if ((dtype == VLA_DT_F32 && t.dtype == "f32") || (dtype == VLA_DT_BF16 && t.dtype == "bf16")) {
        b.upload(ck.data(name), t.nbytes);
    } else {
        std::vector<float> f = ck.f32(name);
        upload_as(b, f.data(), f.size(), dtype);
    }
    return b;
}
DevBuf load_f32(const Checkpoint& ck, const std::string& name, const Shape& shape) { return load_w(ck, name, VLA_DT_F32, shape); }
std::vector<float> host_f32(const Checkpoint& ck, const std::string& name, const Shape& shape) {
    ck.expect(name, shape);
    return ck.f32(name);
}

// bf16 copy of weight `name` [N][K] with the RMSNorm weight `ln` [K] multiplied into its
// columns, for the projection launch that takes the layer's pre-norm inside it.
DevBuf load_folded_bf16(const Checkpoint& ck, const std::string& name, const std::string& ln, int64_t rows, int64_t cols) {
    const std::vector<float> wf = host_f32(ck, name, {rows, cols}), gf = host_f32(ck, ln, {cols});
    const size_t K = gf.size(), N = wf.size() / K;
    std::vector<uint16_t> w(wf.size()), g(K);
    for (size_t i = 0; i < wf.size(); ++i) w[i] = f32_to_bf16(wf[i]);
    for (size_t k = 0; k < K; ++k) g[k] = f32_to_bf16(gf[k]);
    VLA_K(vla_fold_norm_weight_host(w.data(), g.data(), VLA_DT_BF16, (int)N, (int)K, w.data()));
    DevBuf b;
    b.upload(w.data(), w.size() * sizeof(uint16_t));
    return b;
}

// y = W x + b on the host, W [N][K] row-major, double accumulation.
void host_linear(const float* W, const float* b, const float* x, float* y, int N, int K) {
    for (int n = 0; n < N; ++n) {
        double a = 0.0;
        const float* wr = W + (size_t)n * K;
        for (int k = 0; k < K; ++k) a += (double)wr[k] * (double)x[k];
        y[n] = (float)(a + (b ? (double)b[n] : 0.0));
    }
}
float host_silu(float x) { return x / (1.0f + std::exp(-x)); }

struct LayerW {
    bool is_self = true;
    DevBuf ln;                  // expert pre-norm weight (RMS archs)
    DevBuf Wqkv, bqkv;          // self: Q|K|V rows, cross: Q rows
    DevBuf Wqkv_ln;             // the same rows with the pre-norm weight folded in (bf16 RMS archs)
    // bf16 DiT blocks: per denoise step, the rows with (1 + scale) of the block's modulated
    // LayerNorm folded in [steps][rows][W], their column sums and the bias with the shift
    // folded in [steps][rows] (vla_layernorm_attn_qkv_rope)
    DevBuf Wqkv_ada, cs_ada, b_ada;
    DevBuf Wo, bo;
    DevBuf ln2, Wgu, Wgu_ln, Wd;      // FFN half of an RMS-norm layer: post-attention norm, [gate; up], down
    DevBuf W1, b1, W2, b2;            // FFN half of a DiT block (ffn_gelu)
    DevBuf vlm_ln, Wkv_pre, bkv_pre;  // prefix K|V producer
    DevBuf Wk_x, Wv_x;          // SmolVLA cross layers: re-projection of the cached prefix K / V
    KVLayer kv;
    bool needs_prefix = true;
    bool from_text = false;  // cross K/V from the text rows of the prefix (else image rows, or all rows)
};

class FlowExpert : public ModelArch {
  public:
    explicit FlowExpert(const Checkpoint& ck);
    void prefill(const Inputs* in, int batch) override;
    int steps_per_chunk() const override { return steps_; }
    std::vector<float> fetch() override;
    int64_t n_actions() const override { return S_ - n_lead_; }

  protected:
    void run_steps(int n_steps, void* stream) override;
    uint64_t launch_key() const override {
        return ((uint64_t)alloc_gen_ << 40) ^ ((uint64_t)pad_start_ << 20) ^ (uint64_t)pad_end_ ^ ((uint64_t)P_ << 52);
    }

  private:
    void allocate(int B, int P, int P_txt = 0);
    uint32_t alloc_gen_ = 0;
    int tuning_gen_ = -1;

    Arch arch_;
    int dt_ = VLA_DT_F32;
    int L_ = 0, Hq_ = 0, Hkv_ = 0, D_ = 0, W_ = 0, Wv_ = 0, A_ = 0, S_ = 0, n_lead_ = 0, steps_ = 0;
    int I_ = 0;  // FFN width; 0 = the layers stop after the attention half
    int n_img_ = 0, n_lang_max_ = 0, max_views_ = 1, vocab_ = 0, max_state_ = 0;
    int suffix_mask_ = VLA_MASK_NONE;
    float eps_ = 1e-5f, final_eps_ = 1e-6f, dt_step_ = -0.1f;
    bool rope_ = true;

    std::vector<LayerW> layers_;
    // small fp32 tensors kept on the host for per-observation work
    std::vector<float> E_lang_, Wstate_, bstate_, W_sp_, b_sp_;
    DevBuf W_in_, W_out_, b_out_, final_norm_;
    DevBuf W_at2_, b_at2_, m1_;  // action-time MLP: second projection, fp32 scratch [B*S][W]
    bool time_mlp_ = false;
    // GR00T with the DiT head's own input / output MLPs (ActionExpert::encode_state / encode_action /
    // decode, src/modules/action_expert.cpp:41-59; DitHead::proj_out, src/modules/dit_head.cpp:139-147)
    bool head_io_ = false;
    int n_future_ = 0, O_ = 0, Hd_ = 0, Hs_ = 0;  // future tokens, DiT output width, decoder / state-encoder hidden widths
    std::vector<float> se_l1W_, se_l1b_, se_l2W_, se_l2b_, future_;
    DevBuf W3_, b3_, pos_, m2_, po2W_, po2b_, ad1W_, ad1b_, d1_, d2_;
    std::shared_ptr<RowSource> lang_rows_;  // token embeddings left on disk (large vocabularies)
    bool alt_vl_ = false;   // GR00T N1.6 / N1.7: cross layers alternate text / image rows
    int text_every_ = 2, P_txt_ = 0;
    DevBuf vlln_sc_, vlln_sh_;  // vlln as (weight - 1, bias) fp32 [Wv]: the modulated-norm launch computes xn (1 + sc) + sh
    float vlln_eps_ = 1e-5f;
    bool fuse_final_norm_ = true;  // the final norm runs inside the Euler launch
    bool fuse_self_block_ = true;  // GR00T self blocks: norm, projections and attention in one launch (VLA_NO_FUSED_SELF_BLOCK=1: off)
    bool hand_row_stats_ = true;   // GR00T from batch 32: a block's Wo launch leaves the row sums the next block's LayerNorm needs (VLA_NO_ROW_STATS=1: off)
    DevBuf row_stats_;             // [B * S][W / 64][2] fp32
    bool adarms_ = false;  // pi0.5: ada_ holds [steps][2L+1][scale, shift, gate][W]
    DevBuf bias_step_;   // [steps][W] fp32: b_in (+ time embedding of the step)
    DevBuf ada_;         // GR00T: [steps][L+1][2][W] fp32 (scale, shift); slot L is the final norm (zeros)

    // per-call state
    int B_ = 0, P_ = 0, pad_start_ = 0, pad_end_ = 0;
    RopeTable rope_prefill_, rope_self_, rope_cross_;
    DevBuf prefix_, prefix_n_, tmpk_, tmpv_, lead_, x0_, xt_, h_, hn_, q_, att_, mid_;
    PinnedBuf stage_;  // host staging of the prefix embeddings (page-locked)
    KVLayer tmp_kv_;
    AttnWorkspace attn_ws_;
    std::mt19937 rng_{std::random_device{}()};
    hipStream_t last_stream_ = nullptr;
};

FlowExpert::FlowExpert(const Checkpoint& ck) {
    const std::string arch = ck.str("arch");
    // pi0.5 is the pi0 schedule with adaRMS norms, gated residuals, no state token in the
    // suffix and no suffix mask (src/models/pi05.cpp:208-283, 610-631)
    adarms_ = arch == "pi05";
    arch_ = arch == "smolvla" ? Arch::SMOLVLA : (arch == "pi0" || adarms_) ? Arch::PI0 : Arch::GR00T;
    // GR00T N1.6 / N1.7 (AlternateVLDiT): the cross layers alternate between the text rows and
    // the image rows of the backbone features (src/models/gr00tn1d6.cpp:445-467,
    // src/models/gr00tn1d7.cpp:565-590); N1.5 attends to all rows on every cross layer.
    alt_vl_ = arch == "gr00t_n1d6";
    text_every_ = (int)ck.i64("attend_text_every_n", 2);
    const bool interleave = ck.i64("dit_interleave", 1) != 0;
    if (alt_vl_ && text_every_ < 1) throw std::runtime_error("vla: attend_text_every_n must be >= 1");
    dt_ = ck.str("dtype") == "bf16" ? VLA_DT_BF16 : VLA_DT_F32;
    L_ = (int)ck.i64("n_layers");
    Hq_ = (int)ck.i64("n_q_heads");
    Hkv_ = (int)ck.i64("n_kv_heads");
    D_ = (int)ck.i64("head_dim");
    W_ = (int)ck.i64("expert_h");
    I_ = (int)ck.i64("ffn_dim", 0);
    Wv_ = (int)ck.i64("hidden");
    A_ = (int)ck.i64("max_action_dim");
    S_ = (int)ck.i64("n_suffix");
    steps_ = (int)ck.i64("num_steps");
    n_img_ = (int)ck.i64("n_img");
    n_lang_max_ = (int)ck.i64("n_lang", 0);
    max_views_ = (int)ck.i64("max_views", 4);
    vocab_ = (int)ck.i64("vocab", 0);
    max_state_ = (int)ck.i64("max_state_dim", 32);
    eps_ = (float)ck.f64("rms_eps", arch_ == Arch::PI0 ? 1e-6 : 1e-5);
    final_eps_ = (float)ck.f64("norm_out_eps", 1e-6);
    suffix_mask_ = (int)ck.i64("suffix_mask", arch_ == Arch::SMOLVLA            ? VLA_MASK_CAUSAL_SUFFIX
                                              : (arch_ == Arch::PI0 && !adarms_) ? VLA_MASK_PI0_STATE
                                                                                 : VLA_MASK_NONE);
    head_io_ = arch_ == Arch::GR00T && ck.i64("head_io", 0) != 0;
    n_future_ = head_io_ ? (int)ck.i64("num_future") : 0;
    n_lead_ = (arch_ == Arch::SMOLVLA || adarms_) ? 0 : 1 + n_future_;
    rope_ = arch_ != Arch::GR00T;
    dt_step_ = (arch_ == Arch::GR00T ? 1.0f : -1.0f) / (float)steps_;
    const int every = (int)ck.i64("self_attn_every_n", arch_ == Arch::PI0 ? 1 : 2);

    cfg.n_img = n_img_;
    cfg.n_lang = n_lang_max_;
    cfg.n_state = arch_ == Arch::SMOLVLA ? 1 : 0;
    cfg.n_suffix = S_;
    cfg.hidden = Wv_;
    cfg.expert_h = W_;
    cfg.n_q_heads = Hq_;
    cfg.n_kv_heads = Hkv_;
    cfg.head_dim = D_;
    cfg.q_full_dim = (int64_t)Hq_ * D_;
    cfg.kv_full_dim = (int64_t)Hkv_ * D_;
    cfg.n_layers = L_;
    cfg.self_attn_every_n = every;
    cfg.max_state_dim = max_state_;
    cfg.max_action_dim = A_;
    cfg.real_state_dim = ck.i64("real_state_dim", max_state_);
    cfg.real_action_dim = ck.i64("real_action_dim", A_);
    cfg.min_period = ck.f64("min_period", 4e-3);
    cfg.max_period = ck.f64("max_period", 4.0);
    cfg.num_steps = steps_;
    cfg.rms_eps = eps_;
    cfg.rope_n_dims = D_;
    cfg.rope_freq_base = (float)ck.f64("rope_freq_base", 10000.0);
    cfg.denormalized = arch_ != Arch::GR00T;
    cfg.n_prefix = (int64_t)n_img_ + n_lang_max_ + cfg.n_state;
    cfg.n_full = cfg.n_prefix + S_;
    if (!config_is_sane(cfg)) throw std::runtime_error("vla: real_* dims exceed max_* dims");

    if (S_ <= n_lead_) throw std::runtime_error("vla: n_suffix leaves no action rows");
    const int64_t qd = (int64_t)Hq_ * D_, kvd = (int64_t)Hkv_ * D_;
    if (vocab_ > 0) {
        lang_rows_ = ck.row_source("prefix.E_lang");
        if (lang_rows_) {
            if (lang_rows_->rows != vocab_ || lang_rows_->cols != Wv_) throw std::runtime_error("vla: token embedding matrix does not match vocab x hidden");
        } else {
            E_lang_ = host_f32(ck, "prefix.E_lang", {vocab_, Wv_});
        }
    }
    if (ck.has("prefix.vlln_w")) {
        if (arch_ != Arch::GR00T) throw std::runtime_error("vla: prefix.vlln_w belongs to the GR00T heads");
        std::vector<float> sc = host_f32(ck, "prefix.vlln_w", {Wv_}), sh = host_f32(ck, "prefix.vlln_b", {Wv_});
        for (float& v : sc) v -= 1.0f;
        vlln_sc_.upload(sc.data(), sc.size() * sizeof(float));
        vlln_sh_.upload(sh.data(), sh.size() * sizeof(float));
        vlln_eps_ = (float)ck.f64("vlln_eps", 1e-5);
    }
    if (arch_ == Arch::SMOLVLA) {
        Wstate_ = host_f32(ck, "prefix.Wstate", {Wv_, max_state_});
        bstate_ = host_f32(ck, "prefix.bstate", {Wv_});
    } else if (head_io_) {
        O_ = (int)ck.i64("dit_out_dim");
        Hd_ = (int)ck.i64("dec_hidden");
        Hs_ = (int)ck.i64("state_hidden");
        se_l1W_ = host_f32(ck, "aex.se_l1W", {Hs_, max_state_});
        se_l1b_ = host_f32(ck, "aex.se_l1b", {Hs_});
        se_l2W_ = host_f32(ck, "aex.se_l2W", {W_, Hs_});
        se_l2b_ = host_f32(ck, "aex.se_l2b", {W_});
        if (n_future_ > 0) future_ = host_f32(ck, "aex.future_tokens", {n_future_, W_});  // N1.6 / N1.7 have none
    } else if (n_lead_ > 0) {
        W_sp_ = host_f32(ck, "act.W_sp", {W_, max_state_});
        b_sp_ = host_f32(ck, "act.b_sp", {W_});
    }
    if (head_io_) {
        // decode's second projection plays the part of W_out in the Euler launch
        W_out_ = load_f32(ck, "aex.ad_l2W", {A_, Hd_});
        b_out_ = load_f32(ck, "aex.ad_l2b", {A_});
        W3_ = load_f32(ck, "aex.ae_W3", {W_, W_});
        b3_ = load_f32(ck, "aex.ae_b3", {W_});
        const int Sa = S_ - n_lead_;
        const CkptTensor& pe = ck.info("aex.pos_embd");
        if (pe.shape.size() != 2 || pe.shape[1] != W_ || pe.shape[0] < Sa) throw std::runtime_error("vla: aex.pos_embd does not cover the action horizon");
        std::vector<float> pos = ck.f32("aex.pos_embd");
        pos.resize((size_t)Sa * W_);  // rows [0, horizon) (action_expert.cpp:50)
        pos_.upload(pos.data(), pos.size() * sizeof(float));
        po2W_ = load_w(ck, "aex.po2W", dt_, {O_, W_});
        po2b_ = load_f32(ck, "aex.po2b", {O_});
        ad1W_ = load_w(ck, "aex.ad_l1W", dt_, {Hd_, O_});
        ad1b_ = load_f32(ck, "aex.ad_l1b", {Hd_});
    } else {
        W_in_ = load_f32(ck, "act.W_in", {W_, A_});
        W_out_ = load_f32(ck, "act.W_out", {A_, W_});
        b_out_ = load_f32(ck, "act.b_out", {A_});
    }
    if (arch_ != Arch::GR00T && !adarms_) final_norm_ = load_w(ck, "act.norm", dt_, {W_});

    const bool no_norm_fusion = std::getenv("VLA_NO_NORM_FUSION") != nullptr;  // read once, at load
    fuse_final_norm_ = !no_norm_fusion;
    fuse_self_block_ = !no_norm_fusion && std::getenv("VLA_NO_FUSED_SELF_BLOCK") == nullptr;
    hand_row_stats_ = !no_norm_fusion && std::getenv("VLA_NO_ROW_STATS") == nullptr;
    layers_.resize(L_);
    for (int l = 0; l < L_; ++l) {
        LayerW& w = layers_[l];
        const std::string p = "ex." + std::to_string(l) + ".";
        // SmolVLA: self iff l % every == 0 (src/models/smolvla.cpp:1182); GR00T N1.5:
        // cross on even, self on odd layers (src/models/gr00tn1d5.cpp:361-375).
        w.is_self = arch_ == Arch::PI0 ? true : arch_ == Arch::SMOLVLA ? (l % every == 0) : (interleave && l % 2 == 1);
        w.needs_prefix = !(arch_ == Arch::GR00T && w.is_self);
        w.from_text = alt_vl_ && w.needs_prefix && l % (2 * text_every_) == 0;
        const int64_t n_proj = w.is_self ? qd + 2 * kvd : qd;
        if (arch_ != Arch::GR00T && !adarms_) w.ln = load_w(ck, p + "ln", dt_, {W_});
        w.Wqkv = load_w(ck, p + (w.is_self ? "Wqkv" : "Wq"), dt_, {n_proj, W_});
        if (arch_ != Arch::GR00T && !adarms_ && dt_ == VLA_DT_BF16 && W_ % 16 == 0 && !no_norm_fusion)
            w.Wqkv_ln = load_folded_bf16(ck, p + (w.is_self ? "Wqkv" : "Wq"), p + "ln", n_proj, W_);
        if (ck.has(p + (w.is_self ? "bqkv" : "bq"))) w.bqkv = load_f32(ck, p + (w.is_self ? "bqkv" : "bq"), {n_proj});
        w.Wo = load_w(ck, p + "Wo", dt_, {W_, qd});
        if (ck.has(p + "bo")) w.bo = load_f32(ck, p + "bo", {W_});
        if (I_ > 0 && arch_ == Arch::GR00T) {
            w.W1 = load_w(ck, p + "W1", dt_, {I_, W_});
            w.b1 = load_f32(ck, p + "b1", {I_});
            w.W2 = load_w(ck, p + "W2", dt_, {W_, I_});
            w.b2 = load_f32(ck, p + "b2", {W_});
        } else if (I_ > 0) {
            if (!adarms_) w.ln2 = load_w(ck, p + "ln2", dt_, {W_});
            w.Wgu = load_w(ck, p + "Wgu", dt_, {2 * (int64_t)I_, W_});
            w.Wd = load_w(ck, p + "Wd", dt_, {W_, I_});
            if (!adarms_ && dt_ == VLA_DT_BF16 && W_ % 16 == 0 && !no_norm_fusion)
                w.Wgu_ln = load_folded_bf16(ck, p + "Wgu", p + "ln2", 2 * (int64_t)I_, W_);
        }
        if (w.needs_prefix) {
            const std::string v = "vlm." + std::to_string(l) + ".";
            if (arch_ != Arch::GR00T) w.vlm_ln = load_w(ck, v + "ln", dt_, {Wv_});
            w.Wkv_pre = load_w(ck, v + "Wkv", dt_, {2 * kvd, Wv_});
            if (ck.has(v + "bkv")) w.bkv_pre = load_f32(ck, v + "bkv", {2 * kvd});
        }
        if (arch_ == Arch::SMOLVLA && !w.is_self) {
            w.Wk_x = load_w(ck, p + "Wk_x", dt_, {kvd, kvd});
            w.Wv_x = load_w(ck, p + "Wv_x", dt_, {kvd, kvd});
        }
    }

    // Per-step constants.  The time conditioning depends on the step index only,
    // so it is evaluated once here instead of inside every denoise step.
    std::vector<float> bias((size_t)steps_ * W_);
    time_mlp_ = arch_ != Arch::GR00T && !adarms_ && ck.has("act.W_at1");
    if (head_io_) {
        // encode_action (action_expert.cpp:46-52): a = W1 x + b1; m = silu(W2 [a ; tau] + b2);
        // out = W3 m + b3 + pos.  W2 = [W2a | W2t] by columns, tau depends on the step only, so
        // m = silu((W2a W1) x + (W2a b1 + W2t tau_s + b2)): one [W][A] matrix and a per-step bias.
        const std::vector<float> W1 = host_f32(ck, "aex.ae_W1", {W_, A_}), b1 = host_f32(ck, "aex.ae_b1", {W_}),
                                 W2 = host_f32(ck, "aex.ae_W2", {W_, 2 * (int64_t)W_}), b2 = host_f32(ck, "aex.ae_b2", {W_});
        std::vector<float> Wf((size_t)W_ * A_);
        for (int r = 0; r < W_; ++r)
            for (int a = 0; a < A_; ++a) {
                double acc = 0.0;
                for (int k = 0; k < W_; ++k) acc += (double)W2[(size_t)r * 2 * W_ + k] * (double)W1[(size_t)k * A_ + a];
                Wf[(size_t)r * A_ + a] = (float)acc;
            }
        W_in_.upload(Wf.data(), Wf.size() * sizeof(float));
        const int64_t n_buckets = ck.i64("num_buckets", 1000);
        for (int s = 0; s < steps_; ++s) {
            // action_sinusoid(bucket, E, ...): sin first, then cos, the same row for every token (embed.h:47-59)
            const int64_t bucket = (int64_t)((double)s / (double)steps_ * (double)n_buckets);
            const int half = W_ / 2;
            const float stp = std::log(10000.0f) / (float)half, tb = (float)bucket;
            std::vector<float> tau(W_, 0.f);
            for (int i = 0; i < half; ++i) {
                const float e = tb * std::exp(-(float)i * stp);
                tau[i] = std::sin(e);
                tau[half + i] = std::cos(e);
            }
            for (int r = 0; r < W_; ++r) {
                double acc = (double)b2[r];
                for (int k = 0; k < W_; ++k)
                    acc += (double)W2[(size_t)r * 2 * W_ + k] * (double)b1[k] + (double)W2[(size_t)r * 2 * W_ + W_ + k] * (double)tau[k];
                bias[(size_t)s * W_ + r] = (float)acc;
            }
        }
    } else if (time_mlp_) {
        const std::vector<float> b_in = host_f32(ck, "act.b_in", {W_});
        // Action-time MLP (src/models/smolvla.cpp:1397-1403, src/models/pi0.cpp:240-244):
        //   mlp1 = W_at1 . concat(W_in x + b_in, time_s) + b_at1,  suffix = W_at2 silu(mlp1) + b_at2.
        // W_at1 = [Wa | Wt] by columns, so mlp1 = (Wa W_in) x + (Wa b_in + Wt time_s + b_at1):
        // the first two projections collapse into one [W][A] matrix and a per-step bias,
        // both formed here once (double accumulation), and the embed kernel applies the silu.
        const std::vector<float> W_in = ck.f32("act.W_in"), W_at1 = host_f32(ck, "act.W_at1", {W_, 2 * (int64_t)W_}),
                                 b_at1 = host_f32(ck, "act.b_at1", {W_});
        std::vector<float> Wf((size_t)W_ * A_);
        for (int r = 0; r < W_; ++r)
            for (int a = 0; a < A_; ++a) {
                double acc = 0.0;
                for (int k = 0; k < W_; ++k) acc += (double)W_at1[(size_t)r * 2 * W_ + k] * (double)W_in[(size_t)k * A_ + a];
                Wf[(size_t)r * A_ + a] = (float)acc;
            }
        W_in_.upload(Wf.data(), Wf.size() * sizeof(float));
        for (int s = 0; s < steps_; ++s) {
            const float t = 1.0f + (float)s * dt_step_;
            const std::vector<float> te = sinusoidal_time_emb(t, W_, cfg.min_period, cfg.max_period);
            for (int r = 0; r < W_; ++r) {
                double acc = (double)b_at1[r];
                for (int k = 0; k < W_; ++k)
                    acc += (double)W_at1[(size_t)r * 2 * W_ + k] * (double)b_in[k] +
                           (double)W_at1[(size_t)r * 2 * W_ + W_ + k] * (double)te[k];
                bias[(size_t)s * W_ + r] = (float)acc;
            }
        }
        W_at2_ = load_f32(ck, "act.W_at2", {W_, W_});
        b_at2_ = load_f32(ck, "act.b_at2", {W_});
    } else {
        const std::vector<float> b_in = host_f32(ck, "act.b_in", {W_});
        for (int s = 0; s < steps_; ++s) {
            for (int c = 0; c < W_; ++c) bias[(size_t)s * W_ + c] = b_in[c];
            if (arch_ != Arch::GR00T && !adarms_) {
                // t = 1 + step*dt (src/models/pi0.cpp:654-656), embedding of src/layers/embed.h:61-73
                const float t = 1.0f + (float)s * dt_step_;
                const std::vector<float> te = sinusoidal_time_emb(t, W_, cfg.min_period, cfg.max_period);
                for (int c = 0; c < W_; ++c) bias[(size_t)s * W_ + c] += te[c];
            }
        }
    }
    bias_step_.upload(bias.data(), bias.size() * sizeof(float));

    if (adarms_) {
        // cond_s = silu(W_tout silu(W_tin time_s + b_tin) + b_tout) (src/models/pi05.cpp:619-620);
        // (scale, shift, gate) of a norm site = dense_w . cond + dense_b (build_adarms,
        // pi05.cpp:212-215).  Sites per step: 2 per layer (attention, FFN), then the final norm.
        const std::vector<float> Wt1 = host_f32(ck, "te.W_tin", {W_, W_}), bt1 = host_f32(ck, "te.b_tin", {W_}),
                                 Wt2 = host_f32(ck, "te.W_tout", {W_, W_}), bt2 = host_f32(ck, "te.b_tout", {W_});
        const int sites = 2 * L_ + 1;
        std::vector<std::vector<float>> dw(sites), db(sites);
        for (int l = 0; l < L_; ++l) {
            const std::string p = "ex." + std::to_string(l) + ".";
            dw[2 * l] = host_f32(ck, p + "ada_in_w", {3 * (int64_t)W_, W_});
            db[2 * l] = host_f32(ck, p + "ada_in_b", {3 * (int64_t)W_});
            if (I_ > 0) {
                dw[2 * l + 1] = host_f32(ck, p + "ada_post_w", {3 * (int64_t)W_, W_});
                db[2 * l + 1] = host_f32(ck, p + "ada_post_b", {3 * (int64_t)W_});
            }
        }
        dw[2 * L_] = host_f32(ck, "act.ada_final_w", {3 * (int64_t)W_, W_});
        db[2 * L_] = host_f32(ck, "act.ada_final_b", {3 * (int64_t)W_});
        std::vector<float> mod((size_t)steps_ * sites * 3 * W_);
        std::vector<float> c1(W_), cond(W_);
        for (int s = 0; s < steps_; ++s) {
            const float t = 1.0f + (float)s * dt_step_;
            const std::vector<float> te = sinusoidal_time_emb(t, W_, cfg.min_period, cfg.max_period);
            host_linear(Wt1.data(), bt1.data(), te.data(), c1.data(), W_, W_);
            for (auto& v : c1) v = host_silu(v);
            host_linear(Wt2.data(), bt2.data(), c1.data(), cond.data(), W_, W_);
            for (auto& v : cond) v = host_silu(v);
            for (int k = 0; k < sites; ++k)
                if (!dw[k].empty()) host_linear(dw[k].data(), db[k].data(), cond.data(), mod.data() + ((size_t)s * sites + k) * 3 * W_, 3 * W_, W_);
        }
        ada_.upload(mod.data(), mod.size() * sizeof(float));
    }

    if (arch_ == Arch::GR00T) {
        // temb = l2(silu(l1(timesteps_proj(bucket)))) (DitHead::time_emb,
        // src/modules/dit_head.cpp:135-137); per layer (scale, shift) =
        // adaln_w . silu(temb) + adaln_b (src/layers/norm.h:39-41).
        const std::vector<float> l1W = host_f32(ck, "te.l1W", {W_, 256}), l1b = host_f32(ck, "te.l1b", {W_}),
                                 l2W = host_f32(ck, "te.l2W", {W_, W_}), l2b = host_f32(ck, "te.l2b", {W_});
        // per step: L layer slots (scale, shift), slot L = zeros (a plain LayerNorm), slot L + 1 =
        // the output modulation of DitHead::proj_out when the head's own MLPs are present
        std::vector<float> ada((size_t)steps_ * (L_ + 2) * 2 * W_, 0.f);
        std::vector<std::vector<float>> aw(L_), ab(L_);
        for (int l = 0; l < L_; ++l) {
            aw[l] = host_f32(ck, "ex." + std::to_string(l) + ".adaln_w", {2 * (int64_t)W_, W_});
            ab[l] = host_f32(ck, "ex." + std::to_string(l) + ".adaln_b", {2 * (int64_t)W_});
        }
        std::vector<float> po1W, po1b;
        if (head_io_) {
            po1W = host_f32(ck, "aex.po1W", {2 * (int64_t)W_, W_});
            po1b = host_f32(ck, "aex.po1b", {2 * (int64_t)W_});
        }
        const int64_t n_buckets = ck.i64("num_buckets", 1000);
        for (int s = 0; s < steps_; ++s) {
            std::vector<float> tp, t1(W_), temb(W_), st(W_);
            timesteps_proj((int64_t)((double)s / (double)steps_ * (double)n_buckets), tp);
            host_linear(l1W.data(), l1b.data(), tp.data(), t1.data(), W_, 256);
            for (auto& v : t1) v = host_silu(v);
            host_linear(l2W.data(), l2b.data(), t1.data(), temb.data(), W_, W_);
            for (int c = 0; c < W_; ++c) st[c] = host_silu(temb[c]);
            const int nthr = std::min(default_cpu_threads(), L_);
            std::vector<std::thread> pool;
            for (int t = 0; t < nthr; ++t)
                pool.emplace_back([&, t]() {
                    for (int l = t; l < L_; l += nthr)
                        host_linear(aw[l].data(), ab[l].data(), st.data(),
                                    ada.data() + ((size_t)s * (L_ + 2) + l) * 2 * W_, 2 * W_, W_);
                });
            for (auto& th : pool) th.join();
            if (head_io_) {
                // proj_out's dense gives (shift, scale) in that order (dit_head.cpp:140-142, norm.h:36);
                // the norm launch takes (scale, shift)
                std::vector<float> po(2 * (size_t)W_);
                host_linear(po1W.data(), po1b.data(), st.data(), po.data(), 2 * W_, W_);
                float* slot = ada.data() + ((size_t)s * (L_ + 2) + L_ + 1) * 2 * W_;
                std::copy(po.begin() + W_, po.end(), slot);
                std::copy(po.begin(), po.begin() + W_, slot + W_);
            }
        }
        ada_.upload(ada.data(), ada.size() * sizeof(float));

        // The folded operands cost a copy of every Q / QKV weight per denoise step (GR00T N1.5 at 4 steps:
        // 16 layers x (3 W^2 self, W^2 cross) x 2 bytes = 0.6 GB) and the step count comes from the file:
        // above the budget (VLA_ADALN_FOLD_MB, default 2048) the blocks keep adaln + projection as two launches.
        size_t fold_bytes = 0;
        for (int l = 0; l < L_; ++l) fold_bytes += (size_t)steps_ * (size_t)(layers_[l].is_self ? qd + 2 * kvd : qd) * W_ * sizeof(uint16_t);
        const char* fold_mb = std::getenv("VLA_ADALN_FOLD_MB");
        const size_t fold_budget = (size_t)(fold_mb ? std::max(0L, std::atol(fold_mb)) : 2048L) << 20;
        if (fold_bytes > fold_budget)
            std::fprintf(stderr, "vla(gr00t): %d steps of folded adaLN operands would take %zu MB (budget %zu MB); using adaln + projection launches\n",
                         steps_, fold_bytes >> 20, fold_budget >> 20);
        if (dt_ == VLA_DT_BF16 && W_ % 16 == 0 && !no_norm_fusion && fold_bytes <= fold_budget) {
            // the modulation of a block depends on the step only: fold it into one operand set
            // per step, and the pre-norm launch of the block disappears into its projection
            const int nthr = std::min(default_cpu_threads(), L_);
            std::vector<std::thread> pool;
            std::vector<std::string> errors(nthr);
            std::vector<std::vector<uint16_t>> folded(L_);
            std::vector<std::vector<float>> cs(L_), bs(L_);
            for (int t = 0; t < nthr; ++t)
                pool.emplace_back([&, t]() {
                    try {
                        for (int l = t; l < L_; l += nthr) {
                            LayerW& w = layers_[l];
                            const std::string p = "ex." + std::to_string(l) + ".";
                            const int64_t n_proj = w.is_self ? qd + 2 * kvd : qd;
                            const std::vector<float> wf = host_f32(ck, p + (w.is_self ? "Wqkv" : "Wq"), {n_proj, W_});
                            std::vector<float> bf;
                            if (ck.has(p + (w.is_self ? "bqkv" : "bq"))) bf = host_f32(ck, p + (w.is_self ? "bqkv" : "bq"), {n_proj});
                            std::vector<uint16_t> wb(wf.size());
                            for (size_t i = 0; i < wf.size(); ++i) wb[i] = f32_to_bf16(wf[i]);
                            folded[l].resize((size_t)steps_ * wf.size());
                            cs[l].resize((size_t)steps_ * n_proj);
                            bs[l].resize((size_t)steps_ * n_proj);
                            for (int s = 0; s < steps_; ++s) {
                                const float* sc = ada.data() + ((size_t)s * (L_ + 2) + l) * 2 * W_;
                                VLA_K(vla_fold_adaln_weight_host(wb.data(), bf.empty() ? nullptr : bf.data(), sc, sc + W_, (int)n_proj, W_,
                                                                 folded[l].data() + (size_t)s * wf.size(), cs[l].data() + (size_t)s * n_proj,
                                                                 bs[l].data() + (size_t)s * n_proj));
                            }
                        }
                    } catch (const std::exception& e) {
                        errors[t] = e.what();
                    }
                });
            for (auto& th : pool) th.join();
            for (const std::string& e : errors)
                if (!e.empty()) throw std::runtime_error(e);
            for (int l = 0; l < L_; ++l) {  // device work stays on the loading thread
                layers_[l].Wqkv_ada.upload(folded[l].data(), folded[l].size() * sizeof(uint16_t));
                layers_[l].cs_ada.upload(cs[l].data(), cs[l].size() * sizeof(float));
                layers_[l].b_ada.upload(bs[l].data(), bs[l].size() * sizeof(float));
                std::vector<uint16_t>().swap(folded[l]);
            }
        }
    }
}

void FlowExpert::allocate(int B, int P, int P_txt) {
    // the attention workspace is planned under the kernel library's tuning overrides: plan again when they were reloaded
    const int tuning_gen = vla_kernels_tuning_generation();
    if (B == B_ && P == P_ && P_txt == P_txt_ && tuning_gen == tuning_gen_) return;
    tuning_gen_ = tuning_gen;
    B_ = B;
    P_ = P;
    P_txt_ = P_txt;
    ++alloc_gen_;
    const size_t es = dtype_size(dt_);
    attn_ws_.reset();
    for (LayerW& w : layers_) {
        // alternating layers: text rows, or image rows (all rows when there is no text:
        // vl_txt = vl_img then, gr00tn1d6.cpp:443)
        const int prefix = !w.needs_prefix ? 0 : !alt_vl_ ? P : (w.from_text && P_txt > 0) ? P_txt : P - P_txt;
        const int tmax = round_up(prefix + (w.is_self ? S_ : 0), 64);
        w.kv.create(dt_, B, Hkv_, D_, tmax);
        w.kv.n_prefix = prefix;
        attn_ws_.plan(dt_, B, S_, Hq_, Hkv_, D_, prefix + (w.is_self ? S_ : 0));
    }
    attn_ws_.commit();
    if (arch_ == Arch::SMOLVLA) {
        tmp_kv_.create(dt_, B, Hkv_, D_, round_up(P, 64));
        tmpk_.alloc((size_t)B * P * Hkv_ * D_ * es);
        tmpv_.alloc((size_t)B * P * Hkv_ * D_ * es);
    }
    prefix_.alloc((size_t)B * P * Wv_ * es);
    prefix_n_.alloc((size_t)B * P * Wv_ * es);
    lead_.alloc((size_t)B * std::max(n_lead_, 1) * W_ * sizeof(float));
    x0_.alloc((size_t)B * (S_ - n_lead_) * A_ * sizeof(float));
    xt_.alloc((size_t)B * (S_ - n_lead_) * A_ * sizeof(float));
    h_.alloc((size_t)B * S_ * W_ * es);
    hn_.alloc((size_t)B * S_ * W_ * es);
    q_.alloc((size_t)B * S_ * Hq_ * D_ * es);
    att_.alloc((size_t)B * S_ * Hq_ * D_ * es);
    row_stats_.alloc((size_t)B * S_ * ((W_ + 63) / 64) * 2 * sizeof(float));
    if (I_ > 0) mid_.alloc((size_t)B * S_ * I_ * es);
    if (time_mlp_ || head_io_) m1_.alloc((size_t)B * S_ * W_ * sizeof(float));
    if (head_io_) {
        m2_.alloc((size_t)B * S_ * W_ * sizeof(float));
        d1_.alloc((size_t)B * S_ * O_ * es);
        d2_.alloc((size_t)B * S_ * Hd_ * es);
    }
}

void FlowExpert::prefill(const Inputs* in, int batch) {
    if (!in || batch <= 0) throw std::invalid_argument("vla: prefill needs at least one observation");
    const int views = in[0].n_img_views, n_lang = (arch_ == Arch::GR00T && !alt_vl_) ? 0 : in[0].n_lang;
    if (views < 1 || views > max_views_) throw std::invalid_argument("vla: n_img_views out of range");
    if (n_lang < 0 || n_lang > n_lang_max_) throw std::invalid_argument("vla: n_lang out of range");
    for (int b = 0; b < batch; ++b) {
        if (!in[b].precomputed_img_emb) throw std::invalid_argument("vla: precomputed_img_emb is required");
        if (in[b].n_img_views != views || ((arch_ != Arch::GR00T || alt_vl_) && in[b].n_lang != n_lang))
            throw std::invalid_argument("vla: a batch shares one n_img_views and one n_lang");
        if (n_lang > 0 && !in[b].lang_tokens) throw std::invalid_argument("vla: lang_tokens missing");
        for (int i = 0; i < n_lang; ++i)
            if (in[b].lang_tokens[i] < 0 || in[b].lang_tokens[i] >= vocab_)
                throw std::invalid_argument("vla: language token outside the vocabulary");
    }
    const int n_img_tot = views * n_img_;
    // SmolVLA pads the language block to its capacity and appends a state token
    // (src/models/smolvla.cpp:1608-1612); pi0 uses the real length (pi0.cpp:526-528).
    const int P = arch_ == Arch::SMOLVLA ? n_img_tot + n_lang_max_ + 1
                  : arch_ == Arch::PI0   ? n_img_tot + n_lang
                  : alt_vl_              ? n_img_tot + n_lang
                                         : n_img_tot;
    allocate(batch, P, alt_vl_ ? n_lang : 0);
    const int B = batch;
    Ctx C;  // prefill runs on the default stream and is synchronous

    // ---- prefix embeddings: scaled and converted to the model's dtype straight from the
    // callers' buffers into page-locked staging memory by a few threads, an observation per
    // task, and sent to the device in groups while the next group is being converted (the
    // copies are asynchronous; everything below runs on the same stream, after them)
    const size_t es = dtype_size(dt_);
    stage_.reserve((size_t)B * P * Wv_ * es);
    char* const pe = stage_.as<char>();
    const float lang_scale = std::sqrt((float)Wv_);
    const float img_scale = arch_ == Arch::SMOLVLA ? lang_scale : 1.0f;  // smolvla.cpp:1363 vs pi0.cpp:554-555
    std::vector<float> lead_host((size_t)B * std::max(n_lead_, 0) * W_);  // the state (and future) rows in front of the actions
    auto stage_obs = [&](int b) {
        char* dst = pe + (size_t)b * P * Wv_ * es;
        // alternating layers project the image rows and the text rows separately: all image
        // rows of the batch first, then all text rows, each block [B][rows][Wv]
        char* txt_dst = dst + (size_t)n_img_tot * Wv_ * es;
        if (alt_vl_) {
            dst = pe + (size_t)b * n_img_tot * Wv_ * es;
            txt_dst = pe + ((size_t)B * n_img_tot + (size_t)b * n_lang) * Wv_ * es;
        }
        convert_scaled(dst, in[b].precomputed_img_emb, (size_t)n_img_tot * Wv_, img_scale, dt_);
        if (arch_ != Arch::GR00T || alt_vl_) {
            const int rows = arch_ == Arch::SMOLVLA ? n_lang_max_ : n_lang;
            const float ls = alt_vl_ ? 1.0f : lang_scale;  // N1.6: the rows stand for backbone features, unscaled
            std::vector<float> fetched;
            if (lang_rows_) {  // the rows this observation needs, read from the file
                std::vector<int32_t> ids((size_t)rows, 0);
                for (int i = 0; i < n_lang; ++i) ids[i] = in[b].lang_tokens[i];
                fetched.resize((size_t)rows * Wv_);
                if (rows > 0 && !lang_rows_->fetch_locked(ids, fetched.data())) throw std::runtime_error("vla: cannot read token embedding rows");
            }
            for (int i = 0; i < rows; ++i) {
                const int tok = i < n_lang ? in[b].lang_tokens[i] : 0;  // zero-padded ids, smolvla.cpp:1628-1629
                const float* e = lang_rows_ ? fetched.data() + (size_t)i * Wv_ : E_lang_.data() + (size_t)tok * Wv_;
                convert_scaled(txt_dst + (size_t)i * Wv_ * es, e, (size_t)Wv_, ls, dt_);
            }
        }
        std::vector<float> st(max_state_, 0.f);
        if (in[b].state) std::copy(in[b].state, in[b].state + max_state_, st.begin());
        if (arch_ == Arch::SMOLVLA) {
            std::vector<float> row(Wv_);
            host_linear(Wstate_.data(), bstate_.data(), st.data(), row.data(), Wv_, max_state_);
            convert_scaled(dst + (size_t)(P - 1) * Wv_ * es, row.data(), (size_t)Wv_, 1.0f, dt_);
        } else if (head_io_) {
            // encode_state (relu between the two projections), then the learned future tokens
            std::vector<float> h1(Hs_), ld((size_t)n_lead_ * W_);
            host_linear(se_l1W_.data(), se_l1b_.data(), st.data(), h1.data(), Hs_, max_state_);
            for (float& v : h1) v = v > 0.f ? v : 0.f;
            host_linear(se_l2W_.data(), se_l2b_.data(), h1.data(), ld.data(), W_, Hs_);
            std::copy(future_.begin(), future_.end(), ld.begin() + W_);
            std::copy(ld.begin(), ld.end(), lead_host.begin() + (size_t)b * n_lead_ * W_);
        } else if (n_lead_ > 0) {
            host_linear(W_sp_.data(), b_sp_.data(), st.data(), lead_host.data() + (size_t)b * W_, W_, max_state_);
        }
    };
    {
        const int nthr = std::max(1, std::min(default_cpu_threads(), B));
        const int n_groups = alt_vl_ ? 1 : std::min(B, 4);  // the alternating layout interleaves observations: one copy at the end
        for (int gi = 0; gi < n_groups; ++gi) {
            const int b0 = (int)((long)B * gi / n_groups), b1 = (int)((long)B * (gi + 1) / n_groups);
            if (nthr == 1 || b1 - b0 == 1) {
                for (int b = b0; b < b1; ++b) stage_obs(b);
            } else {
                std::vector<std::thread> pool;
                std::vector<std::string> errors(nthr);
                for (int t = 0; t < nthr; ++t)
                    pool.emplace_back([&, t]() {
                        try {
                            for (int b = b0 + t; b < b1; b += nthr) stage_obs(b);
                        } catch (const std::exception& e) {
                            errors[t] = e.what();
                        }
                    });
                for (auto& th : pool) th.join();
                for (const std::string& e : errors)
                    if (!e.empty()) throw std::runtime_error(e);
            }
            const size_t off = alt_vl_ ? 0 : (size_t)b0 * P * Wv_ * es;
            const size_t len = alt_vl_ ? (size_t)B * P * Wv_ * es : (size_t)(b1 - b0) * P * Wv_ * es;
            VLA_HIP(hipMemcpyAsync((char*)prefix_.get() + off, pe + off, len, hipMemcpyHostToDevice, C.stream));
        }
        if (!lead_host.empty()) VLA_HIP(hipMemcpy(lead_.get(), lead_host.data(), lead_host.size() * sizeof(float), hipMemcpyHostToDevice));
    }

    // ---- positions and masks (smolvla.cpp:1633-1672, pi0.cpp:612-616)
    pad_start_ = pad_end_ = 0;
    if (rope_) {
        const RopeSpec rs{D_, cfg.rope_freq_base};
        std::vector<int32_t> pp(P), ps(S_), pc(S_);
        for (int i = 0; i < P; ++i) pp[i] = i;
        int suffix_base = P;
        if (arch_ == Arch::SMOLVLA) {
            const int state_pos = n_img_tot + n_lang;
            pp[P - 1] = state_pos;
            suffix_base = state_pos + 1;
            pad_start_ = n_img_tot + n_lang;
            pad_end_ = n_img_tot + n_lang_max_;
        }
        for (int i = 0; i < S_; ++i) {
            ps[i] = suffix_base + i;
            pc[i] = i;
        }
        rope_prefill_.build(rs, pp);
        rope_self_.build(rs, ps);
        rope_cross_.build(rs, pc);
    }

    // ---- vlln: the affine LayerNorm between the backbone and the DiT head
    // (src/models/gr00tn1d6.cpp:436), in place on every prefix row
    if (vlln_sc_) VLA_K(vla_adaln(prefix_.get(), vlln_sc_.as<float>(), vlln_sh_.as<float>(), prefix_.get(), dt_, B * P, Wv_, vlln_eps_, C.stream));

    // ---- prefix K/V of every layer, once per observation
    Tensor xp = tensor_2d(prefix_.get(), dt_, Wv_, (int64_t)B * P);
    Tensor xn = tensor_2d(prefix_n_.get(), dt_, Wv_, (int64_t)B * P);
    const int kvd = Hkv_ * D_;
    prof_start("prefill", C.stream);
    for (LayerW& w : layers_) {
        if (!w.needs_prefix) continue;
        Tensor Wkv = tensor_2d(w.Wkv_pre.get(), dt_, Wv_, 2 * kvd);
        const float* bkv = w.bkv_pre ? w.bkv_pre.as<float>() : nullptr;
        if (alt_vl_) {
            const bool txt = w.from_text && P_txt_ > 0;
            const int rows = txt ? P_txt_ : P - P_txt_;
            const char* base = (const char*)prefix_.get() + (txt ? (size_t)B * (P - P_txt_) * Wv_ * dtype_size(dt_) : 0);
            Tensor xs = tensor_2d(const_cast<char*>(base), dt_, Wv_, (int64_t)B * rows);
            qkv_rope_append(C, xs, Wkv, bkv, rows, 0, true, true, nullptr, nullptr, w.kv, 0);
            prof_mark("prefix_kv_proj");
            continue;
        }
        if (arch_ == Arch::GR00T) {
            qkv_rope_append(C, xp, Wkv, bkv, P, 0, true, true, nullptr, nullptr, w.kv, 0);
            prof_mark("prefix_kv_proj");
            continue;
        }
        rms_norm(C, xp, w.vlm_ln.get(), eps_, xn);
        prof_mark("prefix_norm");
        if (arch_ == Arch::SMOLVLA && !w.is_self) {
            // expert_cross_kv: K = Wk_x . cachedK_flat, V = Wv_x . cachedV_flat, no second rotation
            qkv_rope_append(C, xn, Wkv, bkv, P, 0, true, true, &rope_prefill_, nullptr, tmp_kv_, 0);
            VLA_K(vla_kv_gather(tmp_kv_.k.get(), tmp_kv_.vt.get(), tmpk_.get(), tmpv_.get(), dt_, B, Hkv_, D_,
                                tmp_kv_.t_max, 0, P, C.stream));
            Tensor tk = tensor_2d(tmpk_.get(), dt_, kvd, (int64_t)B * P), tv = tensor_2d(tmpv_.get(), dt_, kvd, (int64_t)B * P);
            Tensor Wkx = tensor_2d(w.Wk_x.get(), dt_, kvd, kvd), Wvx = tensor_2d(w.Wv_x.get(), dt_, kvd, kvd);
            qkv_rope_append(C, tk, Wkx, nullptr, P, 0, true, false, nullptr, nullptr, w.kv, 0);
            qkv_rope_append(C, tv, Wvx, nullptr, P, 0, false, true, nullptr, nullptr, w.kv, 0);
            prof_mark("prefix_kv_proj_and_cross_reprojection");
        } else {
            qkv_rope_append(C, xn, Wkv, bkv, P, 0, true, true, &rope_prefill_, nullptr, w.kv, 0);
            prof_mark("prefix_kv_proj");
        }
    }

    // ---- initial noise
    const size_t nx = (size_t)(S_ - n_lead_) * A_;
    std::vector<float> x0((size_t)B * nx);
    for (int b = 0; b < B; ++b) {
        if (in[b].noise) {
            std::copy(in[b].noise, in[b].noise + nx, x0.begin() + (size_t)b * nx);
        } else {
            std::normal_distribution<float> nd(0.f, 1.f);
            for (size_t i = 0; i < nx; ++i) x0[(size_t)b * nx + i] = nd(rng_);
        }
    }
    x0_.upload(x0.data(), x0.size() * sizeof(float));
    VLA_HIP(hipDeviceSynchronize());
}

void FlowExpert::run_steps(int n_steps, void* stream) {
    if (B_ == 0) throw std::logic_error("vla: denoise before prefill");
    Ctx C;
    C.stream = (hipStream_t)stream;
    last_stream_ = C.stream;
    const int B = B_, M = B * S_;
    const float scale = 1.0f / std::sqrt((float)D_);
    Tensor h = tensor_2d(h_.get(), dt_, W_, M), hn = tensor_2d(hn_.get(), dt_, W_, M);
    Tensor att = tensor_2d(att_.get(), dt_, (int64_t)Hq_ * D_, M);
    Tensor Q;
    Q.data = q_.get();
    Q.dtype = dt_;
    Q.ne[0] = D_; Q.ne[1] = Hq_; Q.ne[2] = S_; Q.ne[3] = B;
    const size_t xbytes = (size_t)B * (S_ - n_lead_) * A_ * sizeof(float);
    prof_start("step", C.stream);
    for (int it = 0; it < n_steps; ++it) {
        const int s = it % steps_;
        if (s == 0) {
            attn_ws_.begin(C.stream);
            VLA_HIP(hipMemcpyAsync(xt_.get(), x0_.get(), xbytes, hipMemcpyDeviceToDevice, C.stream));
            prof_mark("stage_noise");
        }
        {
            if (head_io_) {
                VLA_K(vla_embed_suffix_act(xt_.as<float>(), W_in_.as<float>(), bias_step_.as<float>() + (size_t)s * W_,
                                           lead_.as<float>(), m1_.get(), VLA_DT_F32, B, S_, n_lead_, A_, W_, VLA_ACT_SILU, C.stream));
                VLA_K(vla_linear(m1_.get(), W3_.get(), b3_.as<float>(), nullptr, m2_.get(), VLA_DT_F32, VLA_DT_F32, M, W_, W_,
                                 C.stream));
                VLA_K(vla_finish_suffix_rows(m2_.as<float>(), pos_.as<float>(), lead_.as<float>(), h.data, dt_, B, S_, n_lead_, W_,
                                             C.stream));
            } else if (time_mlp_) {
                VLA_K(vla_embed_suffix_act(xt_.as<float>(), W_in_.as<float>(), bias_step_.as<float>() + (size_t)s * W_,
                                           n_lead_ ? lead_.as<float>() : nullptr, m1_.get(), VLA_DT_F32, B, S_, n_lead_, A_, W_,
                                           VLA_ACT_SILU, C.stream));
                VLA_K(vla_linear(m1_.get(), W_at2_.get(), b_at2_.as<float>(), nullptr, h.data, VLA_DT_F32, dt_, M, W_, W_,
                                 C.stream));
                if (n_lead_) VLA_K(vla_set_lead_rows(lead_.as<float>(), h.data, dt_, B, S_, n_lead_, W_, C.stream));
            } else {
                VLA_K(vla_embed_suffix(xt_.as<float>(), W_in_.as<float>(), bias_step_.as<float>() + (size_t)s * W_,
                                       n_lead_ ? lead_.as<float>() : nullptr, h.data, dt_, B, S_, n_lead_, A_, W_, C.stream));
            }
            prof_mark("embed_suffix");
            // A block's output projection leaves the row sums of the h it writes for the LayerNorm the next block takes
            // inside its projection launch (GR00T without the FFN half, from batch 32 on, where those launches are the tiled ones).
            const bool stats_path = hand_row_stats_ && arch_ == Arch::GR00T && dt_ == VLA_DT_BF16 && I_ == 0 && B >= 32 &&
                                    W_ % 64 == 0 && W_ / 64 <= 24 && (Hq_ * D_) % 8 == 0;
            bool stats_valid = false;  // row_stats_ describes the current h
            for (int l = 0; l < L_; ++l) {
                LayerW& w = layers_[l];
                const float* h_stats = stats_valid ? row_stats_.as<float>() : nullptr;
                const bool leave_stats = stats_path && l + 1 < L_ && (bool)layers_[l + 1].Wqkv_ada;
                const float* bq = w.bqkv ? w.bqkv.as<float>() : nullptr;
                const int64_t n_rows_w = w.is_self ? (int64_t)(Hq_ + 2 * Hkv_) * D_ : (int64_t)Hq_ * D_;
                const RopeTable* tab = rope_ ? (w.is_self ? &rope_self_ : &rope_cross_) : nullptr;
                const int tok = w.is_self ? w.kv.n_prefix : 0;
                // pi0.5: this step's (scale, shift, gate) of the layer's two norm sites
                const float* mod_in = adarms_ ? ada_.as<float>() + ((size_t)s * (2 * L_ + 1) + 2 * l) * 3 * W_ : nullptr;
                const float* mod_post = adarms_ ? mod_in + 3 * W_ : nullptr;
                // RMS archs in bf16: pre-norm, projection, rotation and append are one launch
                bool done = false;
                if (adarms_) {
                    VLA_K(vla_adarms(h.data, mod_in, mod_in + W_, hn.data, dt_, M, W_, eps_, C.stream));
                    prof_mark("pre_norm");
                    Tensor Wqkv = tensor_2d(w.Wqkv.get(), dt_, W_, n_rows_w);
                    qkv_rope_append(C, hn, Wqkv, bq, S_, Hq_, w.is_self, w.is_self, tab, Q.data, w.kv, tok);
                    done = true;
                }
                if (!done && w.Wqkv_ln) {
                    Tensor Wf = tensor_2d(w.Wqkv_ln.get(), dt_, W_, n_rows_w);
                    done = rmsnorm_qkv_rope_append(C, h, Wf, bq, eps_, S_, Hq_, w.is_self, w.is_self, tab, Q.data, w.kv, tok);
                }
                // a GR00T self block without prefix rows, mask or rotation: norm, projections and attention in one launch
                // (from batch 32 on: a workgroup of that launch takes eight observations and one head, and below
                // that too few of them exist to occupy the chip)
                if (!done && w.Wqkv_ada && w.is_self && fuse_self_block_ && B >= 32 && w.kv.n_prefix == 0 && !tab &&
                    suffix_mask_ == VLA_MASK_NONE && pad_start_ >= pad_end_ && Hq_ == Hkv_) {
                    Tensor Wf = tensor_2d(w.Wqkv_ada.as<uint16_t>() + (size_t)s * n_rows_w * W_, dt_, W_, n_rows_w);
                    if (layernorm_qkv_self_attention(C, h, Wf, w.cs_ada.as<float>() + (size_t)s * n_rows_w,
                                                     w.b_ada.as<float>() + (size_t)s * n_rows_w, eps_, S_, Hq_, D_, scale, att, h_stats)) {
                        prof_mark("norm_qkv_attention_self");
                        Tensor Wo = tensor_2d(w.Wo.get(), dt_, (int64_t)Hq_ * D_, W_);
                        if (leave_stats) linear_row_stats(C, Wo, w.bo ? w.bo.as<float>() : nullptr, att, h.data, h, row_stats_.as<float>());
                        else linear(C, Wo, w.bo ? w.bo.as<float>() : nullptr, att, h.data, h);
                        stats_valid = leave_stats;
                        prof_mark("wo_residual");
                        if (I_ > 0) {
                            Tensor mid = tensor_2d(mid_.get(), dt_, I_, M);
                            const float* z = ada_.as<float>() + ((size_t)s * (L_ + 2) + L_) * 2 * W_;  // zeros: plain LayerNorm
                            adaln(C, h, z, z + W_, eps_, hn);
                            prof_mark("ffn_norm");
                            Tensor W1 = tensor_2d(w.W1.get(), dt_, W_, I_), W2 = tensor_2d(w.W2.get(), dt_, I_, W_);
                            ffn_gelu(C, W1, w.b1.as<float>(), W2, w.b2.as<float>(), hn, h.data, mid, h);
                            prof_mark("ffn_in_out");
                        }
                        continue;
                    }
                }
                if (!done && w.Wqkv_ada) {
                    Tensor Wf = tensor_2d(w.Wqkv_ada.as<uint16_t>() + (size_t)s * n_rows_w * W_, dt_, W_, n_rows_w);
                    done = layernorm_qkv_rope_append(C, h, Wf, w.cs_ada.as<float>() + (size_t)s * n_rows_w,
                                                     w.b_ada.as<float>() + (size_t)s * n_rows_w, eps_, S_, Hq_, w.is_self, w.is_self, tab,
                                                     Q.data, w.kv, tok, h_stats);
                }
                if (!done) {
                    if (arch_ == Arch::GR00T) {
                        const float* sc = ada_.as<float>() + ((size_t)s * (L_ + 2) + l) * 2 * W_;
                        adaln(C, h, sc, sc + W_, eps_, hn);
                    } else {
                        rms_norm(C, h, w.ln.get(), eps_, hn);
                    }
                    prof_mark("pre_norm");
                    Tensor Wqkv = tensor_2d(w.Wqkv.get(), dt_, W_, n_rows_w);
                    qkv_rope_append(C, hn, Wqkv, bq, S_, Hq_, w.is_self, w.is_self, tab, Q.data, w.kv, tok);
                }
                prof_mark(w.is_self ? "qkv_rope_append_self" : "q_rope_cross");
                MaskSpec mask;
                mask.pad_start = pad_start_;
                mask.pad_end = pad_end_;
                mask.kind = w.is_self ? suffix_mask_ : VLA_MASK_NONE;
                const int n_keys = w.is_self ? w.kv.n_prefix + S_ : w.kv.n_prefix;
                flash_attention(C, Q, w.kv, n_keys, mask, scale, att, attn_ws_);
                prof_mark(w.is_self ? "attention_self" : (w.from_text && P_txt_ > 0) ? "attention_cross_text" : "attention_cross");
                Tensor Wo = tensor_2d(w.Wo.get(), dt_, (int64_t)Hq_ * D_, W_);
                if (adarms_) {
                    // h1 = x + o_out * gate_attn; h = h1 + mlp_out * gate_ffn (pi05.cpp:273-281)
                    VLA_K(vla_linear_gated(att.data, Wo.data, nullptr, mod_in + 2 * W_, h.data, h.data, dt_, dt_, M, W_,
                                           Hq_ * D_, C.stream));
                    prof_mark("wo_residual");
                    if (I_ > 0) {
                        Tensor mid = tensor_2d(mid_.get(), dt_, I_, M);
                        VLA_K(vla_adarms(h.data, mod_post, mod_post + W_, hn.data, dt_, M, W_, eps_, C.stream));
                        prof_mark("ffn_norm");
                        VLA_K(vla_glu_linear(hn.data, w.Wgu.get(), nullptr, mid.data, dt_, dt_, M, I_, W_, VLA_ACT_GELU, -1.f,
                                             C.stream));
                        prof_mark("ffn_gate_up");
                        VLA_K(vla_linear_gated(mid.data, w.Wd.get(), nullptr, mod_post + 2 * W_, h.data, h.data, dt_, dt_, M, W_,
                                               I_, C.stream));
                        prof_mark("ffn_down_residual");
                    }
                    continue;
                }
                if (leave_stats) linear_row_stats(C, Wo, w.bo ? w.bo.as<float>() : nullptr, att, h.data, h, row_stats_.as<float>());
                else linear(C, Wo, w.bo ? w.bo.as<float>() : nullptr, att, h.data, h);
                stats_valid = leave_stats;
                prof_mark("wo_residual");
                if (I_ > 0) {
                    // FFN half (smolvla.cpp:845-848, pi0.cpp:227-232, dit_head.cpp:132-133)
                    Tensor mid = tensor_2d(mid_.get(), dt_, I_, M);
                    if (arch_ == Arch::GR00T) {
                        const float* z = ada_.as<float>() + ((size_t)s * (L_ + 2) + L_) * 2 * W_;  // zeros: plain LayerNorm
                        adaln(C, h, z, z + W_, eps_, hn);
                        prof_mark("ffn_norm");
                        Tensor W1 = tensor_2d(w.W1.get(), dt_, W_, I_), W2 = tensor_2d(w.W2.get(), dt_, I_, W_);
                        ffn_gelu(C, W1, w.b1.as<float>(), W2, w.b2.as<float>(), hn, h.data, mid, h);
                        prof_mark("ffn_in_out");
                    } else {
                        const int act = arch_ == Arch::SMOLVLA ? VLA_ACT_SILU : VLA_ACT_GELU;
                        Tensor Wd = tensor_2d(w.Wd.get(), dt_, I_, W_);
                        bool fused = false;
                        if (w.Wgu_ln) {
                            Tensor Wf = tensor_2d(w.Wgu_ln.get(), dt_, W_, 2 * (int64_t)I_);
                            fused = ffn_glu(C, Wf, act, Wd, h, eps_, h.data, mid, h);
                        }
                        if (!fused) {
                            rms_norm(C, h, w.ln2.get(), eps_, hn);
                            Tensor Wgu = tensor_2d(w.Wgu.get(), dt_, W_, 2 * (int64_t)I_);
                            ffn_glu(C, Wgu, act, Wd, hn, -1.f, h.data, mid, h);
                        }
                        prof_mark("ffn_gate_up_down");
                    }
                }
            }
            if (fuse_final_norm_ && !head_io_) {
                // final norm + output projection + Euler update in one launch
                if (adarms_) {
                    const float* mf = ada_.as<float>() + ((size_t)s * (2 * L_ + 1) + 2 * L_) * 3 * W_;  // gate unused (pi05.cpp:628)
                    VLA_K(vla_adanorm_euler_step(xt_.as<float>(), h.data, mf, mf + W_, 0, eps_, W_out_.as<float>(), b_out_.as<float>(),
                                                 dt_, B, S_, n_lead_, A_, W_, dt_step_, C.stream));
                } else if (arch_ == Arch::GR00T) {
                    const float* z = ada_.as<float>() + ((size_t)s * (L_ + 2) + L_) * 2 * W_;  // zeros: plain LayerNorm
                    VLA_K(vla_adanorm_euler_step(xt_.as<float>(), h.data, z, z + W_, 1, final_eps_, W_out_.as<float>(),
                                                 b_out_.as<float>(), dt_, B, S_, n_lead_, A_, W_, dt_step_, C.stream));
                } else {
                    VLA_K(vla_rmsnorm_euler_step(xt_.as<float>(), h.data, final_norm_.get(), eps_, W_out_.as<float>(),
                                                 b_out_.as<float>(), dt_, B, S_, n_lead_, A_, W_, dt_step_, C.stream));
                }
                prof_mark("final_norm_euler_step");
                continue;
            }
            if (adarms_) {
                const float* mf = ada_.as<float>() + ((size_t)s * (2 * L_ + 1) + 2 * L_) * 3 * W_;  // gate unused (pi05.cpp:628)
                VLA_K(vla_adarms(h.data, mf, mf + W_, hn.data, dt_, M, W_, eps_, C.stream));
            } else if (head_io_) {
                // DitHead::proj_out then ActionExpert::decode; its last projection is the Euler launch's
                const float* po = ada_.as<float>() + ((size_t)s * (L_ + 2) + L_ + 1) * 2 * W_;
                adaln(C, h, po, po + W_, final_eps_, hn);
                prof_mark("final_norm");
                VLA_K(vla_linear(hn.data, po2W_.get(), po2b_.as<float>(), nullptr, d1_.get(), dt_, dt_, M, O_, W_, C.stream));
                VLA_K(vla_linear_act(d1_.get(), ad1W_.get(), ad1b_.as<float>(), nullptr, d2_.get(), dt_, dt_, M, Hd_, O_, VLA_ACT_RELU,
                                     C.stream));
                prof_mark("head_decode");
                VLA_K(vla_euler_step(xt_.as<float>(), d2_.get(), W_out_.as<float>(), b_out_.as<float>(), dt_, B, S_, n_lead_, A_, Hd_,
                                     dt_step_, C.stream));
                prof_mark("euler_step");
                continue;
            } else if (arch_ == Arch::GR00T) {
                const float* z = ada_.as<float>() + ((size_t)s * (L_ + 2) + L_) * 2 * W_;  // zeros: plain LayerNorm
                adaln(C, h, z, z + W_, final_eps_, hn);
            } else {
                rms_norm(C, h, final_norm_.get(), eps_, hn);
            }
            prof_mark("final_norm");
            VLA_K(vla_euler_step(xt_.as<float>(), hn.data, W_out_.as<float>(), b_out_.as<float>(), dt_, B, S_, n_lead_,
                                 A_, W_, dt_step_, C.stream));
            prof_mark("euler_step");
        }
    }
}

std::vector<float> FlowExpert::fetch() {
    VLA_HIP(hipDeviceSynchronize());
    const int Sa = S_ - n_lead_;
    std::vector<float> out((size_t)B_ * Sa * A_);
    xt_.download(out.data(), out.size() * sizeof(float));
    for (size_t r = 0; r < (size_t)B_ * Sa; ++r)
        for (int j = (int)cfg.real_action_dim; j < A_; ++j) out[r * A_ + j] = 0.0f;
    return out;
}

}  // namespace

ModelArch* flow_expert_create(const Checkpoint& ck) { return new FlowExpert(ck); }

}  // namespace vla
