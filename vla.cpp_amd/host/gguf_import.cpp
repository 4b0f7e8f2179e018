// GGUF checkpoints -> the in-memory weight container the model builders read.
//
// The reference's loaders read their tensors by the names its converters write
// (SmolVLA: hf_to_gguf, src/models/smolvla.cpp:648-755 and the tensor list at 1099-1236;
// pi0: src/models/pi0.cpp:427-437 with src/modules/gemma_expert.h:46-62; pi0.5:
// src/models/pi05.cpp:459-485; BitVLA: src/models/bitvla.cpp:349-373, 640-700).  This file maps those names and metadata
// keys onto the container's own names, fusing what the kernels want fused:
//   [attn_q; attn_k; attn_v] rows -> Wqkv, [attn_k; attn_v] of a backbone layer -> Wkv,
//   [ffn_gate; ffn_up] rows -> Wgu.
// Only the tensors on the action-expert attention path (and the expert's FFN / embedding
// MLPs around it) are read; vision tower, connector and backbone FFN tensors are ignored.
// Also here: the C ABI over the reader itself (include/vla_gguf.h).
#include <cstdlib>
#include <functional>
#include <memory>
#include <stdexcept>

#include "checkpoint.h"
#include "gguf_reader.h"
#include "vla_gguf.h"
#include "vla_kernels.h"

namespace vla {

bool is_gguf_file(const std::string& path) {
    FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    char m[4] = {0, 0, 0, 0};
    const size_t n = std::fread(m, 1, 4, f);
    std::fclose(f);
    return n == 4 && std::memcmp(m, "GGUF", 4) == 0;
}

namespace {

// Names of the gguf tensors an import read (or left on disk for row fetches), in order: what
// vla_gguf_import_trace reports, so that the name map can be checked against name lists kept
// as data (the reference's converter tests hold them, tests/py/test_converters.py).
thread_local std::vector<std::string>* g_trace = nullptr;
void trace(const std::string& name) {
    if (g_trace) g_trace->push_back(name);
}

// Token embeddings read per request from the file (RowSource); owns its own reader.
struct GgufRows : RowSource {
    gguf_reader r{"gguf"};
    std::string name;
    bool fetch(const std::vector<int32_t>& ids, float* dst) override { return r.fetch_rows_f32(name.c_str(), ids, dst, cols); }
};

// prefix.E_lang from `name`: resident when small, left on disk when the matrix is large
// (VLA_EMBED_ON_DEMAND=1 / 0 forces either; read at load).  The reference fetches the rows
// of every request from the file (fetch_rows_f32, src/models/pi0.cpp:530-534).
void put_token_embeddings(const std::string& path, gguf_reader& g, Checkpoint& ck, const std::string& name, int64_t vocab,
                          int64_t hidden, const std::function<std::vector<float>()>& whole) {
    const char* e = std::getenv("VLA_EMBED_ON_DEMAND");
    const bool lazy = e ? std::atoi(e) != 0 : vocab * hidden * 4 > ((int64_t)256 << 20);
    if (!lazy) {
        ck.add_f32("prefix.E_lang", {vocab, hidden}, whole());
        return;
    }
    const gguf_tensor_meta* t = g.meta(name.c_str());
    if (!t || t->ne[0] != hidden || t->ne[1] != vocab) throw std::runtime_error("vla: gguf tensor " + name + " is not [vocab x hidden]");
    auto rows = std::make_shared<GgufRows>();
    if (!rows->r.open(path)) throw std::runtime_error("vla: cannot reopen " + path + " for row fetches");
    rows->name = name;
    rows->rows = vocab;
    rows->cols = hidden;
    trace(name);
    ck.set_row_source("prefix.E_lang", rows);
}

struct Importer {
    gguf_reader& g;
    Checkpoint& ck;
    bool bf16;

    // fp32 tensor `name` with exactly `rows` x `cols` elements (ne0 = cols)
    std::vector<float> mat(const std::string& name, int64_t rows, int64_t cols) {
        const gguf_tensor_meta* t = g.meta(name.c_str());
        if (!t) throw std::runtime_error("vla: gguf has no tensor " + name);
        const int64_t r = t->nelements() / t->ne[0];
        if (t->ne[0] != cols || r != rows)
            throw std::runtime_error("vla: gguf tensor " + name + " is [" + std::to_string(r) + " x " + std::to_string(t->ne[0]) +
                                     "], expected [" + std::to_string(rows) + " x " + std::to_string(cols) + "]");
        std::vector<float> v = g.read_f32(name.c_str());
        if (v.empty()) throw std::runtime_error("vla: cannot read gguf tensor " + name);
        trace(name);
        return v;
    }
    // Row `id` of a cat_linear weight (src/layers/linear.h:30-37): ggml [out, in, n] holds one
    // [in][out] matrix per embodiment; returned transposed, [out][in], as every projection here
    // stores its weight.  The bias [out, n] gives row `id`.
    std::vector<float> cat_w(const std::string& name, int64_t id, int64_t out, int64_t in) {
        const gguf_tensor_meta* t = g.meta(name.c_str());
        if (!t) throw std::runtime_error("vla: gguf has no tensor " + name);
        if (t->ne[0] != out || t->ne[1] != in || id < 0 || id >= t->ne[2])
            throw std::runtime_error("vla: gguf tensor " + name + " is not [n][" + std::to_string(in) + "][" + std::to_string(out) +
                                     "] with embodiment " + std::to_string(id));
        const std::vector<float> all = g.read_f32(name.c_str());
        if (all.empty()) throw std::runtime_error("vla: cannot read gguf tensor " + name);
        trace(name);
        std::vector<float> w((size_t)out * in);
        const float* src = all.data() + (size_t)id * in * out;
        for (int64_t i = 0; i < in; ++i)
            for (int64_t o = 0; o < out; ++o) w[(size_t)o * in + i] = src[(size_t)i * out + o];
        return w;
    }
    std::vector<float> cat_b(const std::string& name, int64_t id, int64_t out) {
        const gguf_tensor_meta* t = g.meta(name.c_str());
        if (!t || t->ne[0] != out || id < 0 || id >= t->ne[1]) throw std::runtime_error("vla: gguf tensor " + name + " is missing or misshapen");
        const std::vector<float> all = g.read_f32(name.c_str());
        if (all.empty()) throw std::runtime_error("vla: cannot read gguf tensor " + name);
        trace(name);
        return std::vector<float>(all.begin() + id * out, all.begin() + (id + 1) * out);
    }
    std::vector<float> vec(const std::string& name, int64_t n) { return mat(name, 1, n); }

    // matrices in the model's weight type, everything else fp32
    void put_weight(const std::string& name, int64_t rows, int64_t cols, const std::vector<float>& v) {
        if (!bf16) {
            ck.add_f32(name, {rows, cols}, v);
            return;
        }
        std::vector<uint16_t> h(v.size());
        for (size_t i = 0; i < v.size(); ++i) h[i] = gguf_float_to_bf16(v[i]);
        ck.add_tensor(name, "bf16", {rows, cols}, h.data(), h.size() * 2);
    }
    // rows of several gguf matrices stacked into one weight
    void put_stacked(const std::string& name, const std::vector<std::string>& parts, const std::vector<int64_t>& rows, int64_t cols) {
        std::vector<float> all;
        int64_t total = 0;
        for (size_t i = 0; i < parts.size(); ++i) {
            const std::vector<float> p = mat(parts[i], rows[i], cols);
            all.insert(all.end(), p.begin(), p.end());
            total += rows[i];
        }
        put_weight(name, total, cols, all);
    }
};

uint32_t need_u32(const gguf_reader& g, const char* k) {
    if (!g.has(k)) throw std::runtime_error(std::string("vla: gguf missing key '") + k + "'");
    return g.u32(k);
}

// SmolVLA, pi0 and pi0.5 share one layout: metadata under "<arch>.", backbone layers
// "vlm.blk.N.", expert layers "aex.blk.N.", the action projections at the top level.
//   SmolVLA: keys of load_config_from_gguf (src/models/smolvla.cpp:570-634), tensors of
//            smolvla_create (1099-1236) under their GGUF names (648-755); cross layers every
//            self_attn_every_n_layers re-project the cached K / V ([kv_dim, kv_dim]).
//   pi0:     keys src/models/pi0.cpp:252-297, tensors 427-437 and GemmaExpert::declare
//            (src/modules/gemma_expert.h:46-62); Gemma norm weights are stored minus one
//            (f32_gemma_norm adds it back, src/gguf_reader.h:151-181).
//   pi0.5:   keys src/models/pi05.cpp:292-328, tensors 459-485: the expert's norm slots hold
//            the adaRMS modulation dense ([3 expert_h, expert_h] weight and [3 expert_h]
//            bias), the time MLP replaces the action-time MLP, there is no state projection.
void import_flow(const std::string& path, gguf_reader& g, Checkpoint& ck, bool bf16, const std::string& arch) {
    const bool smol = arch == "smolvla", pi05 = arch == "pi05", gemma = !smol;
    const std::string kp = arch + ".";
    auto key = [&](const char* k) { return kp + k; };
    auto u = [&](const char* k) { return (int64_t)need_u32(g, key(k).c_str()); };
    if (g.str(key("architecture").c_str()) != arch) throw std::runtime_error("vla: gguf architecture is not '" + arch + "'");
    const int64_t hidden = u("hidden"), Hq = u("n_q_heads"), Hkv = u("n_kv_heads"), D = u("head_dim"), L = u("n_layers"),
                  W = u("expert_h"), I = u("expert_inter"), S = u("chunk_size"), steps = u("num_steps"), sd = u("max_state_dim"),
                  ad = u("max_action_dim"), n_lang = u("tokenizer_max_length");
    const int64_t every = smol ? u("self_attn_every_n_layers") : 1;
    if (!g.has(key("min_period").c_str()) || !g.has(key("max_period").c_str()))
        throw std::runtime_error("vla: gguf missing key '" + kp + "min_period/max_period'");
    if (every < 1 || L < 1 || Hkv < 1 || Hq % Hkv) throw std::runtime_error("vla: gguf geometry is not usable");
    const gguf_tensor_meta* emb = g.meta("token_embd.weight");
    if (!emb || emb->ne[0] != hidden) throw std::runtime_error("vla: gguf token_embd.weight is missing or has the wrong width");
    const int64_t vocab = smol ? u("vocab_size") : emb->ne[1];
    const int64_t qd = Hq * D, kvd = Hkv * D;
    auto f32_or = [&](const char* k, double dflt) { return g.has(key(k).c_str()) ? (double)g.f32(key(k).c_str()) : dflt; };
    ck.set_key("arch", arch);
    ck.set_key("dtype", bf16 ? "bf16" : "f32");
    ck.set_key("n_layers", L);
    ck.set_key("n_q_heads", Hq);
    ck.set_key("n_kv_heads", Hkv);
    ck.set_key("head_dim", D);
    ck.set_key("hidden", hidden);
    ck.set_key("expert_h", W);
    ck.set_key("ffn_dim", I);
    ck.set_key("n_img", (int64_t)(g.has(key("n_img_tokens").c_str()) ? g.u32(key("n_img_tokens").c_str()) : (smol ? 64 : 256)));
    ck.set_key("n_lang", n_lang);
    ck.set_key("n_suffix", smol || pi05 ? S : S + 1);  // pi0: the state token leads the action chunk (pi0.cpp:526-528)
    ck.set_key("max_action_dim", ad);
    ck.set_key("max_state_dim", sd);
    ck.set_key("real_action_dim", u("real_action_dim"));
    ck.set_key("real_state_dim", u("real_state_dim"));
    ck.set_key("num_steps", steps);
    ck.set_key("rms_eps", smol ? 1e-5 : f32_or("rms_norm_eps", 1e-6));  // smolvla.cpp:623-625, pi0.cpp:290
    ck.set_key("rope_freq_base", gemma && g.has(key("rope_theta").c_str()) ? g.f64(key("rope_theta").c_str()) : 10000.0);
    ck.set_key("self_attn_every_n", every);
    ck.set_key("min_period", g.f64(key("min_period").c_str()));
    ck.set_key("max_period", g.f64(key("max_period").c_str()));
    ck.set_key("vocab", vocab);

    Importer im{g, ck, bf16};
    auto norm = [&](const std::string& name, int64_t n) {  // Gemma stores norm weights minus one
        std::vector<float> v = im.vec(name, n);
        if (gemma)
            for (float& x : v) x += 1.0f;
        return v;
    };
    put_token_embeddings(path, g, ck, "token_embd.weight", vocab, hidden, [&]() { return im.mat("token_embd.weight", vocab, hidden); });
    if (smol) {
        ck.add_f32("prefix.Wstate", {hidden, sd}, im.mat("state_proj.weight", hidden, sd));
        ck.add_f32("prefix.bstate", {hidden}, im.vec("state_proj.bias", hidden));
    } else if (!pi05) {
        ck.add_f32("act.W_sp", {W, sd}, im.mat("state_proj.weight", W, sd));
        ck.add_f32("act.b_sp", {W}, im.vec("state_proj.bias", W));
    }
    ck.add_f32("act.W_in", {W, ad}, im.mat("action_in_proj.weight", W, ad));
    ck.add_f32("act.b_in", {W}, im.vec("action_in_proj.bias", W));
    ck.add_f32("act.W_out", {ad, W}, im.mat("action_out_proj.weight", ad, W));
    ck.add_f32("act.b_out", {ad}, im.vec("action_out_proj.bias", ad));
    if (pi05) {
        ck.add_f32("te.W_tin", {W, W}, im.mat("time_mlp_in.weight", W, W));
        ck.add_f32("te.b_tin", {W}, im.vec("time_mlp_in.bias", W));
        ck.add_f32("te.W_tout", {W, W}, im.mat("time_mlp_out.weight", W, W));
        ck.add_f32("te.b_tout", {W}, im.vec("time_mlp_out.bias", W));
        ck.add_f32("act.ada_final_w", {3 * W, W}, im.mat("aex.output_norm.weight", 3 * W, W));
        ck.add_f32("act.ada_final_b", {3 * W}, im.vec("aex.output_norm.bias", 3 * W));
    } else {
        ck.add_f32("act.W_at1", {W, 2 * W}, im.mat("action_time_mlp_in.weight", W, 2 * W));
        ck.add_f32("act.b_at1", {W}, im.vec("action_time_mlp_in.bias", W));
        ck.add_f32("act.W_at2", {W, W}, im.mat("action_time_mlp_out.weight", W, W));
        ck.add_f32("act.b_at2", {W}, im.vec("action_time_mlp_out.bias", W));
        im.put_weight("act.norm", 1, W, norm("aex.output_norm.weight", W));
    }
    for (int64_t l = 0; l < L; ++l) {
        const std::string a = "aex.blk." + std::to_string(l) + ".", v = "vlm.blk." + std::to_string(l) + ".";
        const std::string e = "ex." + std::to_string(l) + ".", p = "vlm." + std::to_string(l) + ".";
        const bool self = l % every == 0;
        if (pi05) {
            ck.add_f32(e + "ada_in_w", {3 * W, W}, im.mat(a + "attn_norm.weight", 3 * W, W));
            ck.add_f32(e + "ada_in_b", {3 * W}, im.vec(a + "attn_norm.bias", 3 * W));
            ck.add_f32(e + "ada_post_w", {3 * W, W}, im.mat(a + "ffn_norm.weight", 3 * W, W));
            ck.add_f32(e + "ada_post_b", {3 * W}, im.vec(a + "ffn_norm.bias", 3 * W));
        } else {
            im.put_weight(e + "ln", 1, W, norm(a + "attn_norm.weight", W));
            im.put_weight(e + "ln2", 1, W, norm(a + "ffn_norm.weight", W));
        }
        if (self) {
            im.put_stacked(e + "Wqkv", {a + "attn_q.weight", a + "attn_k.weight", a + "attn_v.weight"}, {qd, kvd, kvd}, W);
        } else {
            // cross layers re-project the cached K and V: [kv_dim, kv_dim] (smolvla.cpp:1207-1208)
            im.put_weight(e + "Wq", qd, W, im.mat(a + "attn_q.weight", qd, W));
            im.put_weight(e + "Wk_x", kvd, kvd, im.mat(a + "attn_k.weight", kvd, kvd));
            im.put_weight(e + "Wv_x", kvd, kvd, im.mat(a + "attn_v.weight", kvd, kvd));
        }
        im.put_weight(e + "Wo", W, qd, im.mat(a + "attn_o.weight", W, qd));
        im.put_stacked(e + "Wgu", {a + "ffn_gate.weight", a + "ffn_up.weight"}, {I, I}, W);
        im.put_weight(e + "Wd", W, I, im.mat(a + "ffn_down.weight", W, I));
        im.put_weight(p + "ln", 1, hidden, norm(v + "attn_norm.weight", hidden));
        im.put_stacked(p + "Wkv", {v + "attn_k.weight", v + "attn_v.weight"}, {kvd, kvd}, hidden);
    }
}

// BitVLA language model: keys of load_config (src/models/bitvla.cpp:349-373), the ternary
// projections of each block either as float tensors (quantised again at load, 430-451) or,
// with bitvla.quant.int2_packed, as ladder-packed I8 tensors with a ".scale" sidecar
// (728-747).  The action-token embeddings and the output projection this library's
// token-by-token schedule uses have no counterpart in the reference's file; they are read
// under this library's own names (act.emb, act.W_out, act.b_out) and must be present.
// GR00T N1.5 action head: keys of load_config (src/models/gr00tn1d5.cpp:92-147), DiT tensors of
// DitHead::declare (src/modules/dit_head.cpp:29-85; GGUF names "aex.dit.N.{adaln, attn_q,
// attn_k, attn_v, attn_o, ff0, ff2}.{weight, bias}", the list the reference's converter test
// holds, tests/py/test_converters.py:178-184), the head's own MLPs of ActionExpert::declare
// (src/modules/action_expert.cpp:20-39) with the embodiment's row selected here (id 24 unless
// VLA_GR00T_EMBODIMENT gives a number or a tag of gr00t_n1_5.embodiment_tag_mapping,
// gr00tn1d5.cpp:149-167), "aex.future_tokens" and "aex.pos_embd".  Cross layers (even, or all
// without dit_interleave) take K / V from the backbone features ([inner, backbone_embedding_dim]),
// self layers fuse [q; k; v].  The backbone (vision tower, Qwen3 layers, VL self-attention) is
// not read: precomputed_img_emb stands for its output rows.
//
// N1.6 and N1.7 (variant 6 / 7) share the head and its names under the key prefixes
// gr00t_n1_6. / gr00t_n1_7. (src/models/gr00tn1d6.cpp:96-189, 294-298; src/models/gr00tn1d7.cpp:
// 119-215): no future tokens (the sequence is the state row and action_horizon rows,
// gr00tn1d6.cpp:457), cross layers alternating between the text and the image rows every
// attend_text_every_n_blocks, horizon / action / state defaults 50 / 128 / 128 (N1.6) and
// 40 / 132 / 132 (N1.7), 64 image rows per view, and the embodiment row from
// embodiment_id_mapping: "gr1" else 20 (N1.6), "libero_sim" else 2 (N1.7), VLA_GR00T_EMBODIMENT
// over both; N1.7 also takes VLA_NUM_STEPS (gr00tn1d7.cpp:150-156).  N1.6 feeds the head
// layer_norm(backbone rows) with aex.vlln.{weight, bias} (gr00tn1d6.cpp:436): those are read and
// applied, the input rows standing for the language model's last hidden states.  In N1.5 and
// N1.7 a VL self-attention stack follows vlln; it belongs to the backbone, so neither is read and
// the input rows stand for its output.  The text rows come from token_embd.weight when the
// file holds it at the backbone width (rows left on disk when large); without it there are no
// text rows and the text layers attend to the image rows (gr00tn1d6.cpp:438).
void import_gr00t(const std::string& path, gguf_reader& g, Checkpoint& ck, bool bf16, int variant) {
    const std::string prefix = variant == 5 ? "gr00t_n1_5." : variant == 6 ? "gr00t_n1_6." : "gr00t_n1_7.";
    auto key = [&](const char* k) { return prefix + k; };
    auto u = [&](const char* k) { return (int64_t)need_u32(g, key(k).c_str()); };
    auto u_or = [&](const char* k, int64_t d) { return g.has(key(k).c_str()) ? (int64_t)g.u32(key(k).c_str()) : d; };
    auto f_or = [&](const char* k, double d) { return g.has(key(k).c_str()) ? (double)g.f32(key(k).c_str()) : d; };
    const bool alt = variant != 5;
    const int64_t Wv = u_or("backbone_embedding_dim", 2048), E = u_or("input_embedding_dim", 1536), W = u("dit_hidden"),
                  H = u("dit_heads"), D = u("dit_head_dim"), L = u("dit_layers"), interleave = u_or("dit_interleave", 1),
                  NF = alt ? 0 : u_or("num_target_vision_tokens", 32),
                  AH = u_or("action_horizon", variant == 5 ? 16 : variant == 6 ? 50 : 40),
                  A = u_or("action_dim", variant == 5 ? 32 : variant == 6 ? 128 : 132),
                  sd = u_or("max_state_dim", variant == 5 ? 64 : variant == 6 ? 128 : 132),
                  buckets = u_or("num_timestep_buckets", 1000), n_emb = u_or("max_num_embodiments", 32),
                  text_every = u_or("attend_text_every_n_blocks", 2);
    int64_t steps = u_or("num_inference_timesteps", 4);
    if (variant == 7)
        if (const char* ns = std::getenv("VLA_NUM_STEPS")) {
            char* end = nullptr;
            const long v = std::strtol(ns, &end, 10);
            if (end && *end == '\0' && v >= 1) steps = v;
        }
    if (H < 1 || D < 1 || H * D != W || E != W || L < 1) throw std::runtime_error("vla: gr00t gguf geometry is not usable (heads x head_dim, embedding and DiT widths must agree)");
    if (alt && text_every < 1) throw std::runtime_error("vla: attend_text_every_n_blocks must be >= 1");
    int64_t id = variant == 5 ? 24 : variant == 6 ? 20 : 2;
    const char* map_key = variant == 5 ? "embodiment_tag_mapping" : "embodiment_id_mapping";
    // the id that follows "tag" and a colon in the mapping's JSON text, or -1
    auto lookup = [&](const std::string& tag) -> long {
        const std::string js = g.str(key(map_key).c_str());
        if (variant == 5) {  // gr00tn1d5.cpp:155-158 searches for "tag": as one string
            const std::string k2 = "\"" + tag + "\":";
            const size_t p = js.find(k2);
            return p == std::string::npos ? -1 : std::strtol(js.c_str() + p + k2.size(), nullptr, 10);
        }
        const std::string k2 = "\"" + tag + "\"";  // gr00tn1d6.cpp:150-160: the key, then the next colon
        size_t p = js.find(k2);
        if (p == std::string::npos) return -1;
        p = js.find(':', p + k2.size());
        return p == std::string::npos ? -1 : std::strtol(js.c_str() + p + 1, nullptr, 10);
    };
    if (alt) {
        const long dflt = lookup(variant == 6 ? "gr1" : "libero_sim");
        if (dflt >= 0) id = dflt;
    }
    if (const char* e = std::getenv("VLA_GR00T_EMBODIMENT")) {
        char* end = nullptr;
        const long v = std::strtol(e, &end, 10);
        if (end && *end == '\0') {  // a number; an empty value reads as 0, as in the reference (gr00tn1d5.cpp:150-153)
            id = v;
        } else {
            // a tag: looked up in the mapping; an unknown tag keeps the id with a warning (gr00tn1d5.cpp:154-160)
            const long t = lookup(e);
            if (t >= 0)
                id = t;
            else
                std::fprintf(stderr, "vla(gr00t): embodiment tag '%s' not in %s; using id %lld\n", e, map_key, (long long)id);
        }
    }
    if (id < 0 || id >= n_emb) throw std::runtime_error("vla: embodiment id out of range");
    Importer im{g, ck, bf16};
    const gguf_tensor_meta* ff0 = g.meta("aex.dit.0.ff0.weight");
    const gguf_tensor_meta* po2 = g.meta("aex.dit.proj_out2.weight");
    const gguf_tensor_meta* se1 = g.meta("aex.state_enc.l1.W");
    const gguf_tensor_meta* ad1 = g.meta("aex.act_dec.l1.W");
    const gguf_tensor_meta* pe = g.meta("aex.pos_embd");
    if (!ff0 || !po2 || !se1 || !ad1 || !pe) throw std::runtime_error("vla: gr00t gguf lacks the DiT head tensors (ff0, proj_out2, state_enc, act_dec, pos_embd)");
    const int64_t I = ff0->ne[1], O = po2->ne[1], Hs = se1->ne[0], Hd = ad1->ne[0], max_pos = pe->ne[1];
    // text rows (N1.6 / N1.7): the token embedding matrix at the backbone width, when the file has one
    int64_t vocab = 0, n_lang = 0;
    if (alt) {
        const gguf_tensor_meta* te = g.meta("token_embd.weight");
        if (te && te->ne[0] == Wv && te->nelements() / te->ne[0] > 0) {
            vocab = te->nelements() / te->ne[0];
            n_lang = u_or("max_seq_len", 1024);
        }
    }
    ck.set_key("arch", alt ? "gr00t_n1d6" : "gr00t_n1d5");
    ck.set_key("dtype", bf16 ? "bf16" : "f32");
    ck.set_key("n_layers", L);
    ck.set_key("n_q_heads", H);
    ck.set_key("n_kv_heads", H);
    ck.set_key("head_dim", D);
    ck.set_key("hidden", Wv);
    ck.set_key("expert_h", W);
    ck.set_key("ffn_dim", I);
    ck.set_key("n_img", u_or("n_img_tokens", alt ? 64 : 256));
    ck.set_key("n_lang", n_lang);
    ck.set_key("vocab", vocab);
    if (alt) ck.set_key("attend_text_every_n", text_every);
    ck.set_key("n_suffix", 1 + NF + AH);
    ck.set_key("max_action_dim", A);
    ck.set_key("max_state_dim", sd);
    ck.set_key("real_action_dim", A);
    ck.set_key("real_state_dim", sd);
    ck.set_key("num_steps", steps);
    ck.set_key("rms_eps", f_or("ln_eps", 1e-5));
    ck.set_key("norm_out_eps", f_or("norm_out_eps", 1e-6));
    ck.set_key("dit_interleave", interleave);
    ck.set_key("head_io", (int64_t)1);
    ck.set_key("num_future", NF);
    ck.set_key("dit_out_dim", O);
    ck.set_key("dec_hidden", Hd);
    ck.set_key("state_hidden", Hs);
    ck.set_key("num_buckets", buckets);

    ck.add_f32("te.l1W", {W, 256}, im.mat("aex.dit.time_emb.l1.weight", W, 256));
    ck.add_f32("te.l1b", {W}, im.vec("aex.dit.time_emb.l1.bias", W));
    ck.add_f32("te.l2W", {W, W}, im.mat("aex.dit.time_emb.l2.weight", W, W));
    ck.add_f32("te.l2b", {W}, im.vec("aex.dit.time_emb.l2.bias", W));
    ck.add_f32("aex.po1W", {2 * W, W}, im.mat("aex.dit.proj_out1.weight", 2 * W, W));
    ck.add_f32("aex.po1b", {2 * W}, im.vec("aex.dit.proj_out1.bias", 2 * W));
    im.put_weight("aex.po2W", O, W, im.mat("aex.dit.proj_out2.weight", O, W));
    ck.add_f32("aex.po2b", {O}, im.vec("aex.dit.proj_out2.bias", O));
    ck.add_f32("aex.se_l1W", {Hs, sd}, im.cat_w("aex.state_enc.l1.W", id, Hs, sd));
    ck.add_f32("aex.se_l1b", {Hs}, im.cat_b("aex.state_enc.l1.b", id, Hs));
    ck.add_f32("aex.se_l2W", {W, Hs}, im.cat_w("aex.state_enc.l2.W", id, W, Hs));
    ck.add_f32("aex.se_l2b", {W}, im.cat_b("aex.state_enc.l2.b", id, W));
    ck.add_f32("aex.ae_W1", {W, A}, im.cat_w("aex.act_enc.W1.W", id, W, A));
    ck.add_f32("aex.ae_b1", {W}, im.cat_b("aex.act_enc.W1.b", id, W));
    ck.add_f32("aex.ae_W2", {W, 2 * W}, im.cat_w("aex.act_enc.W2.W", id, W, 2 * W));
    ck.add_f32("aex.ae_b2", {W}, im.cat_b("aex.act_enc.W2.b", id, W));
    ck.add_f32("aex.ae_W3", {W, W}, im.cat_w("aex.act_enc.W3.W", id, W, W));
    ck.add_f32("aex.ae_b3", {W}, im.cat_b("aex.act_enc.W3.b", id, W));
    im.put_weight("aex.ad_l1W", Hd, O, im.cat_w("aex.act_dec.l1.W", id, Hd, O));
    ck.add_f32("aex.ad_l1b", {Hd}, im.cat_b("aex.act_dec.l1.b", id, Hd));
    ck.add_f32("aex.ad_l2W", {A, Hd}, im.cat_w("aex.act_dec.l2.W", id, A, Hd));
    ck.add_f32("aex.ad_l2b", {A}, im.cat_b("aex.act_dec.l2.b", id, A));
    ck.add_f32("aex.pos_embd", {max_pos, W}, im.mat("aex.pos_embd", max_pos, W));
    if (NF > 0) ck.add_f32("aex.future_tokens", {NF, W}, im.mat("aex.future_tokens", NF, W));
    if (vocab > 0) put_token_embeddings(path, g, ck, "token_embd.weight", vocab, Wv, [&]() { return im.mat("token_embd.weight", vocab, Wv); });
    if (variant == 6) {
        ck.set_key("vlln_eps", f_or("vlln_eps", 1e-5));
        ck.add_f32("prefix.vlln_w", {Wv}, im.vec("aex.vlln.weight", Wv));
        ck.add_f32("prefix.vlln_b", {Wv}, im.vec("aex.vlln.bias", Wv));
    }
    for (int64_t l = 0; l < L; ++l) {
        const std::string a = "aex.dit." + std::to_string(l) + ".", e = "ex." + std::to_string(l) + ".", p = "vlm." + std::to_string(l) + ".";
        const bool self = interleave != 0 && l % 2 == 1;
        ck.add_f32(e + "adaln_w", {2 * W, W}, im.mat(a + "adaln.weight", 2 * W, W));
        ck.add_f32(e + "adaln_b", {2 * W}, im.vec(a + "adaln.bias", 2 * W));
        auto cat3 = [&](const std::vector<std::string>& names, int64_t n) {
            std::vector<float> all;
            for (const std::string& nm : names) {
                const std::vector<float> v = im.vec(nm, n);
                all.insert(all.end(), v.begin(), v.end());
            }
            return all;
        };
        if (self) {
            im.put_stacked(e + "Wqkv", {a + "attn_q.weight", a + "attn_k.weight", a + "attn_v.weight"}, {W, W, W}, W);
            ck.add_f32(e + "bqkv", {3 * W}, cat3({a + "attn_q.bias", a + "attn_k.bias", a + "attn_v.bias"}, W));
        } else {
            im.put_weight(e + "Wq", W, W, im.mat(a + "attn_q.weight", W, W));
            ck.add_f32(e + "bq", {W}, im.vec(a + "attn_q.bias", W));
            im.put_stacked(p + "Wkv", {a + "attn_k.weight", a + "attn_v.weight"}, {W, W}, Wv);
            ck.add_f32(p + "bkv", {2 * W}, cat3({a + "attn_k.bias", a + "attn_v.bias"}, W));
        }
        im.put_weight(e + "Wo", W, W, im.mat(a + "attn_o.weight", W, W));
        ck.add_f32(e + "bo", {W}, im.vec(a + "attn_o.bias", W));
        im.put_weight(e + "W1", I, W, im.mat(a + "ff0.weight", I, W));
        ck.add_f32(e + "b1", {I}, im.vec(a + "ff0.bias", I));
        im.put_weight(e + "W2", W, I, im.mat(a + "ff2.weight", W, I));
        ck.add_f32(e + "b2", {W}, im.vec(a + "ff2.bias", W));
    }
}

void import_bitvla(const std::string& path, gguf_reader& g, Checkpoint& ck) {
    const int64_t H = need_u32(g, "bitvla.lm.hidden"), L = need_u32(g, "bitvla.lm.layers"), Hq = need_u32(g, "bitvla.lm.q_heads"),
                  Hkv = need_u32(g, "bitvla.lm.kv_heads"), D = need_u32(g, "bitvla.lm.head_dim"),
                  vocab = need_u32(g, "bitvla.lm.vocab_size");
    if (Hkv < 1 || Hq % Hkv || Hq * D != H) throw std::runtime_error("vla: gguf lm q_heads x head_dim does not match hidden");
    const bool packed = g.has("bitvla.quant.int2_packed") && g.u32("bitvla.quant.int2_packed") != 0;
    const int64_t qd = Hq * D, kvd = Hkv * D;
    const gguf_tensor_meta* emb = g.meta("act.emb");
    const gguf_tensor_meta* wout = g.meta("act.W_out");
    if (!emb || !wout) throw std::runtime_error("vla: bitvla gguf needs the act.emb / act.W_out / act.b_out tensors");
    const int64_t n_act = emb->ne[1], A = wout->ne[1];
    ck.set_key("arch", "bitvla");
    ck.set_key("dtype", "bf16");
    ck.set_key("n_layers", L);
    ck.set_key("n_q_heads", Hq);
    ck.set_key("n_kv_heads", Hkv);
    ck.set_key("head_dim", D);
    ck.set_key("hidden", H);
    ck.set_key("n_img", (int64_t)(g.has("bitvla.vit.n_patches") ? g.u32("bitvla.vit.n_patches") : 256));
    ck.set_key("n_lang", (int64_t)(g.has("bitvla.lm.max_text") ? g.u32("bitvla.lm.max_text") : 256));
    ck.set_key("n_suffix", n_act);
    ck.set_key("max_action_dim", A);
    ck.set_key("real_action_dim", (int64_t)(g.has("bitvla.action.action_dim") ? g.u32("bitvla.action.action_dim") : A));
    ck.set_key("rms_eps", (double)(g.has("bitvla.lm.rms_eps") ? g.f32("bitvla.lm.rms_eps") : 1e-5f));
    ck.set_key("rope_freq_base", (double)(g.has("bitvla.lm.rope_theta") ? g.f32("bitvla.lm.rope_theta") : 500000.f));
    ck.set_key("vocab", vocab);

    Importer im{g, ck, false};
    put_token_embeddings(path, g, ck, "token_embd.weight", vocab, H, [&]() { return im.mat("token_embd.weight", vocab, H); });
    ck.add_f32("act.emb", {n_act, H}, im.mat("act.emb", n_act, H));
    ck.add_f32("act.W_out", {A, H}, im.mat("act.W_out", A, H));
    ck.add_f32("act.b_out", {A}, im.vec("act.b_out", A));
    ck.add_f32("act.norm", {H}, im.vec("lm.output_norm.weight", H));
    for (int64_t l = 0; l < L; ++l) {
        const std::string b = "lm.blk." + std::to_string(l) + ".", o = "lm." + std::to_string(l) + ".";
        {
            std::vector<float> n = im.vec(b + "attn_norm.weight", H), s = im.vec(b + "attn_sub_norm.weight", H);
            std::vector<uint16_t> nh(H), sh(H);
            for (int64_t i = 0; i < H; ++i) {
                nh[i] = gguf_float_to_bf16(n[i]);
                sh[i] = gguf_float_to_bf16(s[i]);
            }
            ck.add_tensor(o + "attn_norm", "bf16", {H}, nh.data(), nh.size() * 2);
            ck.add_tensor(o + "sub_norm", "bf16", {H}, sh.data(), sh.size() * 2);
        }
        if (!packed) {
            std::vector<float> all;
            for (const auto& part : {std::make_pair("attn_q.weight", qd), std::make_pair("attn_k.weight", kvd), std::make_pair("attn_v.weight", kvd)}) {
                const std::vector<float> p = im.mat(b + part.first, part.second, H);
                all.insert(all.end(), p.begin(), p.end());
            }
            ck.add_f32(o + "Wqkv", {qd + 2 * kvd, H}, all);
            ck.add_f32(o + "Wo", {H, qd}, im.mat(b + "attn_o.weight", H, qd));
            continue;
        }
        // ladder-packed: each source tensor goes into the gfx950 word order on its own; that
        // order is blocked by 32 output rows, so the fused tensor is the blocks back to back
        if (qd % 32 || kvd % 32 || H % 128) throw std::runtime_error("vla: gguf int2 tensors need rows % 32 == 0 and K % 128 == 0");
        std::vector<uint32_t> fused;
        std::vector<float> ws;
        for (const auto& part : {std::make_pair("attn_q", qd), std::make_pair("attn_k", kvd), std::make_pair("attn_v", kvd)}) {
            const std::string name = b + part.first + ".weight";
            std::vector<uint8_t> bytes = g.read_convert(name.c_str(), GGUF_T_I8);
            trace(name);
            if ((int64_t)bytes.size() != part.second * H / 4) throw std::runtime_error("vla: gguf int2 tensor " + name + " has the wrong size");
            std::vector<uint32_t> words((size_t)vla_ternary_packed_words((int)part.second, (int)H));
            if (vla_ternary_repack_ladder_host(bytes.data(), (int)part.second, (int)H, words.data()) != VLA_K_OK)
                throw std::runtime_error("vla: cannot re-order gguf int2 tensor " + name);
            fused.insert(fused.end(), words.begin(), words.end());
            const std::vector<float> sc = g.read_f32((b + part.first + ".scale").c_str());
            trace(b + part.first + ".scale");
            if (sc.empty()) throw std::runtime_error("vla: int2 tensor " + name + " has no .scale sidecar");
            ws.push_back(sc[0]);
        }
        ck.add_tensor(o + "Wqkv.p2", "u8", {(int64_t)fused.size() * 4}, fused.data(), fused.size() * 4);
        ck.add_f32(o + "Wqkv.ws", {3}, ws);
        const std::string on = b + "attn_o.weight";
        std::vector<uint8_t> ob = g.read_convert(on.c_str(), GGUF_T_I8);
        trace(on);
        trace(b + "attn_o.scale");
        if ((int64_t)ob.size() != H * qd / 4) throw std::runtime_error("vla: gguf int2 tensor " + on + " has the wrong size");
        ck.add_tensor(o + "Wo.i2", "u8", {(int64_t)ob.size()}, ob.data(), ob.size());
        const std::vector<float> osc = g.read_f32((b + "attn_o.scale").c_str());
        if (osc.empty()) throw std::runtime_error("vla: int2 tensor " + on + " has no .scale sidecar");
        ck.add_f32(o + "Wo.ws", {1}, {osc[0]});
    }
}

}  // namespace

// Weight type of the float architectures: bf16 unless VLA_WEIGHT_DTYPE=f32 (the reference's
// default resident type is BF16 as well, src/models/smolvla.cpp:1965).
Checkpoint import_gguf(const std::string& path) {
    gguf_reader g("gguf");
    if (!g.open(path)) throw std::runtime_error("vla: cannot read gguf " + path);
    const char* wd = std::getenv("VLA_WEIGHT_DTYPE");
    const bool bf16 = !(wd && std::string(wd) == "f32");
    Checkpoint ck;
    if (g.has("smolvla.architecture")) import_flow(path, g, ck, bf16, "smolvla");
    else if (g.has("pi05.architecture")) import_flow(path, g, ck, bf16, "pi05");
    else if (g.has("pi0.architecture")) import_flow(path, g, ck, bf16, "pi0");
    else if (g.has("gr00t_n1_5.architecture")) import_gr00t(path, g, ck, bf16, 5);
    else if (g.has("gr00t_n1_6.architecture")) import_gr00t(path, g, ck, bf16, 6);
    else if (g.has("gr00t_n1_7.architecture")) import_gr00t(path, g, ck, bf16, 7);
    else if (g.has("bitvla.architecture") || g.has("bitvla.lm.hidden")) import_bitvla(path, g, ck);
    else throw std::runtime_error("vla: " + path + ": no importer for this gguf's architecture");
    return ck;
}

}  // namespace vla

// ---------------------------------------------------------------- C ABI over the reader
struct vla_gguf {
    vla::gguf_reader r{"gguf"};
};

extern "C" {

int64_t vla_gguf_import_trace(const char* path, char* out, int64_t cap) {
    if (!path || !out || cap <= 0) return VLA_GGUF_ERR_ARG;
    std::vector<std::string> names;
    try {
        vla::g_trace = &names;
        (void)vla::import_gguf(path);
        vla::g_trace = nullptr;
    } catch (const std::exception& e) {
        vla::g_trace = nullptr;
        std::fprintf(stderr, "%s\n", e.what());
        return VLA_GGUF_ERR_READ;
    }
    std::string all;
    for (const std::string& n : names) all += n + "\n";
    if ((int64_t)all.size() + 1 > cap) return -(int64_t)(all.size() + 1) - 16;
    std::memcpy(out, all.c_str(), all.size() + 1);
    return (int64_t)all.size();
}

vla_gguf* vla_gguf_open(const char* path) {
    if (!path) return nullptr;
    try {
        std::unique_ptr<vla_gguf> g(new vla_gguf());
        if (!g->r.open(path)) return nullptr;
        return g.release();
    } catch (...) {
        return nullptr;
    }
}

void vla_gguf_close(vla_gguf* g) { delete g; }

int32_t vla_gguf_version(const vla_gguf* g) { return g ? (int32_t)g->r.version : 0; }
int64_t vla_gguf_data_offset(const vla_gguf* g) { return g ? (int64_t)g->r.data_off : -1; }
int32_t vla_gguf_has_key(const vla_gguf* g, const char* key) { return g && key && g->r.has(key) ? 1 : 0; }
int32_t vla_gguf_key_type(const vla_gguf* g, const char* key) {
    if (!g || !key) return -1;
    auto it = g->r.kv.find(key);
    return it == g->r.kv.end() ? -1 : (int32_t)it->second.type;
}
uint32_t vla_gguf_u32(const vla_gguf* g, const char* key) { return g && key ? g->r.u32(key) : 0u; }
float vla_gguf_f32(const vla_gguf* g, const char* key) { return g && key ? g->r.f32(key) : 0.f; }
double vla_gguf_f64(const vla_gguf* g, const char* key) { return g && key ? g->r.f64(key) : 0.0; }

int64_t vla_gguf_str(const vla_gguf* g, const char* key, char* buf, int64_t cap) {
    if (!g || !key) return -1;
    const vla::gguf_kv* v = g->r.typed_key(key, vla::GGUF_KV_STRING);
    if (!v) return -1;
    if (buf && cap > 0) {
        const size_t n = std::min((size_t)cap - 1, v->s.size());
        std::memcpy(buf, v->s.data(), n);
        buf[n] = 0;
    }
    return (int64_t)v->s.size();
}

int64_t vla_gguf_array_len(const vla_gguf* g, const char* key, int32_t* elem_type) {
    if (!g || !key) return -1;
    const vla::gguf_kv* v = g->r.typed_key(key, vla::GGUF_KV_ARRAY);
    if (!v) return -1;
    if (elem_type) *elem_type = (int32_t)v->elem_type;
    return (int64_t)v->count;
}

int64_t vla_gguf_n_tensors(const vla_gguf* g) { return g ? (int64_t)g->r.tensors.size() : 0; }

const char* vla_gguf_tensor_name(const vla_gguf* g, int64_t i) {
    if (!g || i < 0 || i >= (int64_t)g->r.tensors.size()) return nullptr;
    return g->r.tensors[(size_t)i].name.c_str();
}

int32_t vla_gguf_tensor_info(const vla_gguf* g, const char* name, int32_t* type, int32_t* n_dims, int64_t ne[4], int64_t* offset,
                             int64_t* nbytes) {
    if (!g || !name) return VLA_GGUF_ERR_ARG;
    const vla::gguf_tensor_meta* t = g->r.meta(name);
    if (!t) return VLA_GGUF_ERR_MISSING;
    if (type) *type = (int32_t)t->type;
    if (n_dims) *n_dims = t->n_dims;
    if (ne)
        for (int d = 0; d < 4; ++d) ne[d] = t->ne[d];
    if (offset) *offset = (int64_t)t->offset;
    if (nbytes) *nbytes = (int64_t)t->nbytes;
    return VLA_GGUF_OK;
}

int32_t vla_gguf_read_raw(vla_gguf* g, const char* name, void* buf, int64_t cap) {
    if (!g || !name || !buf || cap < 0) return VLA_GGUF_ERR_ARG;
    if (!g->r.meta(name)) return VLA_GGUF_ERR_MISSING;
    return g->r.read_raw(name, buf, (size_t)cap) ? VLA_GGUF_OK : VLA_GGUF_ERR_READ;
}

int32_t vla_gguf_read_f32(vla_gguf* g, const char* name, float* out, int64_t n) {
    if (!g || !name || !out) return VLA_GGUF_ERR_ARG;
    const vla::gguf_tensor_meta* t = g->r.meta(name);
    if (!t) return VLA_GGUF_ERR_MISSING;
    if (t->nelements() != n) return VLA_GGUF_ERR_ARG;
    try {
        const std::vector<float> v = g->r.read_f32(name);
        if (v.empty()) return VLA_GGUF_ERR_READ;
        std::memcpy(out, v.data(), v.size() * sizeof(float));
        return VLA_GGUF_OK;
    } catch (...) {
        return VLA_GGUF_ERR_READ;
    }
}

int32_t vla_gguf_read_convert(vla_gguf* g, const char* name, int32_t target_type, int32_t gemma_norm, void* out, int64_t cap) {
    if (!g || !name || !out || cap < 0) return VLA_GGUF_ERR_ARG;
    if (!g->r.meta(name)) return VLA_GGUF_ERR_MISSING;
    try {
        const std::vector<uint8_t> v = g->r.read_convert(name, (uint32_t)target_type, gemma_norm != 0);
        if (v.empty()) return VLA_GGUF_ERR_READ;
        if ((int64_t)v.size() != cap) return VLA_GGUF_ERR_ARG;
        std::memcpy(out, v.data(), v.size());
        return VLA_GGUF_OK;
    } catch (...) {
        return VLA_GGUF_ERR_READ;
    }
}

int32_t vla_gguf_fetch_rows_f32(vla_gguf* g, const char* name, const int32_t* row_ids, int64_t n_rows, float* dst, int64_t cols) {
    if (!g || !name || (!row_ids && n_rows > 0) || !dst || n_rows < 0 || cols <= 0) return VLA_GGUF_ERR_ARG;
    if (!g->r.meta(name)) return VLA_GGUF_ERR_MISSING;
    try {
        const std::vector<int32_t> ids(row_ids, row_ids + n_rows);
        return g->r.fetch_rows_f32(name, ids, dst, cols) ? VLA_GGUF_OK : VLA_GGUF_ERR_READ;
    } catch (...) {
        return VLA_GGUF_ERR_READ;
    }
}

}  // extern "C"
