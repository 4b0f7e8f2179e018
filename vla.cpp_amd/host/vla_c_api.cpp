// The C boundary of include/vla.h: type conversion, argument checks and a
// barrier that keeps C++ exceptions inside (the contract of the reference's
// src/vla_c_api.cpp:43-190: NULL handles -> VLA_ERR_ARG, an empty action vector
// -> VLA_ERR_PREDICT, anything thrown -> VLA_ERR_EXCEPTION, results malloc'd so
// callers may free() them).

#include "vla.h"
#include "vla_serve.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "model.h"

struct vla_model {
    vla::Model* m = nullptr;
};

namespace {

vla::Inputs to_inputs(const vla_inputs& in) {
    vla::Inputs ci;
    ci.precomputed_img_emb = in.precomputed_img_emb;
    ci.n_img_views = in.n_img_views;
    ci.lang_tokens = in.lang_tokens;
    ci.n_lang = in.n_lang;
    ci.state = in.state;
    ci.noise = in.noise;
    ci.timing_detail = in.timing_detail == VLA_TIMING_PHASE ? vla::TimingDetail::PHASE : vla::TimingDetail::NONE;
    return ci;
}

bool inputs_ok(const vla_inputs& in) {
    if (in.n_images < 0 || in.n_lang < 0 || in.n_img_views < 0) return false;
    if (in.n_images > 0 && !in.images) return false;
    if (in.n_lang > 0 && !in.lang_tokens) return false;
    return true;
}

int32_t give(const std::vector<float>& act, float** out_actions, int64_t* out_n) {
    if (act.empty()) return VLA_ERR_PREDICT;
    float* buf = (float*)std::malloc(act.size() * sizeof(float));
    if (!buf) return VLA_ERR_EXCEPTION;
    std::memcpy(buf, act.data(), act.size() * sizeof(float));
    *out_actions = buf;
    *out_n = (int64_t)act.size();
    return VLA_OK;
}

}  // namespace

extern "C" {

int32_t vla_abi_version(void) { return VLA_ABI_VERSION; }

vla_model* vla_model_load(const char* mmproj_path, const char* ckpt_path, const char* config_path) {
    if (!ckpt_path) return nullptr;
    try {
        vla::Model* m = vla::model_load(mmproj_path ? mmproj_path : "", ckpt_path, config_path ? config_path : "");
        if (!m) return nullptr;
        vla_model* h = new (std::nothrow) vla_model();
        if (!h) {
            vla::model_free(m);
            return nullptr;
        }
        h->m = m;
        return h;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla: load failed: %s\n", e.what());
        return nullptr;
    } catch (...) {
        return nullptr;
    }
}

void vla_model_free(vla_model* h) {
    if (!h) return;
    try {
        vla::model_free(h->m);
    } catch (...) {
    }
    delete h;
}

int32_t vla_model_config(const vla_model* h, vla_config* out) {
    if (!h || !h->m || !out) return VLA_ERR_ARG;
    try {
        const vla::Config& c = vla::model_config(h->m);
        std::memset(out, 0, sizeof(*out));
        out->n_img = c.n_img; out->n_lang = c.n_lang; out->n_state = c.n_state;
        out->n_prefix = c.n_prefix; out->n_suffix = c.n_suffix; out->n_full = c.n_full;
        out->hidden = c.hidden; out->expert_h = c.expert_h;
        out->intermediate = c.intermediate; out->expert_inter = c.expert_inter;
        out->n_q_heads = c.n_q_heads; out->n_kv_heads = c.n_kv_heads; out->head_dim = c.head_dim;
        out->q_full_dim = c.q_full_dim; out->kv_full_dim = c.kv_full_dim; out->n_layers = c.n_layers;
        out->self_attn_every_n = c.self_attn_every_n;
        out->max_state_dim = c.max_state_dim; out->max_action_dim = c.max_action_dim;
        out->real_state_dim = c.real_state_dim; out->real_action_dim = c.real_action_dim;
        out->norm_eps = c.norm_eps; out->min_period = c.min_period; out->max_period = c.max_period;
        out->num_steps = c.num_steps; out->rms_eps = c.rms_eps;
        out->rope_n_dims = c.rope_n_dims; out->rope_mode = c.rope_mode; out->rope_freq_base = c.rope_freq_base;
        out->denormalized = c.denormalized ? 1 : 0;
        return VLA_OK;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int32_t vla_predict(vla_model* h, const vla_inputs* in, float** out_actions, int64_t* out_n) {
    if (!h || !h->m || !in || !out_actions || !out_n) return VLA_ERR_ARG;
    *out_actions = nullptr;
    *out_n = 0;
    if (!inputs_ok(*in)) return VLA_ERR_ARG;
    try {
        return give(vla::predict(h->m, to_inputs(*in)), out_actions, out_n);
    } catch (const std::invalid_argument& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return VLA_ERR_ARG;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla: predict failed: %s\n", e.what());
        return VLA_ERR_EXCEPTION;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

void vla_free_actions(float* actions) { std::free(actions); }

int32_t vla_last_stats(const vla_model* h, vla_stats* out) {
    if (!h || !h->m || !out) return VLA_ERR_ARG;
    const vla::Stats& s = vla::last_stats(h->m);
    out->ms_total = s.ms_total; out->ms_vision = s.ms_vision; out->ms_inference = s.ms_inference;
    out->ms_prefill = s.ms_prefill; out->ms_denoise = s.ms_denoise;
    return VLA_OK;
}

int32_t vla_prefill_batch(vla_model* h, const vla_inputs* in, int32_t batch) {
    if (!h || !h->m || !in || batch <= 0) return VLA_ERR_ARG;
    try {
        std::vector<vla::Inputs> ci((size_t)batch);
        for (int32_t b = 0; b < batch; ++b) {
            if (!inputs_ok(in[b])) return VLA_ERR_ARG;
            ci[b] = to_inputs(in[b]);
        }
        h->m->arch->prefill(ci.data(), batch);
        return VLA_OK;
    } catch (const std::invalid_argument& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return VLA_ERR_ARG;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla: prefill failed: %s\n", e.what());
        return VLA_ERR_EXCEPTION;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int32_t vla_denoise_async(vla_model* h, int32_t chunks, void* stream) {
    if (!h || !h->m || chunks <= 0) return VLA_ERR_ARG;
    try {
        h->m->arch->denoise(chunks, stream);
        return VLA_OK;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla: denoise failed: %s\n", e.what());
        return VLA_ERR_EXCEPTION;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int32_t vla_denoise_steps_async(vla_model* h, int32_t n_steps, void* stream) {
    if (!h || !h->m || n_steps <= 0) return VLA_ERR_ARG;
    try {
        h->m->arch->denoise_steps(n_steps, stream);
        return VLA_OK;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla: denoise failed: %s\n", e.what());
        return VLA_ERR_EXCEPTION;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int32_t vla_fetch_actions(vla_model* h, float** out_actions, int64_t* out_n) {
    if (!h || !h->m || !out_actions || !out_n) return VLA_ERR_ARG;
    *out_actions = nullptr;
    *out_n = 0;
    try {
        return give(h->m->arch->fetch(), out_actions, out_n);
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int32_t vla_predict_batch(vla_model* h, const vla_inputs* in, int32_t batch, float** out_actions, int64_t* out_n) {
    if (!out_actions || !out_n) return VLA_ERR_ARG;
    int32_t rc = vla_prefill_batch(h, in, batch);
    if (rc != VLA_OK) return rc;
    rc = vla_denoise_async(h, 1, nullptr);
    if (rc != VLA_OK) return rc;
    return vla_fetch_actions(h, out_actions, out_n);
}

int32_t vla_profile_begin(vla_model* h) {
    if (!h || !h->m) return VLA_ERR_ARG;
    try {
        h->m->arch->profile_begin();
        return VLA_OK;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int64_t vla_profile_end(vla_model* h, char* json_out, int64_t cap) {
    if (!h || !h->m || !json_out || cap <= 0) return VLA_ERR_ARG;
    try {
        const std::string s = h->m->arch->profile_end();
        // too small: the profile is kept, and the size comes back below every vla_status code
        if ((int64_t)s.size() + 1 > cap) return -16 - (int64_t)(s.size() + 1);
        std::memcpy(json_out, s.c_str(), s.size() + 1);
        h->m->arch->profile_discard();
        return (int64_t)s.size();
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla: profile failed: %s\n", e.what());
        return VLA_ERR_EXCEPTION;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

int64_t vla_model_n_actions(const vla_model* h) {
    if (!h || !h->m) return 0;
    return h->m->arch->n_actions();
}

}  // extern "C"
