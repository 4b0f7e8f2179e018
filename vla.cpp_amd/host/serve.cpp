// Request handling of the reference server (src/serving/server.cpp:383-560) behind a C ABI,
// with the queued requests of one call answered by batched engine calls.  Built on the
// public model API only (include/vla.h); the codec is wire.h.
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <utility>

#include "vla_serve.h"
#include "wire.h"

namespace {

using vla::wire::PredictRequest;
using vla::wire::PredictResponse;

int find_non_finite(const std::vector<float>& v) {
    for (size_t i = 0; i < v.size(); ++i)
        if (!std::isfinite(v[i])) return (int)i;
    return -1;
}

// The checks of src/serving/server.cpp:393-509, in its order and with its texts; empty = accepted.
std::string check_request(const PredictRequest& q, const vla_config& cfg, int64_t n_actions) {
    char buf[192];
    if (q.n_images < 1 && q.precomputed_img_emb.empty()) return "PredictRequest must contain images or precomputed_img_emb";
    if (q.n_images > 16) return "too many image views (max 16)";
    if (q.lang_tokens.size() < 1 || (int64_t)q.lang_tokens.size() > cfg.n_lang) {
        std::snprintf(buf, sizeof(buf), "lang_tokens length %d out of range [1, %lld]", (int)q.lang_tokens.size(), (long long)cfg.n_lang);
        return buf;
    }
    for (size_t t = 0; t < q.lang_tokens.size(); ++t)
        if (q.lang_tokens[t] < 0) {
            std::snprintf(buf, sizeof(buf), "lang_tokens[%d] = %d is negative", (int)t, q.lang_tokens[t]);
            return buf;
        }
    if ((int64_t)q.state.size() != cfg.max_state_dim) {
        std::snprintf(buf, sizeof(buf), "state length %d != expected %lld", (int)q.state.size(), (long long)cfg.max_state_dim);
        return buf;
    }
    const int expected_noise_n = (int)(n_actions * cfg.max_action_dim);
    if (!q.noise.empty() && (int)q.noise.size() != expected_noise_n) {
        std::snprintf(buf, sizeof(buf), "noise length %d != 0 or %d (chunk_size * action_dim)", (int)q.noise.size(), expected_noise_n);
        return buf;
    }
    if (q.precomputed_img_emb.empty())
        return "images need the vision tower, which this library does not include; send precomputed_img_emb";
    const int n_views = (int)q.precomputed_img_emb_n_views;
    const int64_t expected = cfg.n_img * cfg.hidden * (int64_t)n_views;
    if (n_views < 1 || (int64_t)q.precomputed_img_emb.size() != expected) {
        std::snprintf(buf, sizeof(buf), "precomputed_img_emb size %d != %lld (n_views=%d * n_img_per_view=%lld * hidden=%lld)",
                      (int)q.precomputed_img_emb.size(), (long long)expected, n_views, (long long)cfg.n_img, (long long)cfg.hidden);
        return buf;
    }
    int bad = find_non_finite(q.precomputed_img_emb);
    if (bad >= 0) {
        std::snprintf(buf, sizeof(buf), "precomputed_img_emb[%d] = %g is not finite (NaN/Inf)", bad, q.precomputed_img_emb[bad]);
        return buf;
    }
    bad = find_non_finite(q.state);
    if (bad >= 0) {
        std::snprintf(buf, sizeof(buf), "state[%d] = %g is not finite (NaN/Inf)", bad, q.state[bad]);
        return buf;
    }
    bad = find_non_finite(q.noise);
    if (bad >= 0) {
        std::snprintf(buf, sizeof(buf), "noise[%d] = %g is not finite (NaN/Inf)", bad, q.noise[bad]);
        return buf;
    }
    return std::string();
}

uint8_t* to_frame(const std::string& body, int64_t* len) {
    uint8_t* f = (uint8_t*)std::malloc(body.size() ? body.size() : 1);
    if (!f) return nullptr;
    if (!body.empty()) std::memcpy(f, body.data(), body.size());
    *len = (int64_t)body.size();
    return f;
}

std::string error_response(uint64_t rid, const std::string& msg) {
    PredictResponse r;
    r.request_id = rid;
    r.error = msg;
    return vla::wire::encode_response(r);
}

}  // namespace

extern "C" {

void vla_serve_free(uint8_t* frame) { std::free(frame); }

int32_t vla_serve_requests(vla_model* m, int32_t n, const uint8_t* const* req, const int64_t* req_len, uint8_t** resp,
                           int64_t* resp_len) {
    if (!m || n < 0 || (n > 0 && (!req || !req_len || !resp || !resp_len))) return VLA_ERR_ARG;
    try {
        vla_config cfg;
        if (vla_model_config(m, &cfg) != VLA_OK) return VLA_ERR_ARG;
        const int64_t n_actions = vla_model_n_actions(m);
        std::vector<PredictRequest> q((size_t)n);
        std::vector<std::string> body((size_t)n);
        std::vector<char> answered((size_t)n, 0);
        // (image views, language length) -> indices: a batch shares both
        std::map<std::pair<int, int>, std::vector<int>> groups;
        for (int i = 0; i < n; ++i) {
            if (!req[i] || req_len[i] < 0 || !vla::wire::parse_request(req[i], (size_t)req_len[i], q[i])) {
                std::fprintf(stderr, "vla-serve: PredictRequest parse failed (size=%lld)\n", (long long)(req[i] ? req_len[i] : -1));
                body[i] = error_response(0, "request parse failed");
                answered[i] = 1;
                continue;
            }
            const std::string err = check_request(q[i], cfg, n_actions);
            if (!err.empty()) {
                body[i] = error_response(q[i].request_id, err);
                answered[i] = 1;
                continue;
            }
            groups[{(int)q[i].precomputed_img_emb_n_views, (int)q[i].lang_tokens.size()}].push_back(i);
        }
        // One engine call for the requests `idx`; fills their bodies and returns the engine's status.
        auto run_group = [&](const std::vector<int>& idx, bool answer_failures) -> int32_t {
            std::vector<vla_inputs> in(idx.size());
            for (size_t k = 0; k < idx.size(); ++k) {
                const PredictRequest& r = q[(size_t)idx[k]];
                vla_inputs& v = in[k];
                std::memset(&v, 0, sizeof(v));
                v.precomputed_img_emb = r.precomputed_img_emb.data();
                v.n_img_views = (int32_t)r.precomputed_img_emb_n_views;
                v.lang_tokens = r.lang_tokens.data();
                v.n_lang = (int32_t)r.lang_tokens.size();
                v.state = r.state.data();
                v.noise = r.noise.empty() ? nullptr : r.noise.data();
                v.attention_mask = r.attention_mask.empty() ? nullptr : reinterpret_cast<const int32_t*>(r.attention_mask.data());
                v.attention_mask_n = (int32_t)r.attention_mask.size();
                v.timing_detail = VLA_TIMING_PHASE;
            }
            float* act = nullptr;
            int64_t act_n = 0;
            // prefix build, then the denoise loop and the copy back, timed as the reference's
            // PHASE detail does for one request (src/models/smolvla.cpp:1898-1912)
            using clk = std::chrono::steady_clock;
            const auto ms = [](clk::time_point x, clk::time_point y) { return std::chrono::duration<float, std::milli>(y - x).count(); };
            const auto t0 = clk::now();
            int32_t rc = vla_prefill_batch(m, in.data(), (int32_t)in.size());
            const auto t1 = clk::now();
            if (rc == VLA_OK) rc = vla_denoise_async(m, 1, nullptr);
            if (rc == VLA_OK) rc = vla_fetch_actions(m, &act, &act_n);
            const auto t2 = clk::now();
            vla_stats st;
            std::memset(&st, 0, sizeof(st));
            st.ms_total = st.ms_inference = ms(t0, t2);
            st.ms_prefill = ms(t0, t1);
            st.ms_denoise = ms(t1, t2);
            const int64_t per = (int64_t)idx.size() ? act_n / (int64_t)idx.size() : 0;
            const bool failed = rc != VLA_OK || !act || per != n_actions * cfg.max_action_dim;
            if (failed && !answer_failures) {
                vla_free_actions(act);
                return rc != VLA_OK ? rc : VLA_ERR_PREDICT;
            }
            for (size_t k = 0; k < idx.size(); ++k) {
                const int i = idx[k];
                if (failed) {
                    body[(size_t)i] = error_response(q[(size_t)i].request_id, "predict failed");
                } else {
                    PredictResponse r;
                    r.request_id = q[(size_t)i].request_id;
                    r.action_chunk.assign(act + (int64_t)k * per, act + (int64_t)(k + 1) * per);
                    r.chunk_size = (uint32_t)n_actions;
                    r.action_dim = (uint32_t)cfg.max_action_dim;
                    r.ms_total = st.ms_total;
                    r.ms_vision = st.ms_vision;
                    r.ms_inference = st.ms_inference;
                    r.ms_prefill = st.ms_prefill;
                    r.ms_denoise = st.ms_denoise;
                    body[(size_t)i] = vla::wire::encode_response(r);
                }
                answered[(size_t)i] = 1;
            }
            vla_free_actions(act);
            return failed ? (rc != VLA_OK ? rc : VLA_ERR_PREDICT) : VLA_OK;
        };
        for (const auto& grp : groups) {
            const std::vector<int>& idx = grp.second;
            // A request the engine itself rejects (an out-of-vocabulary token, say) fails the batched
            // call for everyone in it; the reference serves one request per predict, so only the
            // offender may see an error: on a rejection the members are served one by one.
            if (idx.size() > 1) {
                if (run_group(idx, false) == VLA_OK) continue;
                for (int i : idx) (void)run_group(std::vector<int>{i}, true);
            } else {
                (void)run_group(idx, true);
            }
        }
        for (int i = 0; i < n; ++i) {
            resp[i] = to_frame(body[(size_t)i], &resp_len[i]);
            if (!resp[i]) {
                for (int k = 0; k < i; ++k) {
                    std::free(resp[k]);
                    resp[k] = nullptr;
                }
                return VLA_ERR_EXCEPTION;
            }
        }
        return VLA_OK;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "vla-serve: %s\n", e.what());
        return VLA_ERR_EXCEPTION;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

uint8_t* vla_wire_encode_request(uint64_t request_id, const int32_t* lang_tokens, int32_t n_lang, const float* state, int32_t n_state,
                                 const float* noise, int32_t n_noise, const float* img_emb, int64_t n_img_emb, uint32_t n_views,
                                 int64_t* out_len) {
    if (!out_len || n_lang < 0 || n_state < 0 || n_noise < 0 || n_img_emb < 0) return nullptr;
    try {
        PredictRequest q;
        q.request_id = request_id;
        if (lang_tokens) q.lang_tokens.assign(lang_tokens, lang_tokens + n_lang);
        if (state) q.state.assign(state, state + n_state);
        if (noise) q.noise.assign(noise, noise + n_noise);
        if (img_emb) q.precomputed_img_emb.assign(img_emb, img_emb + n_img_emb);
        q.precomputed_img_emb_n_views = n_views;
        return to_frame(vla::wire::encode_request(q), out_len);
    } catch (...) {
        return nullptr;
    }
}

int32_t vla_wire_decode_response(const uint8_t* frame, int64_t len, vla_wire_response* out, float* actions, int64_t cap_actions,
                                 char* error, int64_t cap_error) {
    if (!frame || len < 0 || !out) return VLA_ERR_ARG;
    try {
        PredictResponse r;
        if (!vla::wire::parse_response(frame, (size_t)len, r)) return VLA_ERR_ARG;
        out->request_id = r.request_id;
        out->chunk_size = r.chunk_size;
        out->action_dim = r.action_dim;
        out->latency_ms_total = r.ms_total;
        out->latency_ms_inference = r.ms_inference;
        out->latency_ms_prefill = r.ms_prefill;
        out->latency_ms_denoise = r.ms_denoise;
        out->latency_ms_vision = r.ms_vision;
        out->n_actions = (int64_t)r.action_chunk.size();
        out->error_len = (int64_t)r.error.size();
        if (actions) {
            if (cap_actions < out->n_actions) return VLA_ERR_ARG;
            if (out->n_actions) std::memcpy(actions, r.action_chunk.data(), r.action_chunk.size() * sizeof(float));
        }
        if (error) {
            if (cap_error < out->error_len) return VLA_ERR_ARG;
            if (out->error_len) std::memcpy(error, r.error.data(), r.error.size());
            if (cap_error > out->error_len) error[out->error_len] = 0;
        }
        return VLA_OK;
    } catch (...) {
        return VLA_ERR_EXCEPTION;
    }
}

}  // extern "C"
