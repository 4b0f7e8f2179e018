/* Model-level C ABI, version 1.
 *
 * Binary-compatible with the reference's include/vla.h (ABI v1,
 * /root/reference include/vla.h:37-161): the same opaque handle, status codes,
 * struct layouts (field order and types are the contract; the ctypes mirror in
 * the reference's bindings/python/vla_cpp/_ffi.py:124-163 binds these) and the
 * same seven entry points, so a program linked against the reference's libvla
 * can be pointed at this library.  Behaviour behind the ABI: the handle drives
 * the MI355X action-expert attention path on one GPU; checkpoints are the
 * reference's GGUF files (the tensors on the path are taken from them) or the
 * flat "VLAW" files written by vla.cpp_amd/checkpoint.py.
 *
 * Ownership rules are the reference's: load pairs with free, predict pairs with
 * vla_free_actions, every pointer inside vla_inputs is only borrowed for the
 * duration of the call, and one vla_predict runs at a time per handle.
 */
#ifndef VLA_H
#define VLA_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VLA_API __attribute__((visibility("default")))

#define VLA_ABI_VERSION 1

typedef struct vla_model vla_model;

/* Status codes, pixel formats and timing detail: the reference's values (include/vla.h:41-57). */
typedef enum { VLA_OK = 0, VLA_ERR_ARG = -1, VLA_ERR_PREDICT = -2, VLA_ERR_EXCEPTION = -3 } vla_status;
/* VLA_ERR_ARG: null handle or malformed inputs; VLA_ERR_PREDICT: the engine produced no actions;
 * VLA_ERR_EXCEPTION: a C++ exception stopped at the boundary. */
typedef enum { VLA_PIXEL_U8 = 0, VLA_PIXEL_F32_RGB_01 = 1 } vla_pixel_format;
typedef enum { VLA_TIMING_NONE = 0, VLA_TIMING_PHASE = 1 } vla_timing_detail;

/* Resolved hyper-parameters (reference: vla::Config, src/model.h:48-87).  Field order and
 * types are the ABI; fields of one type that follow each other share a declaration. */
typedef struct {
    int64_t n_img, n_lang, n_state, n_prefix, n_suffix, n_full;                 /* token counts */
    int64_t hidden, expert_h, intermediate, expert_inter;                        /* widths */
    int64_t n_q_heads, n_kv_heads, head_dim, q_full_dim, kv_full_dim, n_layers;  /* attention geometry */
    int32_t self_attn_every_n;
    int64_t max_state_dim, max_action_dim, real_state_dim, real_action_dim;
    float norm_eps;
    double min_period, max_period; /* sinusoidal time embedding */
    int32_t num_steps;
    float rms_eps;
    int32_t rope_n_dims, rope_mode;
    float rope_freq_base;
    int32_t denormalized;
} vla_config;

typedef struct {
    const void* data;
    int32_t w, h, format; /* format: vla_pixel_format */
} vla_image;

/* One observation.  This library has no vision tower: precomputed_img_emb
 * ([n_img_views * n_img, hidden] floats) is required and `images` is ignored. */
typedef struct {
    const vla_image* images;
    int32_t n_images;
    const float* precomputed_img_emb;
    int32_t n_img_views;
    const int32_t* lang_tokens;
    int32_t n_lang;
    const float* state; /* max_state_dim floats, or NULL for zeros */
    const float* noise; /* n_actions * max_action_dim floats, or NULL to sample */
    const int32_t* attention_mask;
    int32_t attention_mask_n;
    int32_t timing_detail; /* vla_timing_detail */
} vla_inputs;

/* Milliseconds; the phase fields stay zero unless VLA_TIMING_PHASE was asked for. */
typedef struct {
    float ms_total, ms_vision, ms_inference, ms_prefill, ms_denoise;
} vla_stats;

VLA_API int32_t vla_abi_version(void);

/* mmproj_path and config_path are accepted and ignored; ckpt_path names a GGUF
 * or VLAW file.  NULL on any failure. */
VLA_API vla_model * vla_model_load(const char * mmproj_path, const char * ckpt_path, const char * config_path);

VLA_API void vla_model_free(vla_model * m);

VLA_API int32_t vla_model_config(const vla_model * m, vla_config * out);

/* One observation in, one action chunk out: *out_actions receives *out_n
 * malloc'd floats, row-major [n_actions, max_action_dim], columns past
 * real_action_dim zero. */
VLA_API int32_t vla_predict(vla_model * m, const vla_inputs * in, float ** out_actions, int64_t * out_n);

VLA_API void vla_free_actions(float * actions);

VLA_API int32_t vla_last_stats(const vla_model * m, vla_stats * out);

/* ---- Extensions with no counterpart in the reference (it serves batch 1
 * only, src/serving/server.cpp:340-558): independent observations batched, and
 * the two phases of a prediction exposed separately so a server or a benchmark
 * can keep the prefix KV resident and time the denoise loop alone. ---- */

/* Builds the prefix KV for `batch` observations and stages state/noise. */
VLA_API int32_t vla_prefill_batch(vla_model * m, const vla_inputs * in, int32_t batch);
/* Runs `chunks` action chunks (num_steps denoise steps each; the noise is
 * re-staged before every chunk) on `stream` (a hipStream_t or NULL), without
 * synchronising. */
VLA_API int32_t vla_denoise_async(vla_model * m, int32_t chunks, void * stream);
/* Same, counted in denoise steps (the step index cycles through the chunk), for
 * timing a given number of steps. */
VLA_API int32_t vla_denoise_steps_async(vla_model * m, int32_t n_steps, void * stream);
/* Synchronises and copies the last chunk's actions:
 * [batch, n_actions, max_action_dim] floats, malloc'd. */
VLA_API int32_t vla_fetch_actions(vla_model * m, float ** out_actions, int64_t * out_n);
/* vla_prefill_batch + one chunk + vla_fetch_actions. */
VLA_API int32_t vla_predict_batch(vla_model * m, const vla_inputs * in, int32_t batch, float ** out_actions,
                                  int64_t * out_n);

/* Per-launch timing for benchmarks (no counterpart in the reference, whose vla-bench times
 * whole predict() calls, src/serving/vla-bench.cpp:159-195).  Between begin and end, prefill
 * and denoise calls record a HIP event after every kernel launch and denoise launches eagerly
 * instead of replaying its graph.  vla_profile_end synchronises, disarms and writes a JSON
 * object {"phase.label": {"us": average, "launches": count}, ...} -- the time from the
 * previous launch's end to this launch's end on the stream, i.e. the launch in its real
 * sequence, cold caches and dependent-launch gap included.  Returns the string length, or a
 * vla_status (-1 .. -3), or, when cap is too small, -16 - (the size needed): the profile is then
 * kept (nothing is disarmed) and the call can be repeated with a larger buffer. */
VLA_API int32_t vla_profile_begin(vla_model * m);
VLA_API int64_t vla_profile_end(vla_model * m, char * json_out, int64_t cap);

#ifdef __cplusplus
}
#endif

#endif /* VLA_H */
