/* Serving boundary of libvla.so: the reference server's wire format and request checks
 * without its transport.
 *
 * The reference serves `vla.PredictRequest` / `vla.PredictResponse` protobuf messages
 * (src/serving/vla.proto) over a ZeroMQ REP socket, one request at a time
 * (src/serving/server.cpp:296-560).  ZeroMQ and libprotobuf are not part of this library;
 * what is here is what sits between the socket and the engine: a self-contained proto3
 * codec for the two messages, the server's request validation with its error strings, and
 * the step the single-threaded loop cannot do -- answering several queued requests with
 * one batched engine call.  A transport loop (ROUTER / REP, gRPC, shared memory) collects
 * the request frames that are waiting, passes them here and sends the returned frames back.
 */
#ifndef VLA_SERVE_H
#define VLA_SERVE_H

#include <stdint.h>

#include "vla.h"

#ifdef __cplusplus
extern "C" {
#endif

#define VLA_SERVE_API __attribute__((visibility("default")))

/* Answers `n` serialized PredictRequest frames with `n` serialized PredictResponse frames.
 * Every request is parsed and checked as in src/serving/server.cpp:383-509 (same order, same
 * error texts; a request that fails gets a response carrying `error` and its request_id,
 * request_id 0 if it could not be parsed).  Requests that pass are grouped by (image views,
 * language length) and each group runs as one vla_predict_batch call; a response carries
 * request_id, action_chunk [chunk_size x action_dim], chunk_size, action_dim and the
 * latencies of the engine call that served it (src/serving/server.cpp:543-557).
 * Requests must carry precomputed_img_emb: this library has no vision tower, `images` alone is
 * answered with an error.
 * resp[i] is malloc'd (free it with vla_serve_free), resp_len[i] its length.
 * Returns VLA_OK when every frame got a response (including error responses),
 * VLA_ERR_ARG for NULL arguments or n < 0; like vla_predict, one call at a time per handle. */
VLA_SERVE_API int32_t vla_serve_requests(vla_model* m, int32_t n, const uint8_t* const* req, const int64_t* req_len,
                                         uint8_t** resp, int64_t* resp_len);
VLA_SERVE_API void vla_serve_free(uint8_t* frame); /* NULL is fine */

/* Client side of the same codec (what eval/client/vla_cpp_client.py does with the generated
 * protobuf classes): serialize a request from plain arrays, read a response back.
 * vla_wire_encode_request returns a malloc'd frame (vla_serve_free) and its length, NULL on
 * allocation failure; absent arrays are NULL / 0. */
VLA_SERVE_API uint8_t* vla_wire_encode_request(uint64_t request_id, const int32_t* lang_tokens, int32_t n_lang,
                                               const float* state, int32_t n_state, const float* noise, int32_t n_noise,
                                               const float* img_emb, int64_t n_img_emb, uint32_t n_views, int64_t* out_len);

typedef struct {
    uint64_t request_id;
    uint32_t chunk_size, action_dim;
    float latency_ms_total, latency_ms_inference, latency_ms_prefill, latency_ms_denoise, latency_ms_vision;
    int64_t n_actions;   /* floats in action_chunk */
    int64_t error_len;   /* bytes in error, 0 = success */
} vla_wire_response;

/* Parses a PredictResponse frame.  actions (capacity cap_actions floats) and error (capacity
 * cap_error bytes, NUL-terminated when it fits) may be NULL to query the sizes first.
 * Returns VLA_OK, or VLA_ERR_ARG for a malformed frame or too small a buffer. */
VLA_SERVE_API int32_t vla_wire_decode_response(const uint8_t* frame, int64_t len, vla_wire_response* out, float* actions,
                                               int64_t cap_actions, char* error, int64_t cap_error);

/* Action rows per chunk of a loaded model (chunk_size of the responses; the noise of a
 * request is chunk_size * max_action_dim floats). */
VLA_SERVE_API int64_t vla_model_n_actions(const vla_model* m);

#ifdef __cplusplus
}
#endif
#endif
