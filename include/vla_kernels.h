/* Kernel-level C ABI of the MI355X (gfx950) action-expert attention path.
 *
 * Conventions (those of the reference's in-tree kernel layer,
 * src/kernels/bitvla/bitvla_lm_cuda.h:28-30): extern "C", device pointers,
 * plain ints, the stream passed explicitly as the last argument, no device
 * synchronisation inside.  Unlike the reference's void launchers every entry
 * point returns a vla_kstatus, so a bad shape is reported instead of aborting
 * the process (the reference aborts, src/kernels/bitvla/bitnet_kernels.cu:22-29).
 *
 * bf16 values are raw 16-bit patterns (uint16_t); `dtype` arguments take
 * VLA_DT_F32 or VLA_DT_BF16.  "token-major" is [token][head][head_dim], i.e.
 * ggml's [head_dim, n_heads, n_tokens] with ne0 innermost, the layout the
 * reference's projections produce (src/models/smolvla.cpp:825-827).
 *
 * Resident KV cache layout (one K and one V buffer per layer):
 *     K  : [batch][n_kv_heads][t_max][head_dim]
 *     V^T: [batch][n_kv_heads][head_dim][t_max]        (t_max % 8 == 0)
 * The prefix occupies tokens [0, P) and is written once per observation; the
 * action suffix of every denoise step overwrites tokens [P, P+S) in place.
 */
#ifndef VLA_KERNELS_H
#define VLA_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VLA_KAPI __attribute__((visibility("default")))

typedef void* vla_stream_t; /* a hipStream_t */

/* VLA_DT_BF16_P2 is accepted by vla_attn_prefix_suffix only: bf16 storage as VLA_DT_BF16,
 * with the softmax probabilities carried as two bf16 terms (about 16 mantissa bits) through
 * the P.V product, at twice the MFMA work of that product. */
typedef enum { VLA_DT_F32 = 0, VLA_DT_BF16 = 1, VLA_DT_BF16_P2 = 2 } vla_dtype;

typedef enum {
    VLA_K_OK = 0,
    VLA_K_ERR_ARG = -1,    /* null pointer or negative size */
    VLA_K_ERR_SHAPE = -2,  /* a size the kernels do not support (alignment, head_dim, ...) */
    VLA_K_ERR_LAUNCH = -3, /* hipGetLastError() after the launch */
    VLA_K_ERR_WORKSPACE = -4, /* the workspace handed in (or the fixed one) is too small for the shape */
} vla_kstatus;

/* Suffix-block mask generated inside the attention kernel (the reference builds
 * these on the host as additive 0/-inf matrices and uploads them):
 *   NONE          pi0.5 / GR00T DiT / BitVLA: every key visible.
 *   CAUSAL_SUFFIX SmolVLA mask_full (src/models/smolvla.cpp:1651-1664):
 *                 suffix key j (>= n_prefix) is hidden from query i when
 *                 j - n_prefix > i.
 *   PI0_STATE     pi0 full mask (src/models/pi0.cpp:638-653): query 0 (the
 *                 state token) sees only suffix key 0; other queries see all.
 * In every kind, prefix keys in [pad_start, pad_end) are hidden (SmolVLA's
 * padded language tokens); pass pad_start == pad_end for none. */
typedef enum { VLA_MASK_NONE = 0, VLA_MASK_CAUSAL_SUFFIX = 1, VLA_MASK_PI0_STATE = 2 } vla_mask_kind;

/* ---------------------------------------------------------------- KV cache */

/* In-place append, replacing ggml_concat(cached_K, k_rope, 2) /
 * ggml_concat(cached_V, v_h, 2) (src/models/smolvla.cpp:832-833,
 * src/models/pi0.cpp:198-201, src/models/pi05.cpp:255-256).  k_src / v_src are
 * token-major [batch][n_tok][n_kv_heads][head_dim]; they land at tokens
 * [tok_offset, tok_offset + n_tok) of the cache.  Either pair may be NULL. */
VLA_KAPI int vla_kv_append(void* k_cache, void* vt_cache, const void* k_src, const void* v_src, int dtype,
                           int batch, int n_kv_heads, int head_dim, int t_max, int tok_offset, int n_tok,
                           vla_stream_t stream);

/* Inverse of vla_kv_append: reads tokens [tok_offset, tok_offset + n_tok) back
 * into token-major buffers (the [D, Hkv, T] tensor the reference's concat
 * would have produced). */
VLA_KAPI int vla_kv_gather(const void* k_cache, const void* vt_cache, void* k_dst, void* v_dst, int dtype,
                           int batch, int n_kv_heads, int head_dim, int t_max, int tok_offset, int n_tok,
                           vla_stream_t stream);

/* --------------------------------------------------------------- RoPE, norms */

/* Host helper: cos/sin tables [n][head_dim/2] for NeoX RoPE,
 * theta = pos * base^(-2i/D) evaluated in double and rounded once
 * (ggml_rope_ext(..., NEOX, base, freq_scale 1, ext_factor 0, attn_factor 1),
 * src/models/smolvla.cpp:759-766; table form of
 * src/kernels/bitvla/bitvla_lm_cuda.cu:333-342). */
VLA_KAPI int vla_rope_tables_host(const int32_t* pos, int n, int head_dim, double base, float* cos_tab,
                                  float* sin_tab);

/* NeoX rotation in place on a token-major tensor x [n_rows][n_heads][head_dim];
 * row r uses table row r % table_rows (tables [table_rows][head_dim/2]). */
VLA_KAPI int vla_rope_neox(void* x, const float* cos_tab, const float* sin_tab, int dtype, int n_rows,
                           int table_rows, int n_heads, int head_dim, vla_stream_t stream);

/* y = rms_norm(x) * w (src/models/smolvla.cpp:820, src/models/pi0.cpp:170).
 * x, y [M][K] in `dtype`; w [K] in `dtype` or NULL. */
VLA_KAPI int vla_rms_norm(const void* x, const void* w, void* y, int dtype, int M, int K, float eps,
                          vla_stream_t stream);

/* adaLN: y = xn + xn*sc + sh with xn = layer_norm(x) without affine
 * (src/layers/norm.h:37-46, used by src/modules/dit_head.cpp:111).  sc, sh are
 * fp32 [K], shared by all rows. */
VLA_KAPI int vla_adaln(const void* x, const float* sc, const float* sh, void* y, int dtype, int M, int K,
                       float eps, vla_stream_t stream);

/* build_adarms (src/models/pi05.cpp:208-223) with (scale, shift) already evaluated for the
 * step: y = n + n * scale + shift, n = x * rsqrt(mean x^2 + eps) (no centring, no weight).
 * scale, shift fp32 [K]. */
VLA_KAPI int vla_adarms(const void* x, const float* sc, const float* sh, void* y, int dtype, int M, int K, float eps,
                        vla_stream_t stream);

/* ---------------------------------------------------------------- projections */

/* y[M][N] = x[M][K] . W[N][K]^T (+ bias[N], fp32) (+ residual[M][N]), the
 * ggml_mul_mat shape rule (src/act_dtype.h:62-76; src/layers/linear.h:24-27;
 * the Wo + residual of src/models/smolvla.cpp:843, src/models/pi0.cpp:224-225).
 * x, W in `dtype`; residual and y in `out_dtype`; fp32 accumulation. */
VLA_KAPI int vla_linear(const void* x, const void* W, const float* bias, const void* residual, void* y,
                        int dtype, int out_dtype, int M, int N, int K, vla_stream_t stream);

/* Activations of the FFN halves (ggml_silu, ggml_gelu in its tanh form) and of the DiT head's
 * state encoder / action decoder (ggml_relu, src/modules/action_expert.cpp:41-59). */
enum { VLA_ACT_NONE = 0, VLA_ACT_SILU = 1, VLA_ACT_GELU = 2, VLA_ACT_RELU = 3 };

/* vla_linear with an activation between the bias and the residual:
 * y = act(x W^T + b) [+ residual]; the first half of ffn_gelu
 * (src/layers/ffn.h:24-27, used by DitHead::block, src/modules/dit_head.cpp:133). */
VLA_KAPI int vla_linear_act(const void* x, const void* W, const float* bias, const void* residual, void* y, int dtype,
                            int out_dtype, int M, int N, int K, int act, vla_stream_t stream);

/* y = residual + col_gate * (x W^T + b): the gated residual adds of the adaRMS layers,
 * h1 = x + o_out * gate_attn and h = h1 + mlp_out * gate_ffn (src/models/pi05.cpp:273, 281).
 * col_gate fp32 [N] (one factor per output column, the same for every row). */
VLA_KAPI int vla_linear_gated(const void* x, const void* W, const float* bias, const float* col_gate,
                              const void* residual, void* y, int dtype, int out_dtype, int M, int N, int K,
                              vla_stream_t stream);

/* Gated FFN input half in one launch: y[M][I] = act(x Wg^T + bg) * (x Wu^T + bu), replacing
 * mm_w(Wgate) -> ggml_silu / ggml_gelu -> mm_w(Wup) -> ggml_mul (src/models/smolvla.cpp:845-847,
 * src/models/pi0.cpp:227-230, src/layers/ffn.h:35-40).
 *   W_gate_up [2 I][K]: the I gate rows, then the I up rows; bias fp32 [2 I] in the same order or NULL
 *   I a multiple of 32
 *   rms_eps >= 0: the RMSNorm in front of the FFN is taken inside the launch as in
 *     vla_rmsnorm_attn_qkv_rope (rows scaled by rsqrt(mean x^2 + eps), norm weight folded
 *     into both halves of W_gate_up with vla_fold_norm_weight_host; bf16, K % 16 == 0,
 *     else VLA_K_ERR_SHAPE); rms_eps < 0: x is used as it is. */
VLA_KAPI int vla_glu_linear(const void* x, const void* W_gate_up, const float* bias, void* y, int dtype, int out_dtype,
                            int M, int I, int K, int act, float rms_eps, vla_stream_t stream);

/* Fused QKV projection + RoPE + KV append for M = batch*S suffix (or prefix)
 * rows: replaces mm_w(Wq/Wk/Wv) -> reshape -> rope_q_or_k -> ggml_concat
 * (src/models/smolvla.cpp:821-833, src/models/pi0.cpp:174-201,
 * src/modules/dit_head.cpp:113-119).
 *   W    [n_q_heads*D + nk*D + nv*D][K] rows ordered Q, K, V, where
 *        nk = has_k ? n_kv_heads : 0 and nv = has_v ? n_kv_heads : 0
 *   bias fp32 over the same rows, or NULL
 *   cos/sin [S][D/2] (row m uses m % S) or NULL for no rotation (V is never
 *        rotated)
 *   q_out [M][n_q_heads*D] token-major in `dtype` (ignored if n_q_heads == 0)
 *   K rows go to k_cache, V rows to vt_cache at token tok_offset + (m % S) of
 *   batch m / S. */
VLA_KAPI int vla_attn_qkv_rope(const void* x, const void* W, const float* bias, int dtype, int M, int K, int S,
                               int n_q_heads, int n_kv_heads, int has_k, int has_v, int head_dim,
                               const float* cos_tab, const float* sin_tab, void* q_out, void* k_cache,
                               void* vt_cache, int t_max, int tok_offset, vla_stream_t stream);

/* The same launch with the layer's RMSNorm taken inside it: replaces build_norm ->
 * mm_w(Wq/Wk/Wv) -> rope -> concat (src/models/smolvla.cpp:815-833,
 * src/models/pi0.cpp:170-201).  x is the un-normalised residual stream; row m of
 * the projection is scaled by rsqrt(mean_k x[m][k]^2 + rms_eps) before bias and
 * rotation, and the norm weight is expected inside W_folded
 * (W_folded[n][k] = W[n][k] * g[k], vla_fold_norm_weight_host).  bf16 only, K a
 * multiple of 16 and 16-byte aligned operands; VLA_K_ERR_SHAPE otherwise (use
 * vla_rms_norm + vla_attn_qkv_rope then). */
VLA_KAPI int vla_rmsnorm_attn_qkv_rope(const void* x, const void* W_folded, const float* bias, int dtype, int M, int K,
                                       int S, int n_q_heads, int n_kv_heads, int has_k, int has_v, int head_dim,
                                       const float* cos_tab, const float* sin_tab, void* q_out, void* k_cache,
                                       void* vt_cache, int t_max, int tok_offset, float rms_eps, vla_stream_t stream);

/* The same launch with a DiT block's modulated LayerNorm taken inside it: replaces
 * adaln -> mm_w(Wq[/Wk/Wv]) -> rope -> concat (src/layers/norm.h:37-46,
 * src/modules/dit_head.cpp:111-119), xn (1 + scale) + shift with xn = ggml_norm(x).
 * x is the un-normalised residual stream.  The modulation depends on the denoise step
 * only, so it lives in the operands, one set per step (vla_fold_adaln_weight_host):
 *   W_folded[n][k] = W[n][k] (1 + scale[k]),  colsum[n] = sum_k W_folded[n][k],
 *   bias[n] = b[n] + sum_k W[n][k] shift[k]
 * and the launch computes rstd[m] (acc[m][n] - mean[m] colsum[n]) + bias[n] with the
 * mean and variance of row m summed from the operand tiles it multiplies.  bf16 only,
 * K a multiple of 16 and 16-byte aligned operands; VLA_K_ERR_SHAPE otherwise (use
 * vla_adaln + vla_attn_qkv_rope then). */
VLA_KAPI int vla_layernorm_attn_qkv_rope(const void* x, const void* W_folded, const float* colsum, const float* bias,
                                         int dtype, int M, int K, int S, int n_q_heads, int n_kv_heads, int has_k,
                                         int has_v, int head_dim, const float* cos_tab, const float* sin_tab, void* q_out,
                                         void* k_cache, void* vt_cache, int t_max, int tok_offset, float ln_eps,
                                         vla_stream_t stream);

/* A DiT self-attention block's front half in one launch: modulated LayerNorm, the Q / K / V
 * projections and the attention of each observation's S tokens over themselves, replacing
 * adaln -> mm_w(Wq / Wk / Wv) -> attention with enc = nullptr (src/modules/dit_head.cpp:111-125).
 * The block's K and V never reach memory: nothing but this attention reads them.
 *   x [M][K] bf16, M = batch * S rows, observation-major; W_folded [3 * n_heads * head_dim][K]
 *   (Q rows, K rows, V rows), colsum and bias fp32 over the same rows, as for
 *   vla_layernorm_attn_qkv_rope; no rotation, no mask (the DiT block is bidirectional);
 *   out [M][n_heads * head_dim] bf16, token-major as vla_attn_prefix_suffix writes it.
 * Built for head_dim 48, S <= 32, K a multiple of 64 and >= 256, n_heads a multiple of 8, bf16, 16-byte
 * aligned operands; VLA_K_ERR_SHAPE otherwise (use vla_layernorm_attn_qkv_rope +
 * vla_attn_prefix_suffix then). */
VLA_KAPI int vla_layernorm_qkv_self_attention(const void* x, const void* W_folded, const float* colsum, const float* bias,
                                              int dtype, int M, int K, int S, int n_heads, int head_dim, float scale,
                                              float ln_eps, void* out, vla_stream_t stream);

/* Row sums handed from the launch that writes a row to the launch that normalises it (no
 * counterpart in the reference, whose norm is a graph node of its own, src/layers/norm.h:31-48).
 * A DiT block's LayerNorm needs (sum, sum of squares) of every row of h; taken inside the
 * projection launch they are summed again by each of the launch's column tiles, from operand
 * fragments, on the critical path of its K walk.  The output projection of the block before
 * has each value of the row in a register when it writes it:
 *   vla_linear_row_stats = vla_linear for bf16 rows and bf16 output (N a multiple of 64) that
 *     also leaves row_stats [M][N / 64][2] fp32: (sum of squares, sum) of the 64 values, as
 *     written (rounded to bf16), of each (row, 64-column tile);
 *   vla_layernorm_attn_qkv_rope_stats / vla_layernorm_qkv_self_attention_stats = the two calls
 *     above with the LayerNorm's row sums added up from row_stats [M][n_stat_tiles][2] of their
 *     input x (n_stat_tiles = K / 64 <= 24) instead of from x itself.
 * The sums are added in another order than inside the launches: agreement to fp32 rounding. */
VLA_KAPI int vla_linear_row_stats(const void* x, const void* W, const float* bias, const void* residual, void* y,
                                  float* row_stats, int dtype, int M, int N, int K, vla_stream_t stream);
VLA_KAPI int vla_layernorm_attn_qkv_rope_stats(const void* x, const void* W_folded, const float* colsum, const float* bias,
                                               const float* row_stats, int n_stat_tiles, int dtype, int M, int K, int S,
                                               int n_q_heads, int n_kv_heads, int has_k, int has_v, int head_dim,
                                               const float* cos_tab, const float* sin_tab, void* q_out, void* k_cache,
                                               void* vt_cache, int t_max, int tok_offset, float ln_eps, vla_stream_t stream);
VLA_KAPI int vla_layernorm_qkv_self_attention_stats(const void* x, const void* W_folded, const float* colsum,
                                                    const float* bias, const float* row_stats, int n_stat_tiles, int dtype,
                                                    int M, int K, int S, int n_heads, int head_dim, float scale, float ln_eps,
                                                    void* out, vla_stream_t stream);

/* Host helper for the LayerNorm-inside calls above (bf16 weights [N][K], fp32 scale/shift [K], fp32 bias [N]
 * or NULL): writes W_out (bf16, rounded to nearest even; may alias W), colsum_out and
 * bias_out (fp32 [N]); colsum is taken over the rounded W_out, the values the launch
 * multiplies. */
VLA_KAPI int vla_fold_adaln_weight_host(const void* W, const float* bias, const float* scale, const float* shift, int N,
                                        int K, void* W_out, float* colsum_out, float* bias_out);

/* Host helper for the call above: W_out[n][k] = W[n][k] * g[k] in `dtype` (bf16
 * products rounded to nearest even; g is the RMSNorm weight ggml_mul applies after
 * ggml_rms_norm, src/layers/norm.h:31-34).  W_out may alias W. */
VLA_KAPI int vla_fold_norm_weight_host(const void* W, const void* g, int dtype, int N, int K, void* W_out);

/* Unfused tail of the same step for a projection that already exists as a
 * [M][(n_q_heads + 2 n_kv_heads) * D] matrix (the BitVLA ternary GEMM output,
 * src/kernels/bitvla/bitvla_lm_cuda.cu:428-446: transposes, RoPE on Q and K,
 * then K/V into the cache instead of repeat_kv). */
VLA_KAPI int vla_qkv_split_rope_append(const void* qkv, const float* cos_tab, const float* sin_tab, void* q_out,
                                       void* k_cache, void* vt_cache, int dtype, int M, int S, int n_q_heads,
                                       int n_kv_heads, int head_dim, int t_max, int tok_offset, vla_stream_t stream);

/* ------------------------------------------------------------------ attention */

/* out = softmax(scale * Q K^T + mask) V over keys [0, n_keys) of the resident
 * cache, GQA by head-group sharing (q head h reads kv head h / (Hq/Hkv)):
 * replaces ggml_flash_attn_ext / mul_mat + soft_max_ext + mul_mat
 * (src/models/smolvla.cpp:835-842, src/models/pi0.cpp:215-223,
 * src/layers/attn.h:38-58) and the repeat_kv + cuBLAS + softmax sequence of
 * src/kernels/bitvla/bitvla_lm_cuda.cu:446-486.
 *   q   [batch][S][n_q_heads][D] token-major, out [batch][S][n_q_heads*D]
 *   mask: additive fp32 [S][n_keys] shared by heads and batch, or NULL to use
 *   the generated mask (mask_kind, n_prefix, pad_start, pad_end).
 * Shapes whose keys are sliced across workgroups need scratch memory (the slices' partial
 * rows and arrival counters).  This entry point takes it from blocks the library keeps per
 * (device, stream): grown on demand with hipMalloc -- so a shape must have run once on a
 * stream before that stream is captured -- and never freed before the process ends, so a
 * captured graph keeps pointing at live memory.  Calls on one stream are ordered and may
 * share a block; calls on different streams never do. */
VLA_KAPI int vla_attn_prefix_suffix(const void* q, const void* k_cache, const void* vt_cache, void* out,
                                    int dtype, int batch, int S, int n_q_heads, int n_kv_heads, int head_dim,
                                    int t_max, int n_keys, float scale, int mask_kind, int n_prefix,
                                    int pad_start, int pad_end, const float* mask, vla_stream_t stream);

/* The same call with the scratch memory owned by the caller -- what a model handle uses, so
 * that the reference's rule "one vla_predict at a time per handle" (include/vla.h:18-19) is
 * all a caller has to keep: handles never share scratch.
 *   vla_attn_workspace_bytes: bytes the shape needs, 0 when it needs none,
 *     VLA_ATTN_WORKSPACE_UNSUPPORTED when no kernel takes the shape.  It depends on the shape
 *     and on the tuning overrides in force (VLA_ATTN_SPLIT, VLA_ATTN_DIRECT_ROWS,
 *     VLA_ATTN_NO_ARRIVE, VLA_ATTN_PART_F32, VLA_ATTN_DL change how the keys are sliced), not on
 *     pointers: size a workspace after the last vla_kernels_reload_env, or launches return
 *     VLA_K_ERR_WORKSPACE (nothing is written out of bounds either way).
 *   workspace: device memory of at least that many bytes, 16-byte aligned, zero-filled once
 *     before its first use (every launch leaves the part that must stay zero at zero);
 *     NULL is accepted when the shape needs none.  VLA_K_ERR_WORKSPACE if it is too small.
 *   vla_attn_workspace_reset: the part that must be zero, zeroed again (one small fill
 *     kernel; capturable).  A launch that ran to its end leaves it at zero by itself, one
 *     that was cut short (device fault, reset) does not and would poison every later launch on
 *     the workspace: run it at the start of each launch sequence (a model handle does, once
 *     per action chunk). */
#define VLA_ATTN_WORKSPACE_UNSUPPORTED ((size_t)-1)
VLA_KAPI size_t vla_attn_workspace_bytes(int dtype, int batch, int S, int n_q_heads, int n_kv_heads, int head_dim,
                                         int n_keys);
VLA_KAPI int vla_attn_workspace_reset(void* workspace, size_t workspace_bytes, vla_stream_t stream);
VLA_KAPI int vla_attn_prefix_suffix_ws(const void* q, const void* k_cache, const void* vt_cache, void* out,
                                       int dtype, int batch, int S, int n_q_heads, int n_kv_heads, int head_dim,
                                       int t_max, int n_keys, float scale, int mask_kind, int n_prefix,
                                       int pad_start, int pad_end, const float* mask, void* workspace,
                                       size_t workspace_bytes, vla_stream_t stream);

/* vla_attn_prefix_suffix for callers that cannot allocate.  It has no counterpart in the
 * reference; it is for code under HIP graph capture, tight serving loops and harnesses that
 * forbid hipMalloc.  Same arguments, same results (bit for bit), but the scratch memory is a
 * fixed device array inside the library (VLA_ATTN_NOALLOC_SCRATCH_BYTES per GPU, held until
 * the process ends) and no allocating call is made; a shape that needs more returns
 * VLA_K_ERR_WORKSPACE and launches nothing (vla_attn_workspace_bytes tells in advance).
 * Every call on a GPU uses that GPU's one array: calls that may overlap on the device
 * (different streams) race and must be serialised by the caller.  The array's address is
 * looked up on the first call per device; vla_kernels_init() does it ahead of time. */
#define VLA_ATTN_NOALLOC_SCRATCH_BYTES ((size_t)(64u << 10) + ((size_t)16u << 20))
VLA_KAPI int vla_attn_prefix_suffix_noalloc(const void* q, const void* k_cache, const void* vt_cache, void* out,
                                            int dtype, int batch, int S, int n_q_heads, int n_kv_heads,
                                            int head_dim, int t_max, int n_keys, float scale, int mask_kind,
                                            int n_prefix, int pad_start, int pad_end, const float* mask,
                                            vla_stream_t stream);

/* --------------------------------------------------------- flow-matching glue */

/* Suffix embedding h[b][s][:] for one denoise step (stand-in for
 * build_embed_suffix, src/models/pi0.cpp:232-247, and the action_emb of
 * src/models/smolvla.cpp:1398): rows s < n_lead copy lead[b][s][:] (pi0 / DiT
 * state token); other rows are W_in . x_t[b][s - n_lead] + bias_step.
 *   x_t fp32 [batch][S - n_lead][A]; W_in fp32 [W][A]; bias_step fp32 [W];
 *   lead fp32 [batch][n_lead][W] or NULL; h in `out_dtype`.  A <= 136 (GR00T N1.7's 132
 * action values); VLA_K_ERR_SHAPE beyond. */
VLA_KAPI int vla_embed_suffix(const float* x_t, const float* W_in, const float* bias_step, const float* lead,
                              void* h, int out_dtype, int batch, int S, int n_lead, int A, int W,
                              vla_stream_t stream);

/* The same with an activation on the projected rows (lead rows are copied as they are):
 * the first projection of the action-time MLP of build_embed_suffix
 * (src/models/smolvla.cpp:1397-1403, src/models/pi0.cpp:240-244) with the time half of its
 * input folded into bias_step. */
VLA_KAPI int vla_embed_suffix_act(const float* x_t, const float* W_in, const float* bias_step, const float* lead,
                                  void* h, int out_dtype, int batch, int S, int n_lead, int A, int W, int act,
                                  vla_stream_t stream);

/* h[b][s][:] = lead[b][s][:] for s < n_lead, converted to `dtype`: the state-token rows
 * of ggml_concat(state_emb, action_time_emb) (src/models/pi0.cpp:245-246) when the action
 * rows were produced by a projection over all S rows of the suffix. */
VLA_KAPI int vla_set_lead_rows(const float* lead, void* h, int dtype, int batch, int S, int n_lead, int W,
                               vla_stream_t stream);

/* h[b][s][:] = lead[b][s][:] for s < n_lead, else acc[b][s][:] + row_table[s - n_lead][:],
 * converted to `dtype`: the tail of ActionExpert::encode_action
 * (src/modules/action_expert.cpp:46-52: W3 . silu(..) + bias, plus the learned position rows)
 * and of the concat with the state / future-token rows (src/models/gr00tn1d5.cpp:371) when
 * the action rows came out of an fp32 projection over all S rows.  acc fp32 [batch][S][W];
 * row_table fp32 [S - n_lead][W] or NULL; lead fp32 [batch][n_lead][W]. */
VLA_KAPI int vla_finish_suffix_rows(const float* acc, const float* row_table, const float* lead, void* h, int dtype,
                                    int batch, int S, int n_lead, int W, vla_stream_t stream);

/* Output projection + Euler update (src/models/smolvla.cpp:1416-1418,
 * src/models/pi0.cpp:577-587): x_t[b][s] += dt * (W_out . hn[b][n_lead + s] + b_out).
 *   hn [batch][S][W] in `dtype` (already normalised); W_out fp32 [A][W]. */
VLA_KAPI int vla_euler_step(float* x_t, const void* hn, const float* W_out, const float* b_out, int dtype,
                            int batch, int S, int n_lead, int A, int W, float dt, vla_stream_t stream);

/* The same update with the stack's final norm inside the launch: h [batch][S][W] holds the
 * rows before the norm, and each row is normalised (and rounded to `dtype`, as the separate
 * norm launch would store it) right before its projection.
 *   vla_rmsnorm_euler_step: rms_norm(h) * norm_w (norm_w [W] in `dtype` or NULL), the final
 *     norm of src/models/smolvla.cpp:1413-1418 and src/models/pi0.cpp:572-587;
 *   vla_adanorm_euler_step: n + n * scale + shift with scale, shift fp32 [W]; centred != 0:
 *     n = layer_norm(h) without affine (src/layers/norm.h:37-46, the norm_out of
 *     src/modules/dit_head.cpp:139-147), centred == 0: n = h * rsqrt(mean h^2 + eps)
 *     (build_adarms, src/models/pi05.cpp:208-223, final norm at pi05.cpp:628).
 * Meant for the flow heads' widths: rows wider than 2048 are handled but take longer than
 * the norm launch they save. */
VLA_KAPI int vla_rmsnorm_euler_step(float* x_t, const void* h, const void* norm_w, float eps, const float* W_out,
                                    const float* b_out, int dtype, int batch, int S, int n_lead, int A, int W, float dt,
                                    vla_stream_t stream);
VLA_KAPI int vla_adanorm_euler_step(float* x_t, const void* h, const float* scale, const float* shift, int centred,
                                    float eps, const float* W_out, const float* b_out, int dtype, int batch, int S,
                                    int n_lead, int A, int W, float dt, vla_stream_t stream);

/* ------------------------------------------------------------ BitVLA ternary */

/* Per-row int8 quantisation (act_quant_kernel,
 * src/kernels/bitvla/bitnet_kernels.h:465-521): scales[m] = 127 / max(amax, 1e-5).
 * rowsum[m] = sum_k q[m][k] (int32) feeds the ternary GEMM's code-offset
 * correction; may be NULL. */
VLA_KAPI int vla_act_quant_bf16(const uint16_t* in, int8_t* out, float* scales, int32_t* rowsum, int M, int K,
                                vla_stream_t stream);

/* bitvla_rmsnorm_bf16 followed by vla_act_quant_bf16 in one launch (the pair that opens
 * both halves of run_layer, src/kernels/bitvla/bitvla_lm_cuda.cu:422-486); the bf16
 * intermediate is not written.  int8 rows, scales and row sums are bit-identical to the
 * two separate calls for K <= 4096 (longer rows are shared by four wavefronts, which add
 * the squares in another order than the separate RMSNorm: results agree to rounding). */
VLA_KAPI int vla_rmsnorm_act_quant_bf16(const uint16_t* x, const uint16_t* w, int8_t* out, float* scales,
                                        int32_t* rowsum, float eps, int M, int K, vla_stream_t stream);
/* The same on rows formed on the fly from a fused [M][gate(K) | up(K)] projection,
 * x = bf16(relu(gate)^2 * up): gate_up_fused_sqrelu_mul_bf16 -> ffn sub-norm -> act_quant of
 * run_layer (bitvla_lm_cuda.cu:503-513) in one launch, same bits as those calls; the
 * activation is not written.  VLA_K_ERR_SHAPE when K % 8, K > 8192 or a buffer is not
 * 16-byte aligned: callers fall back to the separate calls. */
VLA_KAPI int vla_sqrelu_rmsnorm_act_quant_bf16(const uint16_t* gate_up, const uint16_t* w, int8_t* out, float* scales,
                                               int32_t* rowsum, float eps, int M, int K, vla_stream_t stream);

/* Ternary weight quantisation on the host (recover_ternary_and_scale,
 * src/models/bitvla.cpp:430-451). */
VLA_KAPI int vla_ternary_quant_host(const float* W, int64_t n, int8_t* ternary, float* absmean);

/* Host packers.  A packed word holds the codes t+2 of 16 consecutive k of one
 * output column, value b+4j at bits 8b+2j: the reference's 16-value slot
 * (src/models/bitvla.cpp:470-480).  The gfx950 layout orders the words
 * "MFMA-fragment-major" instead of the wmma "ladder" order: word (n, w), w = k/16,
 * sits at index (((n/32) * (K/32) + w/2) * 2 + w%2) * 32 + n%32, so the 64 words a
 * wavefront feeds to one v_mfma_i32_32x32x32_i8 are contiguous.  Buffers hold
 * vla_ternary_packed_words(N, K) words (N rounded up to 32; pad columns are weight 0). */
VLA_KAPI long vla_ternary_packed_words(int N, int K);
VLA_KAPI int vla_ternary_pack_host(const int8_t* ternary, int N, int K, uint32_t* packed);
VLA_KAPI int vla_ternary_repack_ladder_host(const uint8_t* ladder, int N, int K, uint32_t* packed);

/* out[m][n] = bf16(float(acc) / s[m] * ws[n / (N/ws_num)]),
 * acc = sum_k A[m][k] * t[n][k] exact in int32
 * (ladder_int8xint2_kernel_m_wide, bitnet_kernels.h:285-409).  acc_out
 * (int32 [M][N]) receives the raw accumulators when not NULL; out may then be
 * NULL. */
VLA_KAPI int vla_ternary_gemm(const int8_t* A, const uint32_t* W_packed, uint16_t* out, int32_t* acc_out,
                              const float* s, const int32_t* rowsum, const float* ws, int ws_num, int M, int N,
                              int K, vla_stream_t stream);

/* vla_ternary_gemm followed by bitvla_add_bf16 in one launch:
 * out[m][n] = bf16(bf16(float(acc) / s[m] * ws[g]) + residual[m][n]); out may alias residual
 * (the O projection + residual of run_layer, bitvla_lm_cuda.cu:480-486).  residual may be NULL. */
VLA_KAPI int vla_ternary_gemm_add(const int8_t* A, const uint32_t* W_packed, uint16_t* out, const uint16_t* residual,
                                  const float* s, const int32_t* rowsum, const float* ws, int ws_num, int M, int N,
                                  int K, vla_stream_t stream);

/* The decode step's norm -> quantise -> projection chain in one launch, for M <= 8 rows:
 * vla_rmsnorm_act_quant_bf16(x, norm_w, eps) feeding vla_ternary_gemm_add, with the int8
 * rows, scales and row sums kept on chip (run_layer's attn_norm + QKV and sub_norm + O
 * pairs, bitvla_lm_cuda.cu:421-486, at S = 1).  Same bits as the two calls.  out may alias
 * residual, never x (every workgroup reads whole rows of x while others write out).
 * VLA_K_ERR_SHAPE when M > 8, K > 7168 or K % 128: callers fall back to the pair. */
VLA_KAPI int vla_rmsnorm_ternary_gemv(const uint16_t* x, const uint16_t* norm_w, float eps, const uint32_t* W_packed,
                                      uint16_t* out, const uint16_t* residual, const float* ws, int ws_num, int M,
                                      int N, int K, vla_stream_t stream);
/* The same with x formed on the fly from a fused [M][gate(K) | up(K)] projection,
 * x = bf16(relu(gate)^2 * up): gate_up_fused_sqrelu_mul_bf16 -> ffn sub-norm -> act_quant ->
 * down projection (+ residual) of run_layer (bitvla_lm_cuda.cu:503-520) in one launch, same
 * bits as those calls for K <= 4096, equal to rounding beyond. */
VLA_KAPI int vla_sqrelu_rmsnorm_ternary_gemv(const uint16_t* gate_up, const uint16_t* norm_w, float eps,
                                             const uint32_t* W_packed, uint16_t* out, const uint16_t* residual,
                                             const float* ws, int ws_num, int M, int N, int K, vla_stream_t stream);

/* The same launch for the fused Q | K | V projection of one appended token per batch row,
 * with vla_qkv_split_rope_append (S = 1) in its epilogue: Q rotated to q_out [batch][Hq][D],
 * K rotated into k_cache at slot tok_offset, V into vt_cache (attn_norm -> QKV -> RoPE ->
 * cache of run_layer, bitvla_lm_cuda.cu:421-460).  cos_row / sin_row: the D/2 table entries
 * of the token's position.  W_paired: the packed weight with its rows reordered by
 * vla_ternary_pair_rope_rows_host (a rotation pair in one 32-row block).  Same bits as
 * vla_rmsnorm_ternary_gemv + vla_qkv_split_rope_append.  N = (Hq + 2 Hkv) D;
 * VLA_K_ERR_SHAPE when batch > 8, K > 4096, K % 128, D % 32 or a scale group (N / ws_num)
 * is not whole heads. */
VLA_KAPI int vla_rmsnorm_ternary_gemv_rope_append(const uint16_t* x, const uint16_t* norm_w, float eps,
                                                  const uint32_t* W_paired, const float* ws, int ws_num,
                                                  const float* cos_row, const float* sin_row, uint16_t* q_out,
                                                  uint16_t* k_cache, uint16_t* vt_cache, int batch, int n_q_heads,
                                                  int n_kv_heads, int head_dim, int K, int t_max, int tok_offset,
                                                  vla_stream_t stream);
/* paired = packed with row n of every Q and K head taken from row
 * (n < 16 ? 16 b + n : D/2 + 16 b + n - 16) of 32-row block b of that head; V rows unchanged.
 * Host memory, vla_ternary_packed_words(N, K) words each, no overlap. */
VLA_KAPI int vla_ternary_pair_rope_rows_host(const uint32_t* packed, int n_q_heads, int n_kv_heads, int head_dim,
                                             int K, uint32_t* paired);

/* -------------------------------------- BitVLA layer helpers (same signatures
 * as src/kernels/bitvla/bitvla_lm_cuda.h:54-155 with hipStream_t / uint16_t) */
VLA_KAPI int bitvla_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* out, float eps, int M, int K,
                                 vla_stream_t stream);
VLA_KAPI int bitvla_rope_neox_bf16(uint16_t* inout, const float* cos_tab, const float* sin_tab, int H, int S,
                                   int D, vla_stream_t stream);
VLA_KAPI int bitvla_softmax_scaled_bf16(uint16_t* inout, float scale, int n_rows, int S, vla_stream_t stream);
VLA_KAPI int bitvla_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out, int N, vla_stream_t stream);
VLA_KAPI int bitvla_repeat_kv_bf16(const uint16_t* in, uint16_t* out, int n_q, int n_kv, int seq, int hd,
                                   vla_stream_t stream);
VLA_KAPI int bitvla_transpose_sNhd_to_NshHd_bf16(const uint16_t* in, uint16_t* out, int S, int N, int hd,
                                                 vla_stream_t stream);
VLA_KAPI int bitvla_transpose_NshHd_to_sNhd_bf16(const uint16_t* in, uint16_t* out, int N, int S, int hd,
                                                 vla_stream_t stream);
VLA_KAPI int bitvla_gather_rows_bf16(const uint16_t* in, uint16_t* out, const int32_t* row_ids, int n_rows,
                                     int K, vla_stream_t stream);
/* bitvla_act_quant_cuda / bitlinear_int8xint2_m / bitlinear_int8xint2
 * (src/kernels/bitvla/bitnet_kernels.cu:31,76,118) with the reference's exact
 * argument lists.  B is the gfx950 packed layout (see vla_ternary_pack_host);
 * the row sums the GEMM needs are computed on the same stream into a buffer
 * the library owns, so one call at a time per process. */
VLA_KAPI int bitvla_act_quant(const uint16_t* in, int8_t* out, float* scales, int M, int K, vla_stream_t stream);
VLA_KAPI int bitlinear_int8xint2_m(int8_t* A, int8_t* B, uint16_t* out, float* s, float* ws, int M, int N, int K,
                                   vla_stream_t stream);
VLA_KAPI int bitlinear_int8xint2(int8_t* A, int8_t* B, uint16_t* out, float* s, float* ws, int M, int N, int K,
                                 vla_stream_t stream);

/* out[s][k] = bf16(relu(gate[s][k])^2 * up[s][k]) on a fused [seq][gate(ffn) | up(ffn)] projection
 * (gate_up_fused_sqrelu_mul_bf16, src/kernels/bitvla/bitvla_lm_cuda.cu:525-548). */
VLA_KAPI int gate_up_fused_sqrelu_mul_bf16(const uint16_t* gu, uint16_t* out, int seq, int ffn, vla_stream_t stream);

/* The context form of the BitVLA language model (bitvla_lm_layer_cuda and
 * bitvla_lm_cuda_{init,set_layer,set_output_norm,forward,free},
 * src/kernels/bitvla/bitvla_lm_cuda.h:211-286; run_layer,
 * src/kernels/bitvla/bitvla_lm_cuda.cu:395-522): same fields, arguments and meaning, device
 * pointers owned by the caller.  Differences: *_packed weights are in the gfx950 word order
 * (vla_ternary_pack_host / vla_ternary_repack_ladder_host, one buffer of
 * vla_ternary_packed_words(N, K) words per tensor); *_ws hold one fp32 scale per tensor, two for
 * gate_up (gate, up); attention runs as one fused kernel with fp32 scores instead of bf16
 * scores between two library GEMMs.  forward() copies d_in, runs every layer over all `seq`
 * tokens (no mask, positions 0..seq-1) and writes the output-normed hidden states; it launches
 * on `stream` without synchronising and returns 0, or -1 for seq > max_seq, an unbound layer
 * or a failed launch.  One forward at a time per context. */
typedef struct {
    uint16_t* attn_norm_w;
    uint16_t* attn_sub_norm_w;
    uint16_t* ffn_norm_w;
    uint16_t* ffn_sub_norm_w;
    int8_t* q_packed;
    float* q_ws;
    int8_t* k_packed;
    float* k_ws;
    int8_t* v_packed;
    float* v_ws;
    int8_t* o_packed;
    float* o_ws;
    int8_t* gate_up_packed;
    float* gate_up_ws;
    int8_t* down_packed;
    float* down_ws;
} bitvla_lm_layer_hip;
typedef struct bitvla_lm_hip_ctx bitvla_lm_hip_ctx;
VLA_KAPI bitvla_lm_hip_ctx* bitvla_lm_hip_init(int hidden, int n_q, int n_kv, int head_dim, int ffn, int n_layers,
                                               float rope_base, float rms_eps, int max_seq);
VLA_KAPI void bitvla_lm_hip_free(bitvla_lm_hip_ctx* ctx);
VLA_KAPI void bitvla_lm_hip_set_layer(bitvla_lm_hip_ctx* ctx, int L, const bitvla_lm_layer_hip* layer);
VLA_KAPI void bitvla_lm_hip_set_output_norm(bitvla_lm_hip_ctx* ctx, const uint16_t* w);
VLA_KAPI int bitvla_lm_hip_forward(bitvla_lm_hip_ctx* ctx, const uint16_t* d_in, uint16_t* d_out, int seq,
                                   vla_stream_t stream);

/* Library identification, for a loader that wants to check what it bound. */
VLA_KAPI const char* vla_kernels_arch(void); /* "gfx950" */

/* Optional set-up for the current device, so that no later call has to do it lazily: reads
 * the tuning overrides from the environment and resolves the fixed scratch array of
 * vla_attn_prefix_suffix_noalloc.  0 or a vla_kstatus. */
VLA_KAPI int vla_kernels_init(void);
/* Reads the tuning overrides (VLA_ATTN_*, VLA_GEMM_*, VLA_TERNARY_TILE; tests and tuning
 * only) from the environment again.  No launch path reads the environment.  Not thread-safe
 * against launches: call it while no other thread is inside the library.  Workspaces sized
 * before the call (vla_attn_workspace_bytes, a model handle's own) may be too small after it:
 * a handle plans its workspace again at its next prefill. */
VLA_KAPI void vla_kernels_reload_env(void);
/* Number of vla_kernels_reload_env calls so far: what a holder of a planned workspace compares to know that it must plan again. */
VLA_KAPI int vla_kernels_tuning_generation(void);

#ifdef __cplusplus
}
#endif
#endif /* VLA_KERNELS_H */
