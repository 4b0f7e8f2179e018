"""CPU oracle for the action-expert attention hot path (TEST INFRASTRUCTURE ONLY).

ctypes front end of ``liboracle.so`` (built from ``oracle.cpp`` by the Makefile
beside it).  Only tests, the smoke check and the benchmark's CPU-baseline leg
import this package; the shipped library never does.

Every wrapper takes and returns numpy arrays; layouts are row-major and
"token-major" means ``[token][head][head_dim]``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with the Makefile in this directory."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i8p = ctypes.POINTER(ctypes.c_int8)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def _p(a, ty):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle wants contiguous arrays"
    return a.ctypes.data_as(ty)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


_lib.orc_f32_to_bf16.restype = ctypes.c_uint16
_lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
_lib.orc_bf16_to_f32.restype = ctypes.c_float
_lib.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
_lib.orc_silu.restype = ctypes.c_float
_lib.orc_silu.argtypes = [ctypes.c_float]
_lib.orc_num_threads.restype = ctypes.c_int


def num_threads():
    return int(_lib.orc_num_threads())


def set_num_threads(n):
    _lib.orc_set_num_threads(int(n))


# Accumulation of linear() and attention() when the caller does not say: double for parity
# checks (the default, never changed by tests); the benchmark's CPU-baseline leg switches to
# fp32 SIMD-style accumulation, which is what a CPU inference engine runs.
_DEFAULT_ACC64 = True


def set_default_accumulation(acc64):
    global _DEFAULT_ACC64
    _DEFAULT_ACC64 = bool(acc64)


# ---------------------------------------------------------------- bf16 helpers
def to_bf16(x):
    """fp32 array -> uint16 array of bf16 bit patterns (round to nearest even)."""
    x = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    _lib.orc_to_bf16(_p(x, _f32p), _p(y, _u16p), ctypes.c_int64(x.size))
    return y


def from_bf16(u):
    u = np.ascontiguousarray(u, dtype=np.uint16)
    y = np.empty(u.shape, dtype=np.float32)
    _lib.orc_from_bf16(_p(u, _u16p), _p(y, _f32p), ctypes.c_int64(u.size))
    return y


def round_bf16(x):
    """fp32 -> nearest bf16 value, returned as fp32."""
    return from_bf16(to_bf16(x))


def f32_to_bf16_trunc(x):
    return (np.ascontiguousarray(x, np.float32).view(np.uint32) >> 16).astype(np.uint16)


# ------------------------------------------------------------------------ rope
def rope_tables(pos, D, base):
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    n = pos.size
    c = np.empty((n, D // 2), np.float32)
    s = np.empty((n, D // 2), np.float32)
    _lib.orc_rope_tables(_p(pos, _i32p), n, D, ctypes.c_double(base), _p(c, _f32p), _p(s, _f32p))
    return c, s


def rope_tables_f32_powf(n_tok, D, base):
    c = np.empty((n_tok, D // 2), np.float32)
    s = np.empty((n_tok, D // 2), np.float32)
    _lib.orc_rope_tables_f32_powf(n_tok, D, ctypes.c_float(base), _p(c, _f32p), _p(s, _f32p))
    return c, s


def rope_neox(x, cos_t, sin_t):
    """x [n_tok, n_heads, D] -> rotated copy."""
    y = _f32(x).copy()
    n_tok, n_heads, D = y.shape
    cos_t, sin_t = _f32(cos_t), _f32(sin_t)
    assert cos_t.shape == (n_tok, D // 2)
    _lib.orc_rope_neox(_p(y, _f32p), _p(cos_t, _f32p), _p(sin_t, _f32p), n_tok, n_heads, D)
    return y


def rotate_half(x):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_rotate_half(_p(x, _f32p), _p(y, _f32p), x.size)
    return y


# ---------------------------------------------------------------- linear, norm
def linear(x, W, b=None, acc64=None):
    acc64 = _DEFAULT_ACC64 if acc64 is None else acc64
    x, W = _f32(x), _f32(W)
    M, K = x.shape
    N, K2 = W.shape
    assert K == K2
    b = None if b is None else _f32(b)
    y = np.empty((M, N), np.float32)
    _lib.orc_linear(_p(x, _f32p), _p(W, _f32p), _p(b, _f32p), _p(y, _f32p), M, N, K, int(acc64))
    return y


def rms_norm(x, w, eps):
    x = _f32(x)
    M, K = x.shape
    w = None if w is None else _f32(w)
    y = np.empty_like(x)
    _lib.orc_rms_norm(_p(x, _f32p), _p(w, _f32p), _p(y, _f32p), M, K, ctypes.c_float(eps))
    return y


def layer_norm(x, w, b, eps):
    x = _f32(x)
    M, K = x.shape
    w = None if w is None else _f32(w)
    b = None if b is None else _f32(b)
    y = np.empty_like(x)
    _lib.orc_layer_norm(_p(x, _f32p), _p(w, _f32p), _p(b, _f32p), _p(y, _f32p), M, K, ctypes.c_float(eps))
    return y


def adaln(x, sc, sh, eps):
    x, sc, sh = _f32(x), _f32(sc), _f32(sh)
    M, K = x.shape
    y = np.empty_like(x)
    _lib.orc_adaln(_p(x, _f32p), _p(sc, _f32p), _p(sh, _f32p), _p(y, _f32p), M, K, ctypes.c_float(eps))
    return y


def adarms(x, scale, shift, eps):
    """adaRMS (build_adarms, src/models/pi05.cpp:208-224): n = rms_norm(x) without a weight,
    then (n + n * scale) + shift in that order."""
    n = rms_norm(x, None, eps)
    return ((n + n * _f32(scale)) + _f32(shift)).astype(np.float32)


def silu(x):
    x = _f32(x)
    return (x / (1.0 + np.exp(-x.astype(np.float64)))).astype(np.float32)


def gelu(x):
    """ggml_gelu: the tanh form 0.5 x (1 + tanh(sqrt(2/pi) x (1 + 0.044715 x^2))), as the
    reference's FFN halves use it (src/layers/ffn.h:24-27, src/models/pi0.cpp:229).  ggml's
    CPU kernel reads a 16-bit lookup table for this function; the table is not reproduced
    (parity unpinned at that level), the formula is."""
    x = _f32(x).astype(np.float64)
    return (0.5 * x * (1.0 + np.tanh(0.7978845608028654 * x * (1.0 + 0.044715 * x * x)))).astype(np.float32)


def ffn_glu(x, Wg, Wu, Wd, act):
    """Wd (act(Wg x) * (Wu x)): the gated FFN of the SmolVLA expert (act = silu,
    src/models/smolvla.cpp:845-847) and of the Gemma expert (act = gelu, src/models/pi0.cpp:227-231)."""
    return linear(act(linear(x, Wg)) * linear(x, Wu), Wd)


def ffn_gelu(x, W1, b1, W2, b2):
    """ffn_gelu (src/layers/ffn.h:24-27): W2 gelu(W1 x + b1) + b2."""
    return linear(gelu(linear(x, W1, b1)), W2, b2)


# ------------------------------------------------------------ concat / softmax
def kv_concat(cache, suffix):
    """[P, ...] ++ [S, ...] along axis 0 into a fresh array (any dtype)."""
    cache = np.ascontiguousarray(cache)
    suffix = np.ascontiguousarray(suffix)
    assert cache.dtype == suffix.dtype and cache.shape[1:] == suffix.shape[1:]
    P, S = cache.shape[0], suffix.shape[0]
    row_bytes = int(np.prod(cache.shape[1:])) * cache.dtype.itemsize
    out = np.empty((P + S,) + cache.shape[1:], cache.dtype)
    _lib.orc_kv_concat(cache.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(P),
                       suffix.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(S),
                       ctypes.c_int64(row_bytes), out.ctypes.data_as(ctypes.c_void_p))
    return out


def softmax_ext(kq, mask, scale):
    y = _f32(kq).copy()
    rows, T = y.shape
    mask = None if mask is None else _f32(mask)
    _lib.orc_softmax_ext(_p(y, _f32p), _p(mask, _f32p), ctypes.c_float(scale), rows, T)
    return y


def softmax_scaled_bf16(u16, scale):
    y = np.ascontiguousarray(u16, np.uint16).copy()
    rows, S = y.shape
    _lib.orc_softmax_scaled_bf16(_p(y, _u16p), ctypes.c_float(scale), rows, S)
    return y


def attention(Q, K, V, mask, scale, acc64=None):
    """Q [S,Hq,D], K/V [T,Hkv,D] token-major, mask [S,T] additive or None -> [S, Hq*D]."""
    acc64 = _DEFAULT_ACC64 if acc64 is None else acc64
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    S, Hq, D = Q.shape
    T, Hkv, D2 = K.shape
    assert D == D2 and V.shape == K.shape and Hq % Hkv == 0
    mask = None if mask is None else _f32(mask)
    if mask is not None:
        assert mask.shape == (S, T)
    out = np.empty((S, Hq * D), np.float32)
    _lib.orc_attention(_p(Q, _f32p), _p(K, _f32p), _p(V, _f32p), _p(mask, _f32p), ctypes.c_float(scale),
                       S, T, Hq, Hkv, D, _p(out, _f32p), int(acc64))
    return out


# ----------------------------------------------------------------------- masks
def mask_smolvla_full(P, S, pad_start, pad_end):
    m = np.empty((S, P + S), np.float32)
    _lib.orc_mask_smolvla_full(P, S, pad_start, pad_end, _p(m, _f32p))
    return m


def mask_smolvla_prefix_only(P, S, pad_start, pad_end):
    m = np.empty((S, P), np.float32)
    _lib.orc_mask_smolvla_prefix_only(P, S, pad_start, pad_end, _p(m, _f32p))
    return m


def mask_smolvla_prefill(P, pad_start, pad_end, state_pos):
    m = np.empty((P, P), np.float32)
    pos = np.empty(P, np.int32)
    _lib.orc_mask_smolvla_prefill(P, pad_start, pad_end, state_pos, _p(m, _f32p), _p(pos, _i32p))
    return m, pos


def mask_pi0_full(P, S):
    m = np.empty((S, P + S), np.float32)
    _lib.orc_mask_pi0_full(P, S, _p(m, _f32p))
    return m


def mask_causal(seq):
    m = np.empty((seq, seq), np.float32)
    _lib.orc_mask_causal(seq, _p(m, _f32p))
    return m


# ------------------------------------------------------------- time embeddings
def timesteps_proj(bucket):
    out = np.empty(256, np.float32)
    _lib.orc_timesteps_proj(ctypes.c_int64(bucket), _p(out, _f32p))
    return out


def action_sinusoid(bucket, dim, T):
    out = np.empty((T, dim), np.float32)
    _lib.orc_action_sinusoid(ctypes.c_int64(bucket), ctypes.c_int64(dim), ctypes.c_int64(T), _p(out, _f32p))
    return out


def sinusoidal_time_emb(t, dim, min_p, max_p):
    out = np.empty(dim, np.float32)
    _lib.orc_sinusoidal_time_emb(ctypes.c_double(t), ctypes.c_int64(dim), ctypes.c_double(min_p),
                                 ctypes.c_double(max_p), _p(out, _f32p))
    return out


# --------------------------------------------------------------------- ternary
def weight_quant_ternary(W):
    W = _f32(W)
    t = np.empty(W.shape, np.int8)
    am = ctypes.c_float(0)
    _lib.orc_weight_quant_ternary(_p(W, _f32p), ctypes.c_int64(W.size), _p(t, _i8p), ctypes.byref(am))
    return t, np.float32(am.value)


def pack_ladder_int2(Wt):
    Wt = np.ascontiguousarray(Wt, np.int8)
    N, K = Wt.shape
    assert N % 16 == 0 and K % 128 == 0
    out = np.empty(N * K // 4, np.uint8)
    _lib.orc_pack_ladder_int2(_p(Wt, _i8p), ctypes.c_int64(N), ctypes.c_int64(K), _p(out, _u8p))
    return out


def unpack_ladder_int2(packed, N, K):
    packed = np.ascontiguousarray(packed, np.uint8)
    assert packed.size == N * K // 4
    W = np.empty((N, K), np.int8)
    _lib.orc_unpack_ladder_int2(_p(packed, _u8p), ctypes.c_int64(N), ctypes.c_int64(K), _p(W, _i8p))
    return W


def decode_i2s_to_i8s(word):
    out = np.empty(16, np.int8)
    _lib.orc_decode_i2s_to_i8s(ctypes.c_uint32(int(word)), _p(out, _i8p))
    return out


def act_quant(x):
    """fp32 [M,K] -> (int8 [M,K], scales fp32 [M]) with scales = 127/amax."""
    x = _f32(x)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    s = np.empty(M, np.float32)
    _lib.orc_act_quant(_p(x, _f32p), M, K, _p(q, _i8p), _p(s, _f32p))
    return q, s


def act_fake_quant(x):
    x = _f32(x)
    M, K = x.shape
    y = np.empty_like(x)
    _lib.orc_act_fake_quant(_p(x, _f32p), M, K, _p(y, _f32p))
    return y


def ternary_gemm_i32(A, Wt):
    A = np.ascontiguousarray(A, np.int8)
    Wt = np.ascontiguousarray(Wt, np.int8)
    M, K = A.shape
    N, K2 = Wt.shape
    assert K == K2
    acc = np.empty((M, N), np.int32)
    _lib.orc_ternary_gemm_i32(_p(A, _i8p), _p(Wt, _i8p), M, N, K, _p(acc, _i32p))
    return acc


def ternary_epilogue(acc, s, ws):
    """bf16(float(acc)/s[m]*ws[n // (N/len(ws))]) as uint16 bit patterns."""
    acc = np.ascontiguousarray(acc, np.int32)
    s, ws = _f32(s), _f32(ws)
    M, N = acc.shape
    out = np.empty((M, N), np.uint16)
    _lib.orc_ternary_epilogue(_p(acc, _i32p), _p(s, _f32p), _p(ws, _f32p), M, N, ws.size, _p(out, _u16p))
    return out


def bit_linear_f32(x, Wt, absmean):
    x = _f32(x)
    Wt = np.ascontiguousarray(Wt, np.int8)
    M, K = x.shape
    N = Wt.shape[0]
    y = np.empty((M, N), np.float32)
    _lib.orc_bit_linear_f32(_p(x, _f32p), _p(Wt, _i8p), ctypes.c_float(absmean), _p(y, _f32p), M, N, K)
    return y


# ------------------------------------------------------- BitVLA layout helpers
def repeat_kv(u16, n_q):
    u16 = np.ascontiguousarray(u16, np.uint16)
    n_kv, seq, hd = u16.shape
    out = np.empty((n_q, seq, hd), np.uint16)
    _lib.orc_repeat_kv_u16(_p(u16, _u16p), _p(out, _u16p), n_q, n_kv, seq, hd)
    return out


def transpose_sHd_to_Hsd(u16, H):
    u16 = np.ascontiguousarray(u16, np.uint16)
    S, HD = u16.shape
    hd = HD // H
    out = np.empty((H, S, hd), np.uint16)
    _lib.orc_transpose_sHd_to_Hsd_u16(_p(u16, _u16p), _p(out, _u16p), S, H, hd)
    return out


def transpose_Hsd_to_sHd(u16):
    u16 = np.ascontiguousarray(u16, np.uint16)
    H, S, hd = u16.shape
    out = np.empty((S, H * hd), np.uint16)
    _lib.orc_transpose_Hsd_to_sHd_u16(_p(u16, _u16p), _p(out, _u16p), H, S, hd)
    return out


def gather_rows(u16, ids):
    u16 = np.ascontiguousarray(u16, np.uint16)
    ids = np.ascontiguousarray(ids, np.int32)
    out = np.empty((ids.size, u16.shape[1]), np.uint16)
    _lib.orc_gather_rows_u16(_p(u16, _u16p), _p(out, _u16p), _p(ids, _i32p), ids.size, u16.shape[1])
    return out
