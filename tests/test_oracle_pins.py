"""Pins the CPU oracle before anything is compared against it.

Each check is either a vector the reference's own tests hold
(tests/test_rope_conventions.cpp, tests/test_dit_common.cpp), a hand-worked
case of an in-tree definition (ladder pack, 2-bit decode, act-quant), or
something the mathematics fixes (closed forms, invariants, special cases that
reduce to a library routine, brute force in float64 / int64).
"""
import math

import numpy as np
import pytest
import torch

import oracle as orc

NEG = -np.inf


# ----------------------------------------------------------------------- bf16
def test_bf16_round_to_nearest_even_and_nan():
    # 1 + 2^-8 is exactly between two bf16 values: ties to even (1.0).
    assert orc.to_bf16(np.float32([1.0 + 2.0 ** -8]))[0] == 0x3F80
    # 1 + 3*2^-8 ties to 1 + 2^-6 (even mantissa 0x02).
    assert orc.to_bf16(np.float32([1.0 + 3 * 2.0 ** -8]))[0] == 0x3F82
    assert orc.to_bf16(np.float32([np.inf]))[0] == 0x7F80
    assert (orc.to_bf16(np.float32([np.nan]))[0] & 0x7FC0) == 0x7FC0
    x = np.random.default_rng(1).standard_normal(4096).astype(np.float32)
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.to_bf16(x), t)
    assert np.array_equal(orc.from_bf16(t), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    assert orc.f32_to_bf16_trunc(np.float32([1.0 + 3 * 2.0 ** -8]))[0] == 0x3F81


# ----------------------------------------------------------------------- rope
def test_rope_rotate_half_vector_from_reference_test():
    # tests/test_rope_conventions.cpp:65-72: x = 1..8, rotate_half pairs (x0,x4).
    rh = orc.rotate_half(np.arange(1, 9, dtype=np.float32))
    assert rh[0] == -5.0 and rh[4] == 1.0
    assert np.array_equal(rh, np.float32([-5, -6, -7, -8, 1, 2, 3, 4]))


def test_rope_is_x_cos_plus_rotate_half_sin():
    r = np.random.default_rng(2)
    D = 8
    x = r.standard_normal((3, 2, D)).astype(np.float32)
    pos = np.int32([3, 0, 290])
    c, s = orc.rope_tables(pos, D, 10000.0)
    y = orc.rope_neox(x, c, s)
    for t in range(3):
        for h in range(2):
            cf = np.concatenate([c[t], c[t]])
            sf = np.concatenate([s[t], s[t]])
            want = x[t, h] * cf + orc.rotate_half(x[t, h]) * sf
            assert np.allclose(y[t, h], want, rtol=0, atol=1e-6)
    # position 0 is the identity
    assert np.array_equal(y[1], x[1])


def test_rope_tables_closed_form_and_invariants():
    D, base = 64, 10000.0
    pos = np.int32([0, 1, 49, 241, 290, 866])
    c, s = orc.rope_tables(pos, D, base)
    i = np.arange(D // 2, dtype=np.float64)
    ang = pos[:, None].astype(np.float64) * base ** (-2.0 * i / D)
    assert np.array_equal(c, np.cos(ang).astype(np.float32))
    assert np.array_equal(s, np.sin(ang).astype(np.float32))
    # pair norms preserved; relative-position property <R_m q, R_n k> = f(m - n)
    r = np.random.default_rng(3)
    q = r.standard_normal((1, 1, D)).astype(np.float32)
    k = r.standard_normal((1, 1, D)).astype(np.float32)

    def rot(v, p):
        cc, ss = orc.rope_tables(np.int32([p]), D, base)
        return orc.rope_neox(v, cc, ss)[0, 0].astype(np.float64)

    assert abs(np.linalg.norm(rot(q, 123)) - np.linalg.norm(q)) < 1e-5
    d1 = rot(q, 17) @ rot(k, 5)
    d2 = rot(q, 212) @ rot(k, 200)
    assert abs(d1 - d2) < 1e-4
    # A swapped pairing (interleaved) would break this: energy of pair (i, i+D/2)
    y = rot(q, 77)
    e_in = q[0, 0, :D // 2].astype(np.float64) ** 2 + q[0, 0, D // 2:].astype(np.float64) ** 2
    e_out = y[:D // 2] ** 2 + y[D // 2:] ** 2
    assert np.allclose(e_in, e_out, atol=1e-5)


def test_rope_table_definitions_are_close_but_not_identical():
    # The CUDA twin's fp32 powf table (bitvla_lm_cuda.cu:333-342) against the
    # fp64 table the build adopts: the distance is what makes exact ggml angle
    # evaluation matter at the 1e-5 level, so it is measured, not assumed.
    D, base, n = 128, 500000.0, 520
    c64, s64 = orc.rope_tables(np.arange(n, dtype=np.int32), D, base)
    c32, s32 = orc.rope_tables_f32_powf(n, D, base)
    err = max(np.abs(c64 - c32).max(), np.abs(s64 - s32).max())
    assert err < 2e-4
    assert np.array_equal(c64[0], c32[0]) and np.array_equal(s64[0], s32[0])


# ------------------------------------------------------------ time embeddings
def _close(a, b):
    return abs(a - b) <= 1e-6 * (1.0 + abs(b))


def test_timesteps_proj_values_from_reference_test():
    # tests/test_dit_common.cpp:32-48
    out = orc.timesteps_proj(0)
    assert out.shape == (256,)
    assert all(_close(out[i], 1.0) and _close(out[128 + i], 0.0) for i in range(128))
    out = orc.timesteps_proj(250)
    lm = np.float32(math.log(10000.0))
    for i in (0, 1, 63, 127):
        emb = np.float32(250.0) * np.exp(-lm * np.float32(i) / np.float32(127.0), dtype=np.float32)
        assert _close(out[i], math.cos(emb)) and _close(out[128 + i], math.sin(emb))
    assert _close(out[0], math.cos(250.0))


def test_action_sinusoid_values_from_reference_test():
    # tests/test_dit_common.cpp:51-73
    out = orc.action_sinusoid(0, 8, 3)
    assert out.shape == (3, 8)
    assert np.allclose(out[:, :4], 0.0, atol=1e-6) and np.allclose(out[:, 4:], 1.0, atol=1e-6)
    out = orc.action_sinusoid(500, 8, 3)
    step = np.float32(math.log(10000.0)) / np.float32(4)
    for i in range(4):
        emb = np.float32(500.0) * np.exp(-np.float32(i) * step, dtype=np.float32)
        assert _close(out[0, i], math.sin(emb)) and _close(out[0, 4 + i], math.cos(emb))
    assert np.array_equal(out[1], out[0]) and np.array_equal(out[2], out[0])
    # opposite trig orders (test_dit_common.cpp:76-86)
    tp, a = orc.timesteps_proj(7), orc.action_sinusoid(7, 256, 1)[0]
    assert _close(tp[0], math.cos(7.0)) and _close(a[0], math.sin(7.0))


def test_sinusoidal_time_emb_closed_form():
    # src/layers/embed.h:61-73: log-spaced periods, sin first.
    dim, mn, mx, t = 16, 4e-3, 4.0, 0.7
    out = orc.sinusoidal_time_emb(t, dim, mn, mx)
    half = dim // 2
    frac = np.arange(half) / (half - 1)
    period = mn * (mx / mn) ** frac
    want = 2 * np.pi / period * t
    assert np.allclose(out[:half], np.sin(want), atol=1e-6)
    assert np.allclose(out[half:], np.cos(want), atol=1e-6)
    # first period is min_period, last is max_period
    assert _close(out[0], math.sin(2 * math.pi / mn * t))
    assert _close(out[half - 1], math.sin(2 * math.pi / mx * t))
    out2 = orc.sinusoidal_time_emb(t, 2, mn, mx)  # half == 1 -> frac 0
    assert _close(out2[0], math.sin(2 * math.pi / mn * t))


# -------------------------------------------------------------- linear / norm
def test_linear_matches_float64_matmul_and_is_not_transposed():
    r = np.random.default_rng(4)
    x = r.standard_normal((7, 40)).astype(np.float32)
    W = r.standard_normal((13, 40)).astype(np.float32)
    b = r.standard_normal(13).astype(np.float32)
    want = (x.astype(np.float64) @ W.astype(np.float64).T + b).astype(np.float32)
    assert np.array_equal(orc.linear(x, W, b), want)
    assert np.allclose(orc.linear(x, W, b, acc64=False), want, rtol=1e-5, atol=1e-5)
    # one-hot input picks a column of W (a transposed operand would pick a row)
    e = np.zeros((1, 40), np.float32)
    e[0, 5] = 1.0
    assert np.array_equal(orc.linear(e, W)[0], W[:, 5])


def test_norms_against_torch():
    r = np.random.default_rng(5)
    x = r.standard_normal((5, 96)).astype(np.float32) * 3 + 1
    w = r.standard_normal(96).astype(np.float32)
    b = r.standard_normal(96).astype(np.float32)
    xt = torch.from_numpy(x).double()
    rms = xt / torch.sqrt((xt * xt).mean(-1, keepdim=True) + 1e-5) * torch.from_numpy(w).double()
    assert np.allclose(orc.rms_norm(x, w, 1e-5), rms.float().numpy(), rtol=1e-6, atol=1e-6)
    ln = torch.nn.functional.layer_norm(xt, (96,), torch.from_numpy(w).double(), torch.from_numpy(b).double(), 1e-5)
    assert np.allclose(orc.layer_norm(x, w, b, 1e-5), ln.float().numpy(), rtol=1e-5, atol=1e-5)
    # rms_norm of a constant row is sign(x) (eps aside); adaLN = xn*(1+sc)+sh
    assert np.allclose(orc.rms_norm(np.full((1, 8), -3.0, np.float32), None, 0.0), -1.0)
    sc, sh = r.standard_normal(96).astype(np.float32), r.standard_normal(96).astype(np.float32)
    xn = torch.nn.functional.layer_norm(xt, (96,), None, None, 1e-5).float().numpy()
    assert np.allclose(orc.adaln(x, sc, sh, 1e-5), xn * (1 + sc) + sh, rtol=1e-5, atol=1e-5)
    # adaRMS: float64 evaluation of rms(x)*(1+scale)+shift; scale = -1 leaves the shift alone;
    # a constant row normalises to its sign, so the output is sign*(1+scale)+shift
    rn = (xt / torch.sqrt((xt * xt).mean(-1, keepdim=True) + 1e-6)).numpy()
    assert np.allclose(orc.adarms(x, sc, sh, 1e-6), rn * (1 + sc.astype(np.float64)) + sh, rtol=1e-5, atol=1e-5)
    assert np.allclose(orc.adarms(x, np.full(96, -1.0, np.float32), sh, 1e-6), np.broadcast_to(sh, x.shape), atol=1e-6)
    assert np.allclose(orc.adarms(np.full((1, 96), -2.0, np.float32), sc, sh, 0.0), -(1 + sc) + sh, atol=1e-6)
    assert np.allclose(orc.silu(np.float32([0.0, 1.0, -2.0])),
                       torch.nn.functional.silu(torch.tensor([0.0, 1.0, -2.0])).numpy(), atol=1e-7)
    # gelu, tanh form: known values, torch's tanh-approximate gelu, odd part x/2 (gelu(x) - gelu(-x) = x)
    g = orc.gelu(np.float32([0.0, 1.0, -1.0, 3.0]))
    assert np.allclose(g, [0.0, 0.8411919906, -0.1588080094, 2.9963626], atol=2e-7)
    xs = np.linspace(-6, 6, 97).astype(np.float32)
    assert np.allclose(orc.gelu(xs), torch.nn.functional.gelu(torch.tensor(xs), approximate="tanh").numpy(), atol=1e-6)
    assert np.allclose(orc.gelu(xs) - orc.gelu(-xs), xs, atol=1e-6)
    # the FFN compositions against a float64 evaluation of their definitions
    xx = r.standard_normal((5, 24)).astype(np.float32)
    Wg, Wu = r.standard_normal((32, 24)).astype(np.float32), r.standard_normal((32, 24)).astype(np.float32)
    Wd, b1, b2 = r.standard_normal((24, 32)).astype(np.float32), r.standard_normal(32).astype(np.float32), r.standard_normal(24).astype(np.float32)
    x64 = xx.astype(np.float64)
    gate = x64 @ Wg.T.astype(np.float64)
    want = ((gate / (1 + np.exp(-gate))) * (x64 @ Wu.T)) @ Wd.T.astype(np.float64)
    assert np.allclose(orc.ffn_glu(xx, Wg, Wu, Wd, orc.silu), want, rtol=1e-5, atol=1e-4)
    h = x64 @ Wg.T + b1
    want = (0.5 * h * (1 + np.tanh(np.sqrt(2 / np.pi) * h * (1 + 0.044715 * h * h)))) @ Wd.T + b2
    assert np.allclose(orc.ffn_gelu(xx, Wg, b1, Wd, b2), want, rtol=1e-5, atol=1e-4)


# ---------------------------------------------------------- concat / softmax
def test_kv_concat_is_a_byte_copy():
    r = np.random.default_rng(6)
    for dt in (np.float32, np.uint16):
        a = r.integers(0, 60000, (241, 5, 64)).astype(dt)
        b = r.integers(0, 60000, (50, 5, 64)).astype(dt)
        out = orc.kv_concat(a, b)
        assert out.shape == (291, 5, 64) and np.array_equal(out, np.concatenate([a, b], 0))
    assert orc.kv_concat(a[:0], b).shape[0] == 50  # empty cache


def test_softmax_ext_against_torch_and_masking():
    r = np.random.default_rng(7)
    kq = r.standard_normal((6, 33)).astype(np.float32) * 4
    mask = np.zeros((6, 33), np.float32)
    mask[:, 10:15] = NEG
    mask[2, 20:] = NEG
    got = orc.softmax_ext(kq, mask, 0.125)
    want = torch.softmax(torch.from_numpy(kq).double() * 0.125 + torch.from_numpy(mask).double(), -1).float().numpy()
    assert np.allclose(got, want, rtol=1e-6, atol=1e-7)
    assert np.all(got[:, 10:15] == 0) and np.allclose(got.sum(-1), 1, atol=1e-6)
    u = orc.to_bf16(kq)
    sm = orc.from_bf16(orc.softmax_scaled_bf16(u, 0.25))
    want = torch.softmax(torch.from_numpy(orc.from_bf16(u)).double() * 0.25, -1).float().numpy()
    assert np.allclose(sm, want, rtol=1e-2, atol=1e-3)


# ------------------------------------------------------------------ attention
def _sdpa(Q, K, V, mask, scale):
    S, Hq, D = Q.shape
    T, Hkv, _ = K.shape
    q = torch.from_numpy(Q).double().permute(1, 0, 2)
    k = torch.from_numpy(K).double().permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)
    v = torch.from_numpy(V).double().permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)
    m = None if mask is None else torch.from_numpy(mask).double()
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=m, scale=scale)
    return o.permute(1, 0, 2).reshape(S, Hq * D).float().numpy()


@pytest.mark.parametrize("S,T,Hq,Hkv,D", [(50, 291, 15, 5, 64), (51, 867, 8, 1, 256), (17, 296, 32, 32, 48), (1, 513, 20, 5, 128)])
def test_attention_against_torch_sdpa(S, T, Hq, Hkv, D):
    r = np.random.default_rng(8)
    Q = r.standard_normal((S, Hq, D)).astype(np.float32)
    K = r.standard_normal((T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((T, Hkv, D)).astype(np.float32)
    scale = 1.0 / math.sqrt(D)
    P = T - S if T > S else 0
    mask = orc.mask_smolvla_full(P, S, max(P - 9, 0), max(P - 1, 0)) if P > 0 else None
    for m in (None, mask):
        got = orc.attention(Q, K, V, m, scale)
        want = _sdpa(Q, K, V, m, scale)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    got32 = orc.attention(Q, K, V, mask, scale, acc64=False)
    assert np.allclose(got32, want, rtol=1e-4, atol=1e-5)


def test_attention_special_cases():
    r = np.random.default_rng(9)
    S, T, Hq, Hkv, D = 4, 12, 6, 2, 8
    K = r.standard_normal((T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((T, Hkv, D)).astype(np.float32)
    mask = np.zeros((S, T), np.float32)
    mask[:, 3:6] = NEG
    # all-zero Q -> uniform average of the unmasked V rows of the right kv head
    out = orc.attention(np.zeros((S, Hq, D), np.float32), K, V, mask, 0.3).reshape(S, Hq, D)
    keep = [t for t in range(T) if not 3 <= t < 6]
    for h in range(Hq):
        assert np.allclose(out[0, h], V[keep, h // 3].mean(0), atol=1e-6)
    # a huge logit on one key copies that V row
    Q = np.zeros((S, Hq, D), np.float32)
    Q[:, :, 0] = 1.0
    K2 = np.zeros_like(K)
    K2[7, :, 0] = 1e4
    out = orc.attention(Q, K2, V, mask, 1.0).reshape(S, Hq, D)
    assert np.allclose(out[1, 4], V[7, 1], atol=1e-6)
    # garbage in masked key columns does not change the result
    Q = r.standard_normal((S, Hq, D)).astype(np.float32)
    base = orc.attention(Q, K, V, mask, 0.3)
    K3, V3 = K.copy(), V.copy()
    K3[3:6] = 1e6
    V3[3:6] = -1e6
    assert np.array_equal(orc.attention(Q, K3, V3, mask, 0.3), base)
    # permuting unmasked keys (with their values and mask columns) changes nothing
    perm = r.permutation(T)
    out = orc.attention(Q, K[perm], V[perm], mask[:, perm], 0.3)
    assert np.allclose(out, base, rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------------- masks
def test_mask_properties():
    P, S = 241, 50
    m = orc.mask_smolvla_full(P, S, 200, 240)
    assert m.shape == (S, P + S)
    assert np.all(m[:, :200] == 0) and np.all(m[:, 200:240] == NEG) and np.all(m[:, 240] == 0)
    suf = m[:, P:]
    assert np.array_equal(suf == 0, np.tril(np.ones((S, S), bool)))  # causal
    assert np.all((m == 0).sum(1) > 0)  # no row fully masked
    assert np.array_equal(orc.mask_smolvla_prefix_only(P, S, 200, 240), m[:, :P])
    pm, pos = orc.mask_smolvla_prefill(P, 200, 240, 200)
    assert np.all(pm[:P - 1, P - 1] == NEG) and pm[P - 1, P - 1] == 0
    assert np.array_equal(pos[:P - 1], np.arange(P - 1)) and pos[P - 1] == 200
    p0 = orc.mask_pi0_full(816, 51)
    assert np.all(p0[:, :816] == 0)
    assert p0[0, 816] == 0 and np.all(p0[0, 817:] == NEG) and np.all(p0[1:, 816:] == 0)
    c = orc.mask_causal(5)
    assert np.array_equal(c == 0, np.tril(np.ones((5, 5), bool)))


# -------------------------------------------------------------------- ternary
def test_decode_hand_word_including_code_zero():
    # bitnet_kernels.h:78-88: word i = (i2s >> 2i) & 0x03030303, minus 2 per byte.
    # Byte b carries values b, b+4, b+8, b+12 at bits 0,2,4,6.
    codes = [0, 1, 2, 3, 3, 2, 1, 0, 2, 2, 1, 1, 0, 3, 0, 3]
    word = 0
    for v, c in enumerate(codes):
        b, j = v % 4, v // 4
        word |= c << (8 * b + 2 * j)
    got = orc.decode_i2s_to_i8s(word)
    assert list(got) == [c - 2 for c in codes]
    assert got[0] == -2  # code 0 is representable and decodes to -2
    assert list(orc.decode_i2s_to_i8s(0xFFFFFFFF)) == [1] * 16
    assert list(orc.decode_i2s_to_i8s(0xAAAAAAAA)) == [0] * 16


def test_pack_ladder_hand_worked_slots():
    # src/models/bitvla.cpp:453-483 worked by hand for N=16, K=256.
    N, K = 16, 256
    W = np.zeros((N, K), np.int8)
    W[0, :16] = [-1, 0, 1, 0, 1, 1, -1, 0, 0, 0, 0, 0, -1, -1, 1, 1]
    packed = orc.pack_ladder_int2(W)
    assert list(packed[:4]) == [109, 110, 231, 234]
    zero_byte = 2 | 2 << 2 | 2 << 4 | 2 << 6
    assert np.all(packed[4:8] == zero_byte)
    # slot order inside a 16-row block: y_in_half (8 rows), sub_k, y_half, major_k, k_0
    marks = {1: (1, 0), 8: (0, 16), 16: (8, 0), 32: (0, 32), 128: (0, 128)}
    for slot, (n, k) in marks.items():
        W2 = np.zeros((N, K), np.int8)
        W2[n, k] = 1
        p = orc.pack_ladder_int2(W2)
        assert p[4 * slot] == (3 | 2 << 2 | 2 << 4 | 2 << 6), slot
        assert np.count_nonzero(p != zero_byte) == 1


@pytest.mark.parametrize("N,K", [(16, 128), (640, 2560), (48, 384)])
def test_pack_unpack_round_trip_uses_two_independent_restatements(N, K):
    r = np.random.default_rng(10)
    W = r.integers(-1, 2, (N, K)).astype(np.int8)
    packed = orc.pack_ladder_int2(W)
    assert packed.size == N * K // 4
    assert np.array_equal(orc.unpack_ladder_int2(packed, N, K), W)
    # raw bytes (as the reference's GEMM check feeds them) may hold code 0 -> -2
    raw = r.integers(0, 256, N * K // 4).astype(np.uint8)
    U = orc.unpack_ladder_int2(raw, N, K)
    assert U.min() == -2 and U.max() == 1


def test_weight_quant_absmean_and_ties():
    W = np.float32([[0.5, -0.5, 1.5, -1.5], [0.2, 2.5, -3.0, 0.0]])
    t, am = orc.weight_quant_ternary(W)
    assert am == np.float32(np.abs(W.astype(np.float64)).mean())
    inv = np.float32(1.0) / am
    want = np.clip(np.rint(W * inv), -1, 1).astype(np.int8)  # rint = half to even
    assert np.array_equal(t, want)
    t0, am0 = orc.weight_quant_ternary(np.zeros((2, 2), np.float32))
    assert am0 == np.float32(1e-5) and not t0.any()
    # ties: W/absmean = +-0.5 -> 0, 1.5 -> 2 -> clamp 1
    W = np.float32([[1.0, -1.0, 3.0, -3.0]])  # absmean 2 -> 0.5, -0.5, 1.5, -1.5
    t, am = orc.weight_quant_ternary(W)
    assert am == 2.0 and list(t[0]) == [0, 0, 1, -1]


def test_act_quant_ties_floor_clamp():
    # scale = 127/amax; make amax = 127 so x*scale = x and ties are visible.
    x = np.float32([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -127.0, 3.49]])
    q, s = orc.act_quant(x)
    assert s[0] == 1.0
    assert list(q[0]) == [127, 0, 2, 2, 0, -2, -127, 3]
    q, s = orc.act_quant(np.zeros((1, 8), np.float32))
    assert s[0] == np.float32(127.0) / np.float32(1e-5) and not q.any()
    x = np.float32([[1e-6, -1e-6, 4e-6, 0]])  # below the amax floor: scale stays 127/1e-5
    q, s = orc.act_quant(x)
    assert s[0] == np.float32(127.0) / np.float32(1e-5) and list(q[0]) == [13, -13, 51, 0]
    r = np.random.default_rng(11)
    x = r.standard_normal((9, 2560)).astype(np.float32)
    q, s = orc.act_quant(x)
    amax = np.abs(x).max(1)
    assert np.array_equal(s, np.float32(127.0) / amax)
    assert np.array_equal(q, np.clip(np.rint(x * s[:, None]), -128, 127).astype(np.int8))
    assert np.abs(q).max() == 127
    fq = orc.act_fake_quant(x)
    assert np.allclose(fq, q.astype(np.float32) * (np.float32(1.0) / s)[:, None], rtol=0, atol=0)


def test_ternary_gemm_and_epilogue_brute_force():
    r = np.random.default_rng(12)
    M, N, K = 37, 48, 256
    A = r.integers(-127, 128, (M, K)).astype(np.int8)
    Wt = r.integers(-2, 2, (N, K)).astype(np.int8)
    acc = orc.ternary_gemm_i32(A, Wt)
    assert np.array_equal(acc, (A.astype(np.int64) @ Wt.astype(np.int64).T).astype(np.int32))
    s = (40 + r.integers(0, 100, M)).astype(np.float32)
    ws = (0.01 + 0.001 * r.integers(0, 50, 3)).astype(np.float32)
    out = orc.ternary_epilogue(acc, s, ws)
    g = np.arange(N) // (N // 3)
    want = orc.to_bf16((acc.astype(np.float32) / s[:, None]) * ws[g][None, :])
    assert np.array_equal(out, want)
    # worst case magnitude stays inside int32
    A = np.full((1, 2560), -128, np.int8)
    Wt = np.full((1, 2560), -2, np.int8)
    assert orc.ternary_gemm_i32(A, Wt)[0, 0] == 128 * 2 * 2560


def test_bit_linear_cpu_twin_equals_integer_path_up_to_rounding():
    # src/models/bitvla.cpp:173-176 (fp32 fake-quant GEMM) and the int8 x ternary
    # kernel compute the same number: acc / s * absmean.
    r = np.random.default_rng(13)
    M, N, K = 5, 32, 256
    x = r.standard_normal((M, K)).astype(np.float32)
    W = (r.standard_normal((N, K)) * 0.02).astype(np.float32)
    t, am = orc.weight_quant_ternary(W)
    y = orc.bit_linear_f32(x, t, am)
    q, s = orc.act_quant(x)
    acc = orc.ternary_gemm_i32(q, t)
    assert np.allclose(y, acc.astype(np.float64) / s[:, None] * am, rtol=2e-6, atol=1e-7)


def test_layout_helpers():
    r = np.random.default_rng(14)
    S, H, hd = 7, 4, 6
    x = r.integers(0, 65536, (S, H * hd)).astype(np.uint16)
    t = orc.transpose_sHd_to_Hsd(x, H)
    assert np.array_equal(t, x.reshape(S, H, hd).transpose(1, 0, 2))
    assert np.array_equal(orc.transpose_Hsd_to_sHd(t), x)
    rep = orc.repeat_kv(t[:2], 6)
    assert np.array_equal(rep, np.repeat(t[:2], 3, axis=0))  # kv_h = q_h * n_kv / n_q
    ids = np.int32([3, 3, 0, 6])
    assert np.array_equal(orc.gather_rows(x, ids), x[ids])


def test_squared_relu_glu_hand_values():
    # relu(gate)^2 * up on [gate | up]: negative gates give 0 whatever up is; 1.5^2 * -2 = -4.5;
    # the product is rounded to bf16 once (3^2 * 1.0078125 = 9.0703125 -> 9.0625)
    import oracle.chunk as orc_chunk
    gu = np.float32([[-1.0, 1.5, 3.0, 0.0, 7.0, -2.0, 1.0078125, 5.0]])
    assert list(orc_chunk.sqrelu_mul(gu, 4)[0]) == [0.0, -4.5, 9.0625, 0.0]
