"""Kernel-level parity on a real MI355X: every C-ABI entry point against the CPU
oracle on the same seeded inputs.

Bars: bit-exact for copies / integer work (KV append+gather, layout helpers,
act-quant, ternary int32 accumulators and their bf16 epilogue); fp32 kernels
within 1e-5 relative (max-abs error over max-abs value); bf16 kernels within
2e-2 relative / 1e-2 absolute.
"""
import ctypes
import math

import numpy as np
import pytest
import torch

import oracle as orc
from conftest import mt19937_raw
from util import dev, host, pkg, rel_err

pytestmark = pytest.mark.gpu

F32, BF16 = pkg.VLA_DT_F32, pkg.VLA_DT_BF16
FP32_TOL = 1e-5


def sync():
    torch.cuda.synchronize()


def bf16_close(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) <= 1e-2 + 2e-2 * np.abs(want)))


def as_f32(t, dtype):
    a = host(t)
    return orc.from_bf16(a.view(np.uint16)) if dtype == BF16 else a


def to_dev(a, dtype):
    return dev(orc.to_bf16(a)) if dtype == BF16 else dev(np.asarray(a, np.float32))


def empty(shape, dtype):
    return torch.zeros(shape, dtype=torch.int16 if dtype == BF16 else torch.float32, device="cuda")


# ------------------------------------------------------------------ KV cache
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("B,Hkv,D,P,S", [(1, 5, 64, 241, 50), (3, 1, 256, 816, 51), (2, 32, 48, 296, 0), (2, 5, 128, 512, 7)])
def test_kv_append_then_gather_is_the_reference_concat(dtype, B, Hkv, D, P, S):
    r = np.random.default_rng(100 + B + D)
    npdt = np.uint16 if dtype == BF16 else np.float32
    mk = lambda n: (r.integers(0, 65536, (B, n, Hkv, D)).astype(np.uint16) if dtype == BF16
                    else r.standard_normal((B, n, Hkv, D)).astype(np.float32))
    kp, vp, ks, vs = mk(P), mk(P), mk(S), mk(S)
    t_max = (P + S + 63) // 64 * 64
    kc, vc = empty((B, Hkv, t_max, D), dtype), empty((B, Hkv, D, t_max), dtype)
    pkg.call("vla_kv_append", kc, vc, dev(kp), dev(vp), dtype, B, Hkv, D, t_max, 0, P)
    # two denoise steps overwrite the same suffix slots; the prefix is untouched
    junk = mk(S)
    pkg.call("vla_kv_append", kc, vc, dev(junk), dev(junk), dtype, B, Hkv, D, t_max, P, S)
    pkg.call("vla_kv_append", kc, vc, dev(ks), dev(vs), dtype, B, Hkv, D, t_max, P, S)
    kd, vd = empty((B, P + S, Hkv, D), dtype), empty((B, P + S, Hkv, D), dtype)
    pkg.call("vla_kv_gather", kc, vc, kd, vd, dtype, B, Hkv, D, t_max, 0, P + S)
    sync()
    for b in range(B):
        assert np.array_equal(host(kd, npdt)[b], orc.kv_concat(kp[b], ks[b]))
        assert np.array_equal(host(vd, npdt)[b], orc.kv_concat(vp[b], vs[b]))
    # layouts: K [B][Hkv][t][D], V^T [B][Hkv][D][t]
    assert np.array_equal(host(kc, npdt)[:, :, :P], kp.transpose(0, 2, 1, 3))
    assert np.array_equal(host(vc, npdt)[:, :, :, :P], vp.transpose(0, 2, 3, 1))
    lib = pkg.lib()
    assert lib.vla_kv_append(kc.data_ptr(), vc.data_ptr(), kd.data_ptr(), vd.data_ptr(), dtype, B, Hkv, D, t_max,
                             t_max - 1, 2, None) == pkg.VLA_K_ERR_SHAPE


# --------------------------------------------------------------- RoPE / norms
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_rope_neox(dtype):
    r = np.random.default_rng(101)
    B, S, H, D = 2, 50, 15, 64
    x = r.standard_normal((B * S, H, D)).astype(np.float32)
    if dtype == BF16:
        x = orc.round_bf16(x)
    pos = np.arange(S, dtype=np.int32) + 242
    c, s = orc.rope_tables(pos, D, 10000.0)
    xd = to_dev(x, dtype)
    pkg.call("vla_rope_neox", xd, dev(c), dev(s), dtype, B * S, S, H, D)
    sync()
    want = np.concatenate([orc.rope_neox(x[b * S:(b + 1) * S], c, s) for b in range(B)])
    got = as_f32(xd, dtype)
    if dtype == F32:
        assert rel_err(got, want) < 1e-6
    else:
        assert np.array_equal(got, orc.round_bf16(want)) or bf16_close(got, want)


def test_bitvla_rope_head_major_bf16():
    r = np.random.default_rng(102)
    H, S, D = 20, 37, 128
    x = orc.round_bf16(r.standard_normal((H, S, D)).astype(np.float32))
    c, s = orc.rope_tables(np.arange(S, dtype=np.int32), D, 500000.0)
    xd = dev(orc.to_bf16(x))
    pkg.call("bitvla_rope_neox_bf16", xd, dev(c), dev(s), H, S, D)
    sync()
    want = orc.rope_neox(x.transpose(1, 0, 2).copy(), c, s).transpose(1, 0, 2)
    got = orc.from_bf16(host(xd, np.uint16))
    assert bf16_close(got, want) and rel_err(got, want) < 8e-3


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("M,K", [(50, 720), (51, 1024), (17, 1536), (3, 2560), (1600, 720), (816, 1024), (1088, 1536), (200, 4096), (65, 724)])
def test_rms_norm_and_adaln(dtype, M, K):
    r = np.random.default_rng(103)
    x = (r.standard_normal((M, K)) * 2 + 0.5).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(K)).astype(np.float32)
    sc, sh = (0.1 * r.standard_normal(K)).astype(np.float32), (0.1 * r.standard_normal(K)).astype(np.float32)
    if dtype == BF16:
        x, w = orc.round_bf16(x), orc.round_bf16(w)
    y = empty((M, K), dtype)
    pkg.call("vla_rms_norm", to_dev(x, dtype), to_dev(w, dtype), y, dtype, M, K, 1e-5)
    y2 = empty((M, K), dtype)
    pkg.call("vla_adaln", to_dev(x, dtype), dev(sc), dev(sh), y2, dtype, M, K, 1e-5)
    sync()
    want, want2 = orc.rms_norm(x, w, 1e-5), orc.adaln(x, sc, sh, 1e-5)
    if dtype == F32:
        assert rel_err(host(y), want) < FP32_TOL and rel_err(host(y2), want2) < FP32_TOL
    else:
        assert bf16_close(as_f32(y, dtype), want) and bf16_close(as_f32(y2, dtype), want2)
    if dtype == BF16:  # the BitVLA-named entry point is the same kernel
        y3 = empty((M, K), dtype)
        pkg.call("bitvla_rmsnorm_bf16", to_dev(x, dtype), to_dev(w, dtype), y3, 1e-5, M, K)
        sync()
        assert np.array_equal(host(y3), host(y))


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("M,K,N", [(50, 1024, 1024), (800, 1024, 1024), (50, 4096, 1024), (7, 720, 200)])
def test_adarms_and_gated_residual_projection(dtype, M, K, N):
    """pi0.5's norm and its gated residual (src/models/pi05.cpp:208-224, 273-282):
    y = rms(x) (1 + scale) + shift;  out = residual + (x W^T) * gate[column]."""
    r = np.random.default_rng(140 + M)
    x = (r.standard_normal((M, K)) * 2 + 0.5).astype(np.float32)
    sc, sh = (0.2 * r.standard_normal(K)).astype(np.float32), (0.2 * r.standard_normal(K)).astype(np.float32)
    W = (0.02 * r.standard_normal((N, K))).astype(np.float32)
    gate = (1 + 0.2 * r.standard_normal(N)).astype(np.float32)
    res = r.standard_normal((M, N)).astype(np.float32)
    if dtype == BF16:
        x, W, res = orc.round_bf16(x), orc.round_bf16(W), orc.round_bf16(res)
    y = empty((M, K), dtype)
    pkg.call("vla_adarms", to_dev(x, dtype), dev(sc), dev(sh), y, dtype, M, K, 1e-6)
    out = empty((M, N), dtype)
    pkg.call("vla_linear_gated", to_dev(x, dtype), to_dev(W, dtype), None, dev(gate), to_dev(res, dtype), out, dtype, dtype, M, N, K)
    ones = torch.ones(N, dtype=torch.float32, device="cuda")
    plain = empty((M, N), dtype)
    pkg.call("vla_linear_gated", to_dev(x, dtype), to_dev(W, dtype), None, ones, to_dev(res, dtype), plain, dtype, dtype, M, N, K)
    ref = empty((M, N), dtype)
    pkg.call("vla_linear", to_dev(x, dtype), to_dev(W, dtype), None, to_dev(res, dtype), ref, dtype, dtype, M, N, K)
    sync()
    want_y = orc.adarms(x, sc, sh, 1e-6)
    want = res + orc.linear(x, W) * gate
    if dtype == F32:
        assert rel_err(host(y), want_y) < FP32_TOL and rel_err(host(out), want) < FP32_TOL
    else:
        assert bf16_close(as_f32(y, dtype), want_y) and bf16_close(as_f32(out, dtype), want)
    assert np.array_equal(host(plain), host(ref))  # a gate of ones: the plain projection, bit for bit
    with pytest.raises(RuntimeError):  # the gate is not optional
        pkg.call("vla_linear_gated", to_dev(x, dtype), to_dev(W, dtype), None, None, to_dev(res, dtype), plain, dtype, dtype, M, N, K)


# ---------------------------------------------------------------- projections
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("M,N,K", [(50, 720, 960), (1, 64, 128), (130, 200, 72), (17, 1536, 1536), (64, 32, 720)])
def test_linear_bias_residual(dtype, M, N, K):
    r = np.random.default_rng(104 + M)
    x = r.standard_normal((M, K)).astype(np.float32)
    W = (0.02 * r.standard_normal((N, K))).astype(np.float32)
    b = (0.1 * r.standard_normal(N)).astype(np.float32)
    res = r.standard_normal((M, N)).astype(np.float32)
    if dtype == BF16:
        x, W, res = orc.round_bf16(x), orc.round_bf16(W), orc.round_bf16(res)
    y = empty((M, N), dtype)
    pkg.call("vla_linear", to_dev(x, dtype), to_dev(W, dtype), dev(b), to_dev(res, dtype), y, dtype, dtype, M, N, K)
    y0 = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    pkg.call("vla_linear", to_dev(x, dtype), to_dev(W, dtype), None, None, y0, dtype, F32, M, N, K)
    sync()
    want0 = orc.linear(x, W)
    want = want0 + b + res
    if dtype == F32:
        assert rel_err(host(y), want) < FP32_TOL and rel_err(host(y0), want0) < FP32_TOL
    else:
        assert rel_err(host(y0), want0) < 1e-5  # fp32 accumulate of exact bf16 products
        assert bf16_close(as_f32(y, dtype), want)


@pytest.mark.parametrize("M,N,K", [(50, 720, 960), (3, 37, 2048), (64, 1601, 52), (33, 8, 4), (50, 64, 2052)])
def test_fp32_rows_of_one_observation_take_the_fma_kernel(M, N, K, monkeypatch):
    """At most 64 fp32 rows go through the FMA kernel (8 columns per workgroup, 16 partial sums
    per output).  It and the MFMA kernel (pinned with VLA_GEMM_TILE) against the oracle at the
    fp32 bar and against each other, with ragged N, K not a multiple of 64, bias, activation,
    column gate and residual."""
    r = np.random.default_rng(1700 + N)
    x = r.standard_normal((M, K)).astype(np.float32)
    W = (r.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    b = (0.1 * r.standard_normal(N)).astype(np.float32)
    gate = (1.0 + 0.2 * r.standard_normal(N)).astype(np.float32)
    res = r.standard_normal((M, N)).astype(np.float32)
    outs = []
    for tile in (None, "4"):
        if tile is None:
            monkeypatch.delenv("VLA_GEMM_TILE", raising=False)
        else:
            monkeypatch.setenv("VLA_GEMM_TILE", tile)
        pkg.lib().vla_kernels_reload_env()
        y, y2, y3 = empty((M, N), F32), empty((M, N), F32), empty((M, N), BF16)
        pkg.call("vla_linear_act", dev(x), dev(W), dev(b), dev(res), y, F32, F32, M, N, K, pkg.VLA_ACT_SILU)
        pkg.call("vla_linear_gated", dev(x), dev(W), None, dev(gate), dev(res), y2, F32, F32, M, N, K)
        pkg.call("vla_linear", dev(x), dev(W), dev(b), to_dev(orc.round_bf16(res), BF16), y3, F32, BF16, M, N, K)
        sync()
        outs.append((host(y), host(y2), as_f32(y3, BF16)))
    monkeypatch.delenv("VLA_GEMM_TILE", raising=False)
    pkg.lib().vla_kernels_reload_env()
    lin = orc.linear(x, W)
    want = orc.silu(lin + b) + res
    want2 = lin * gate + res
    want3 = lin + b + orc.round_bf16(res)
    for got, got2, got3 in outs:
        assert rel_err(got, want) < FP32_TOL and rel_err(got2, want2) < FP32_TOL
        assert bf16_close(got3, want3)
    assert rel_err(outs[0][0], outs[1][0]) < FP32_TOL


@pytest.mark.parametrize("M,N,K", [(150, 720, 720), (333, 200, 1104), (64, 1600, 48)])
def test_linear_bf16_every_kernel_and_tiling_gives_the_same_bits(tune, M, N, K):
    """The direct-to-LDS kernel and the register-staged one, in every tile configuration, add
    the products of a row in the same order (ascending k, 16 at a time): identical outputs,
    including partial k-tiles (K not a multiple of 64 or 128) and ragged M and N."""
    r = np.random.default_rng(1040 + M)
    x = orc.round_bf16(r.standard_normal((M, K)).astype(np.float32))
    W = orc.round_bf16((0.05 * r.standard_normal((N, K))).astype(np.float32))
    res = orc.round_bf16(r.standard_normal((M, N)).astype(np.float32))
    xd, Wd, rd = to_dev(x, BF16), to_dev(W, BF16), to_dev(res, BF16)
    outs = {}
    for dl, tile, stages in [("0", t, "0") for t in "01234"] + [("1", t, ns) for t in "01234" for ns in "234"] + [("1", "5", "0")]:
        if True:
            tune.set("VLA_GEMM_DL", dl)
            tune.set("VLA_GEMM_TILE", tile)
            tune.set("VLA_GEMM_STAGES", stages)
            y = torch.zeros((M, N), dtype=torch.float32, device="cuda")
            pkg.call("vla_linear", xd, Wd, None, None, y, BF16, F32, M, N, K)
            yb = empty((M, N), BF16)
            pkg.call("vla_linear", xd, Wd, None, rd, yb, BF16, BF16, M, N, K)
            sync()
            outs[(dl, tile, stages)] = (host(y), host(yb))
    want = orc.linear(x, W)
    first = outs[("0", "0", "0")]
    assert rel_err(first[0], want) < 1e-5
    assert bf16_close(orc.from_bf16(first[1].view(np.uint16)), want + res)
    for key, (y, yb) in outs.items():
        assert np.array_equal(y, first[0]), key
        assert np.array_equal(yb.view(np.uint16), first[1].view(np.uint16)), key


@pytest.mark.parametrize("rows_max", [32, 64])
@pytest.mark.parametrize("M,N,K", [(17, 1536, 1536), (1, 64, 128), (5, 200, 720), (32, 96, 2048), (50, 720, 960), (64, 24, 72)])
def test_few_bf16_rows_take_the_split_k_kernel(tune, rows_max, M, N, K):
    """A few bf16 rows through a projection: 16 columns per workgroup, K split over its
    wavefronts (up to 32 rows by default, up to 64 when asked).  Against the oracle and against
    the tiled kernel, with bias, residual, fp32 output, ragged N (not a multiple of 16) and K
    (not a multiple of 32).  The sums are formed in another order than by the tiled kernel."""
    r = np.random.default_rng(7100 + M + N)
    x = orc.round_bf16(r.standard_normal((M, K)).astype(np.float32))
    W = orc.round_bf16((0.05 * r.standard_normal((N, K))).astype(np.float32))
    b = (0.1 * r.standard_normal(N)).astype(np.float32)
    res = orc.round_bf16(r.standard_normal((M, N)).astype(np.float32))
    xd, Wd, rd = to_dev(x, BF16), to_dev(W, BF16), to_dev(res, BF16)

    def run():
        y = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        pkg.call("vla_linear", xd, Wd, None, None, y, BF16, F32, M, N, K)
        yb = torch.zeros((M, N), dtype=torch.int16, device="cuda")
        pkg.call("vla_linear", xd, Wd, dev(b), rd, yb, BF16, BF16, M, N, K)
        yi = rd.clone()  # in place: the residual is the output
        pkg.call("vla_linear", xd, Wd, dev(b), yi, yi, BF16, BF16, M, N, K)
        sync()
        return host(y), as_f32(yb, BF16), as_f32(yi, BF16)

    tune.set("VLA_GEMM_ROWS_MAX", rows_max)
    got = run()
    tune.set("VLA_GEMM_ROWS_MAX", 0)
    tiled = run()
    want = orc.linear(x, W)
    assert rel_err(got[0], want) < 1e-5 and rel_err(tiled[0], want) < 1e-5
    assert bf16_close(got[1], want + b + res) and np.array_equal(got[1], got[2])
    assert rel_err(got[0], tiled[0]) < 1e-5 and rel_err(got[1], tiled[1]) < 8e-3


@pytest.mark.parametrize("rows_max", [32, 64])
@pytest.mark.parametrize("name,B,S,Hq,Hkv,D,K,norm,rope,self_layer", [
    ("gr00t-self-1", 1, 17, 32, 32, 48, 1536, "layer", False, True),
    ("gr00t-cross-q-1", 1, 17, 32, 32, 48, 1536, "layer", False, False),
    ("smolvla-self-1", 1, 50, 15, 5, 64, 720, "rms", True, True),
    ("pi0-1", 1, 51, 8, 1, 256, 1024, "rms", True, True),
    ("two-short-observations", 2, 9, 4, 2, 64, 328, "none", True, True),
    ("bitvla-shape", 1, 7, 20, 5, 128, 256, "none", True, True),
])
def test_few_bf16_rows_fused_qkv_on_the_split_k_kernel(tune, rows_max, name, B, S, Hq, Hkv, D, K, norm, rope, self_layer):
    """The fused Q | K | V projection of a few rows on the split-K kernel: plain, with the RMS
    pre-norm and with the modulated LayerNorm taken inside, rotation pairs, append at an offset
    into the caches; against the oracle and against the tiled kernel."""
    r = np.random.default_rng(7200 + K + S)
    M, P = B * S, 11
    nkv = Hkv if self_layer else 0
    N = (Hq + 2 * nkv) * D
    eps = 1e-5
    x = orc.round_bf16((2.0 * r.standard_normal((M, K)) * (1.0 + 3.0 * r.random((M, 1))) + 1.5 * r.standard_normal((M, 1))).astype(np.float32))
    W = orc.round_bf16((0.02 * r.standard_normal((N, K))).astype(np.float32))
    b = (0.1 * r.standard_normal(N)).astype(np.float32)
    sc, sh = (0.3 * r.standard_normal(K)).astype(np.float32), (0.3 * r.standard_normal(K)).astype(np.float32)
    g = orc.round_bf16((1.0 + 0.3 * r.standard_normal(K)).astype(np.float32))
    c, s_ = orc.rope_tables(np.arange(S, dtype=np.int32) + P + 1, D, 10000.0)
    cd, sd = (dev(c), dev(s_)) if rope else (None, None)
    t_max = (P + S + 63) // 64 * 64

    def run():
        kc, vc = empty((B, Hkv, t_max, D), BF16), empty((B, Hkv, D, t_max), BF16)
        q = empty((M, Hq * D), BF16)
        if norm == "layer":
            Wf, cs, bs = np.empty((N, K), np.uint16), np.empty(N, np.float32), np.empty(N, np.float32)
            assert pkg.lib().vla_fold_adaln_weight_host(orc.to_bf16(W).ctypes.data, b.ctypes.data, sc.ctypes.data, sh.ctypes.data, N, K,
                                                        Wf.ctypes.data, cs.ctypes.data, bs.ctypes.data) == 0
            pkg.call("vla_layernorm_attn_qkv_rope", to_dev(x, BF16), dev(Wf), dev(cs), dev(bs), BF16, M, K, S, Hq, Hkv,
                     int(self_layer), int(self_layer), D, cd, sd, q, kc, vc, t_max, P, eps)
        elif norm == "rms":
            Wf = np.empty((N, K), np.uint16)
            assert pkg.lib().vla_fold_norm_weight_host(orc.to_bf16(W).ctypes.data, orc.to_bf16(g).ctypes.data, BF16, N, K, Wf.ctypes.data) == 0
            pkg.call("vla_rmsnorm_attn_qkv_rope", to_dev(x, BF16), dev(Wf), dev(b), BF16, M, K, S, Hq, Hkv, int(self_layer),
                     int(self_layer), D, cd, sd, q, kc, vc, t_max, P, eps)
        else:
            pkg.call("vla_attn_qkv_rope", to_dev(x, BF16), to_dev(W, BF16), dev(b), BF16, M, K, S, Hq, Hkv, int(self_layer),
                     int(self_layer), D, cd, sd, q, kc, vc, t_max, P)
        out = [as_f32(q, BF16).reshape(M, Hq, D)]
        if self_layer:
            kd, vd = empty((B, S, Hkv, D), BF16), empty((B, S, Hkv, D), BF16)
            pkg.call("vla_kv_gather", kc, vc, kd, vd, BF16, B, Hkv, D, t_max, P, S)
            out += [as_f32(kd, BF16).reshape(M, Hkv, D), as_f32(vd, BF16).reshape(M, Hkv, D)]
        sync()
        return out

    xin = orc.adaln(x, sc, sh, eps) if norm == "layer" else (orc.rms_norm(x, g, eps) if norm == "rms" else x)
    y = orc.linear(xin, W, b)
    want = [y[:, :Hq * D].reshape(M, Hq, D)]
    if self_layer:
        want += [y[:, Hq * D:(Hq + Hkv) * D].reshape(M, Hkv, D), y[:, (Hq + Hkv) * D:].reshape(M, Hkv, D)]
    if rope:
        for i in range(min(2, len(want))):
            want[i] = np.concatenate([orc.rope_neox(want[i][bb * S:(bb + 1) * S], c, s_) for bb in range(B)])
    tune.set("VLA_GEMM_ROWS_MAX", rows_max)
    got = run()
    tune.set("VLA_GEMM_ROWS_MAX", 0)
    tiled = run()
    for gf, gt, w in zip(got, tiled, want):
        assert bf16_close(gf, w) and rel_err(gf, w) < 8e-3
        assert rel_err(gf, gt) < 8e-3


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("name,B,S,Hq,Hkv,D,K,rope,bias,P", [
    ("smolvla-self", 2, 50, 15, 5, 64, 720, True, False, 241),
    ("pi0", 1, 51, 8, 1, 256, 1024, True, False, 816),
    ("dit-self", 2, 17, 32, 32, 48, 1536, False, True, 0),
    ("bitvla-shape", 1, 7, 20, 5, 128, 256, True, False, 512),
])
def test_fused_qkv_rope_append(dtype, name, B, S, Hq, Hkv, D, K, rope, bias, P):
    r = np.random.default_rng(105)
    M, N = B * S, (Hq + 2 * Hkv) * D
    x = r.standard_normal((M, K)).astype(np.float32)
    W = (0.02 * r.standard_normal((N, K))).astype(np.float32)
    bvec = (0.1 * r.standard_normal(N)).astype(np.float32) if bias else None
    if dtype == BF16:
        x, W = orc.round_bf16(x), orc.round_bf16(W)
    c, s = orc.rope_tables(np.arange(S, dtype=np.int32) + P + 1, D, 10000.0)
    t_max = (P + S + 63) // 64 * 64
    kc, vc = empty((B, Hkv, t_max, D), dtype), empty((B, Hkv, D, t_max), dtype)
    q = empty((M, Hq * D), dtype)
    pkg.call("vla_attn_qkv_rope", to_dev(x, dtype), to_dev(W, dtype), None if bvec is None else dev(bvec), dtype, M, K, S,
             Hq, Hkv, 1, 1, D, dev(c) if rope else None, dev(s) if rope else None, q, kc, vc, t_max, P)
    kd, vd = empty((B, S, Hkv, D), dtype), empty((B, S, Hkv, D), dtype)
    pkg.call("vla_kv_gather", kc, vc, kd, vd, dtype, B, Hkv, D, t_max, P, S)
    sync()
    y = orc.linear(x, W, bvec)
    qw = y[:, :Hq * D].reshape(M, Hq, D)
    kw = y[:, Hq * D:(Hq + Hkv) * D].reshape(M, Hkv, D)
    vw = y[:, (Hq + Hkv) * D:].reshape(M, Hkv, D)
    if rope:
        qw = np.concatenate([orc.rope_neox(qw[b * S:(b + 1) * S], c, s) for b in range(B)])
        kw = np.concatenate([orc.rope_neox(kw[b * S:(b + 1) * S], c, s) for b in range(B)])
    gq = as_f32(q, dtype).reshape(M, Hq, D)
    gk = as_f32(kd, dtype).reshape(M, Hkv, D)
    gv = as_f32(vd, dtype).reshape(M, Hkv, D)
    if dtype == F32:
        assert rel_err(gq, qw) < FP32_TOL and rel_err(gk, kw) < FP32_TOL and rel_err(gv, vw) < FP32_TOL
    else:
        assert bf16_close(gq, qw) and bf16_close(gk, kw) and bf16_close(gv, vw)
        assert rel_err(gq, qw) < 8e-3
    # the prefix region of the cache was not touched
    assert not host(kc)[:, :, :P].any() and not host(vc)[:, :, :, :P].any()


@pytest.mark.parametrize("name,B,S,Hq,Hkv,D,K,self_layer,P", [
    ("smolvla-self", 2, 50, 15, 5, 64, 720, True, 241),
    ("smolvla-cross-q", 3, 50, 15, 5, 64, 720, False, 0),
    ("pi0", 1, 51, 8, 1, 256, 1024, True, 816),
    ("one-partial-k-tile", 1, 5, 2, 1, 64, 48, True, 3),
])
def test_rmsnorm_inside_qkv_launch(name, B, S, Hq, Hkv, D, K, self_layer, P):
    """Pre-norm taken inside the projection launch (norm weight folded into W on the host,
    rows scaled by rsqrt(mean square + eps) in the epilogue) against the oracle's
    rms_norm -> linear -> rope, and against the two-launch GPU path."""
    r = np.random.default_rng(1105 + K)
    M = B * S
    nkv = Hkv if self_layer else 0
    N = (Hq + 2 * nkv) * D
    eps = 1e-5
    x = orc.round_bf16((3.0 * r.standard_normal((M, K)) * (1.0 + r.random((M, 1)) * 4)).astype(np.float32))
    g = orc.round_bf16((1.0 + 0.3 * r.standard_normal(K)).astype(np.float32))
    W = orc.round_bf16((0.02 * r.standard_normal((N, K))).astype(np.float32))
    c, s_ = orc.rope_tables(np.arange(S, dtype=np.int32) + P + 1, D, 10000.0)
    t_max = (P + S + 63) // 64 * 64

    def run(fused):
        kc, vc = empty((B, Hkv, t_max, D), BF16), empty((B, Hkv, D, t_max), BF16)
        q = empty((M, Hq * D), BF16)
        if fused:
            Wf = np.empty((N, K), np.uint16)
            assert pkg.lib().vla_fold_norm_weight_host(orc.to_bf16(W).ctypes.data, orc.to_bf16(g).ctypes.data, BF16, N, K,
                                                       Wf.ctypes.data) == 0
            pkg.call("vla_rmsnorm_attn_qkv_rope", to_dev(x, BF16), dev(Wf), None, BF16, M, K, S, Hq, Hkv, int(self_layer),
                     int(self_layer), D, dev(c), dev(s_), q, kc, vc, t_max, P, eps)
        else:
            hn = empty((M, K), BF16)
            pkg.call("vla_rms_norm", to_dev(x, BF16), to_dev(g, BF16), hn, BF16, M, K, eps)
            pkg.call("vla_attn_qkv_rope", hn, to_dev(W, BF16), None, BF16, M, K, S, Hq, Hkv, int(self_layer),
                     int(self_layer), D, dev(c), dev(s_), q, kc, vc, t_max, P)
        out = [as_f32(q, BF16).reshape(M, Hq, D)]
        if self_layer:
            kd, vd = empty((B, S, Hkv, D), BF16), empty((B, S, Hkv, D), BF16)
            pkg.call("vla_kv_gather", kc, vc, kd, vd, BF16, B, Hkv, D, t_max, P, S)
            out += [as_f32(kd, BF16).reshape(M, Hkv, D), as_f32(vd, BF16).reshape(M, Hkv, D)]
        sync()
        return out

    y = orc.linear(orc.rms_norm(x, g, eps), W)
    want = [y[:, :Hq * D].reshape(M, Hq, D)]
    if self_layer:
        want += [y[:, Hq * D:(Hq + Hkv) * D].reshape(M, Hkv, D), y[:, (Hq + Hkv) * D:].reshape(M, Hkv, D)]
    for i in range(min(2, len(want))):  # Q and K are rotated, V is not
        want[i] = np.concatenate([orc.rope_neox(want[i][b * S:(b + 1) * S], c, s_) for b in range(B)])
    fused, pair = run(True), run(False)
    for gf, gp, w in zip(fused, pair, want):
        assert bf16_close(gf, w) and rel_err(gf, w) < 8e-3
        assert rel_err(gf, gp) < 8e-3


@pytest.mark.parametrize("name,B,S,Hq,Hkv,D,K,self_layer,bias", [
    ("gr00t-self", 3, 17, 32, 32, 48, 1536, True, True),
    ("gr00t-cross-q", 64, 17, 32, 32, 48, 1536, False, True),
    ("64-wide-heads", 2, 17, 24, 24, 64, 1536, True, True),
    ("small-no-bias", 2, 5, 2, 2, 64, 48, True, False),
    ("partial-row-tile", 1, 33, 4, 4, 64, 272, False, True),
])
def test_modulated_layernorm_inside_qkv_launch(name, B, S, Hq, Hkv, D, K, self_layer, bias):
    """A DiT block's adaLN taken inside the projection launch ((1 + scale) folded into W, the
    shift into the bias, rows centred and scaled in the epilogue from sums taken over the
    operand tiles) against the oracle's adaln -> linear, and against the two-launch GPU path.
    Rows carry a mean of the size of their spread, so a dropped mean term fails."""
    r = np.random.default_rng(2207 + K)
    M = B * S
    nkv = Hkv if self_layer else 0
    N = (Hq + 2 * nkv) * D
    eps = 1e-5
    x = orc.round_bf16((2.0 * r.standard_normal((M, K)) * (1.0 + 3.0 * r.random((M, 1))) + 1.5 * r.standard_normal((M, 1))).astype(np.float32))
    sc = (0.3 * r.standard_normal(K)).astype(np.float32)
    sh = (0.3 * r.standard_normal(K)).astype(np.float32)
    W = orc.round_bf16((0.02 * r.standard_normal((N, K))).astype(np.float32))
    b = (0.1 * r.standard_normal(N)).astype(np.float32) if bias else None
    t_max = (S + 63) // 64 * 64

    def run(fused):
        kc, vc = empty((B, Hkv, t_max, D), BF16), empty((B, Hkv, D, t_max), BF16)
        q = empty((M, Hq * D), BF16)
        if fused:
            Wf, cs, bs = np.empty((N, K), np.uint16), np.empty(N, np.float32), np.empty(N, np.float32)
            assert pkg.lib().vla_fold_adaln_weight_host(orc.to_bf16(W).ctypes.data, None if b is None else b.ctypes.data,
                                                        sc.ctypes.data, sh.ctypes.data, N, K, Wf.ctypes.data, cs.ctypes.data,
                                                        bs.ctypes.data) == 0
            pkg.call("vla_layernorm_attn_qkv_rope", to_dev(x, BF16), dev(Wf), dev(cs), dev(bs), BF16, M, K, S, Hq, Hkv,
                     int(self_layer), int(self_layer), D, None, None, q, kc, vc, t_max, 0, eps)
        else:
            hn = empty((M, K), BF16)
            pkg.call("vla_adaln", to_dev(x, BF16), dev(sc), dev(sh), hn, BF16, M, K, eps)
            pkg.call("vla_attn_qkv_rope", hn, to_dev(W, BF16), None if b is None else dev(b), BF16, M, K, S, Hq, Hkv,
                     int(self_layer), int(self_layer), D, None, None, q, kc, vc, t_max, 0)
        out = [as_f32(q, BF16).reshape(M, Hq, D)]
        if self_layer:
            kd, vd = empty((B, S, Hkv, D), BF16), empty((B, S, Hkv, D), BF16)
            pkg.call("vla_kv_gather", kc, vc, kd, vd, BF16, B, Hkv, D, t_max, 0, S)
            out += [as_f32(kd, BF16).reshape(M, Hkv, D), as_f32(vd, BF16).reshape(M, Hkv, D)]
        sync()
        return out

    y = orc.linear(orc.adaln(x, sc, sh, eps), W, b)
    want = [y[:, :Hq * D].reshape(M, Hq, D)]
    if self_layer:
        want += [y[:, Hq * D:(Hq + Hkv) * D].reshape(M, Hkv, D), y[:, (Hq + Hkv) * D:].reshape(M, Hkv, D)]
    fused, pair = run(True), run(False)
    for gf, gp, w in zip(fused, pair, want):
        assert bf16_close(gf, w) and rel_err(gf, w) < 8e-3
        assert rel_err(gf, gp) < 8e-3
    # the mean term matters at this input: a norm that does not centre the rows is far outside the bar
    assert rel_err(orc.linear(orc.rms_norm(x, None, eps) * (1 + sc) + sh, W, b)[:, :Hq * D].reshape(M, Hq, D), want[0]) > 5e-2
    # fp32 rows are not served by this launch
    assert pkg.lib().vla_layernorm_attn_qkv_rope(x.ctypes.data, W.ctypes.data, sc.ctypes.data, None, F32, M, K, S, Hq, Hkv, 0, 0, D,
                                                 None, None, x.ctypes.data, None, None, t_max, 0, eps, None) == pkg.VLA_K_ERR_SHAPE


@pytest.mark.parametrize("B,S,H,K,bias", [(64, 17, 32, 1536, True), (3, 17, 32, 1536, True), (9, 17, 8, 256, False), (5, 5, 8, 320, True),
                                          (1, 32, 16, 448, True), (11, 16, 8, 256, True)])
def test_dit_self_block_front_half_in_one_launch(B, S, H, K, bias):
    """adaLN -> Q / K / V -> attention of each observation's tokens over themselves
    (src/modules/dit_head.cpp:111-125 with enc = nullptr) as one launch, against the oracle's
    adaln -> linear -> attention with Q, K, V rounded to bf16 as both GPU paths keep them, and
    against the two-launch path.  Batches that do not fill the last workgroup's eight
    observations, few heads, short K; rows carry a mean of the size of their spread."""
    D = 48
    r = np.random.default_rng(4100 + B * S + K)
    M, N = B * S, 3 * H * D
    eps, scale = 1e-5, 1.0 / np.sqrt(D)
    x = orc.round_bf16((2.0 * r.standard_normal((M, K)) * (1.0 + 3.0 * r.random((M, 1))) + 1.5 * r.standard_normal((M, 1))).astype(np.float32))
    sc = (0.3 * r.standard_normal(K)).astype(np.float32)
    sh = (0.3 * r.standard_normal(K)).astype(np.float32)
    W = orc.round_bf16((r.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))  # scores of about one unit: the softmax is far from uniform
    b = (0.1 * r.standard_normal(N)).astype(np.float32) if bias else None
    Wf, cs, bs = np.empty((N, K), np.uint16), np.empty(N, np.float32), np.empty(N, np.float32)
    assert pkg.lib().vla_fold_adaln_weight_host(orc.to_bf16(W).ctypes.data, None if b is None else b.ctypes.data, sc.ctypes.data,
                                                sh.ctypes.data, N, K, Wf.ctypes.data, cs.ctypes.data, bs.ctypes.data) == 0
    dWf, dcs, dbs, dx = dev(Wf), dev(cs), dev(bs), to_dev(x, BF16)
    fused = empty((M, H * D), BF16)
    pkg.call("vla_layernorm_qkv_self_attention", dx, dWf, dcs, dbs, BF16, M, K, S, H, D, scale, eps, fused)
    t_max = 64
    kc, vc = empty((B, H, t_max, D), BF16), empty((B, H, D, t_max), BF16)
    q, pair = empty((M, H * D), BF16), empty((M, H * D), BF16)
    pkg.call("vla_layernorm_attn_qkv_rope", dx, dWf, dcs, dbs, BF16, M, K, S, H, H, 1, 1, D, None, None, q, kc, vc, t_max, 0, eps)
    pkg.call("vla_attn_prefix_suffix", q, kc, vc, pair, BF16, B, S, H, H, D, t_max, S, scale, pkg.VLA_MASK_NONE, 0, 0, 0, None)
    sync()
    y = orc.round_bf16(orc.linear(orc.adaln(x, sc, sh, eps), W, b)).reshape(B, S, 3, H, D)
    want = np.empty((B, S, H, D), np.float32)
    for bb in range(B):
        want[bb] = orc.attention(y[bb, :, 0], y[bb, :, 1], y[bb, :, 2], np.zeros((S, S), np.float32), scale).reshape(S, H, D)
    got, two = as_f32(fused, BF16).reshape(B, S, H, D), as_f32(pair, BF16).reshape(B, S, H, D)
    # Held to the oracle as the modulated-LayerNorm projection is (8e-3 of the largest value:
    # a Q, K or V element that rounds to the other bf16 neighbour moves an output by up to an
    # ulp of the largest V), and no further from it than the two-launch path; the two GPU paths
    # share the folded weights and differ by the order of their sums.
    e1, e2 = rel_err(got, want), rel_err(two, want)
    assert e1 < 8e-3 and e1 <= 1.25 * e2 + 1e-3, (e1, e2)
    assert rel_err(got, two) < 8e-3, rel_err(got, two)  # one bf16 ulp of the largest output
    assert np.mean(np.abs(got - want)) < 2e-3 * np.abs(want).max()
    # the attention is really over the observation's own tokens: uniform weights are far off
    assert rel_err(np.broadcast_to(y[:, :, 2].mean(1, keepdims=True), want.shape), want) > 5e-2
    # shapes the launch is not built for are refused, not served slowly
    assert pkg.lib().vla_layernorm_qkv_self_attention(dx.data_ptr(), dWf.data_ptr(), dcs.data_ptr(), None, BF16, M, K, S, H, 64, scale,
                                                      eps, fused.data_ptr(), None) == pkg.VLA_K_ERR_SHAPE


@pytest.mark.parametrize("B,S,H,K", [(64, 17, 32, 1536), (5, 17, 8, 1536), (40, 9, 8, 512)])
def test_row_sums_handed_from_the_output_projection_to_the_next_layernorm(B, S, H, K):
    """A block's output projection leaves (sum of squares, sum) of the rows it writes, per 64-column
    tile; the next block's projection launches (LayerNorm inside) add those up instead of summing the
    rows themselves.  The sums against numpy on the bf16 values written; both consumers with the
    handed-over sums against the same launches without them (another order of the same sums) and
    against the oracle."""
    D = 48
    r = np.random.default_rng(9100 + B + K)
    M, Kin = B * S, H * D
    att = orc.round_bf16(r.standard_normal((M, Kin)).astype(np.float32))
    Wo = orc.round_bf16((0.03 * r.standard_normal((K, Kin))).astype(np.float32))
    bo = (0.1 * r.standard_normal(K)).astype(np.float32)
    h0 = orc.round_bf16((2.0 * r.standard_normal((M, K)) + 1.5 * r.standard_normal((M, 1))).astype(np.float32))
    nt = K // 64
    h = to_dev(h0, BF16)
    stats = torch.zeros((M, nt, 2), dtype=torch.float32, device="cuda")
    pkg.call("vla_linear_row_stats", to_dev(att, BF16), to_dev(Wo, BF16), dev(bo), h, h, stats, BF16, M, K, Kin)
    h_ref = to_dev(h0, BF16)
    pkg.call("vla_linear", to_dev(att, BF16), to_dev(Wo, BF16), dev(bo), h_ref, h_ref, BF16, BF16, M, K, Kin)
    sync()
    hv = as_f32(h, BF16)
    assert np.array_equal(hv, as_f32(h_ref, BF16))  # the same projection
    st = host(stats)
    tiles = hv.reshape(M, nt, 64).astype(np.float64)
    assert np.allclose(st[:, :, 1], tiles.sum(-1), rtol=1e-5, atol=1e-4)
    assert np.allclose(st[:, :, 0], (tiles * tiles).sum(-1), rtol=1e-5, atol=1e-4)

    sc, sh = (0.3 * r.standard_normal(K)).astype(np.float32), (0.3 * r.standard_normal(K)).astype(np.float32)
    eps = 1e-5
    scale = 1.0 / np.sqrt(D)

    def folded(W, b):
        N = W.shape[0]
        Wf, cs, bs = np.empty((N, K), np.uint16), np.empty(N, np.float32), np.empty(N, np.float32)
        assert pkg.lib().vla_fold_adaln_weight_host(orc.to_bf16(W).ctypes.data, b.ctypes.data, sc.ctypes.data, sh.ctypes.data, N, K,
                                                    Wf.ctypes.data, cs.ctypes.data, bs.ctypes.data) == 0
        return dev(Wf), dev(cs), dev(bs)

    # cross block: Q projection
    Wq = orc.round_bf16((0.02 * r.standard_normal((H * D, K))).astype(np.float32))
    bq = (0.1 * r.standard_normal(H * D)).astype(np.float32)
    Wf, cs, bs = folded(Wq, bq)
    q1, q2 = empty((M, H * D), BF16), empty((M, H * D), BF16)
    pkg.call("vla_layernorm_attn_qkv_rope_stats", h, Wf, cs, bs, stats, nt, BF16, M, K, S, H, H, 0, 0, D, None, None, q1, None, None, 64, 0, eps)
    pkg.call("vla_layernorm_attn_qkv_rope", h, Wf, cs, bs, BF16, M, K, S, H, H, 0, 0, D, None, None, q2, None, None, 64, 0, eps)
    sync()
    want = orc.linear(orc.adaln(hv, sc, sh, eps), Wq, bq)
    g1, g2 = as_f32(q1, BF16), as_f32(q2, BF16)
    assert bf16_close(g1, want) and rel_err(g1, want) < 8e-3 and rel_err(g1, g2) < 8e-3
    # self block in one launch (its own shape limits: heads in eights, K >= 256)
    W3 = orc.round_bf16((0.02 * r.standard_normal((3 * H * D, K))).astype(np.float32))
    b3 = (0.1 * r.standard_normal(3 * H * D)).astype(np.float32)
    Wf, cs, bs = folded(W3, b3)
    o1, o2 = empty((M, H * D), BF16), empty((M, H * D), BF16)
    pkg.call("vla_layernorm_qkv_self_attention_stats", h, Wf, cs, bs, stats, nt, BF16, M, K, S, H, D, scale, eps, o1)
    pkg.call("vla_layernorm_qkv_self_attention", h, Wf, cs, bs, BF16, M, K, S, H, D, scale, eps, o2)
    sync()
    y = orc.round_bf16(orc.linear(orc.adaln(hv, sc, sh, eps), W3, b3))
    qkv = y.reshape(B, S, 3, H, D)
    want = np.stack([orc.attention(qkv[b, :, 0], qkv[b, :, 1], qkv[b, :, 2], np.zeros((S, S), np.float32), scale).reshape(S, H * D)
                     for b in range(B)]).reshape(M, H * D)
    g1, g2 = as_f32(o1, BF16), as_f32(o2, BF16)
    assert rel_err(g1, want) < 8e-3 and rel_err(g1, g2) < 8e-3  # one bf16 ulp
    # what the hand-over does not take
    assert pkg.lib().vla_linear_row_stats(h.data_ptr(), Wf.data_ptr(), None, None, h.data_ptr(), stats.data_ptr(), BF16, M, 72, K, None) == pkg.VLA_K_ERR_SHAPE
    assert pkg.lib().vla_layernorm_attn_qkv_rope_stats(h.data_ptr(), Wf.data_ptr(), cs.data_ptr(), None, stats.data_ptr(), nt + 1, BF16, M, K, S, H, H,
                                                       0, 0, D, None, None, q1.data_ptr(), None, None, 64, 0, eps, None) == pkg.VLA_K_ERR_SHAPE


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("M,I,K,act,bias", [(50, 2048, 720, "silu", False), (130, 96, 72, "gelu", True), (1600, 256, 720, "silu", False),
                                           (17, 6144, 1536, "gelu", True)])
def test_glu_linear_and_linear_act(dtype, M, I, K, act, bias):
    """Gate/up projection with the activation and the product in the epilogue, and the
    activation between bias and residual of vla_linear_act, against the oracle."""
    r = np.random.default_rng(1300 + M)
    x = r.standard_normal((M, K)).astype(np.float32)
    Wgu = (0.05 * r.standard_normal((2 * I, K))).astype(np.float32)
    b = (0.1 * r.standard_normal(2 * I)).astype(np.float32) if bias else None
    res = r.standard_normal((M, I)).astype(np.float32)
    if dtype == BF16:
        x, Wgu, res = orc.round_bf16(x), orc.round_bf16(Wgu), orc.round_bf16(res)
    fact = orc.silu if act == "silu" else orc.gelu
    code = pkg.VLA_ACT_SILU if act == "silu" else pkg.VLA_ACT_GELU
    y = empty((M, I), dtype)
    pkg.call("vla_glu_linear", to_dev(x, dtype), to_dev(Wgu, dtype), None if b is None else dev(b), y, dtype, dtype, M, I, K,
             code, -1.0)
    y2 = empty((M, I), dtype)
    pkg.call("vla_linear_act", to_dev(x, dtype), to_dev(Wgu[:I], dtype), None if b is None else dev(b[:I]),
             to_dev(res, dtype), y2, dtype, dtype, M, I, K, code)
    sync()
    gate = orc.linear(x, Wgu[:I], None if b is None else b[:I])
    want = fact(gate) * orc.linear(x, Wgu[I:], None if b is None else b[I:])
    want2 = fact(gate) + res
    if dtype == F32:
        assert rel_err(host(y), want) < FP32_TOL and rel_err(host(y2), want2) < FP32_TOL
    else:
        assert bf16_close(as_f32(y, dtype), want) and bf16_close(as_f32(y2, dtype), want2)
    if dtype == BF16 and K % 16 == 0:
        # the RMS pre-norm inside the launch (norm weight folded into both halves of the weights)
        g = orc.round_bf16((1.0 + 0.3 * r.standard_normal(K)).astype(np.float32))
        xs = orc.round_bf16(x * 3.0)
        Wf = np.empty((2 * I, K), np.uint16)
        assert pkg.lib().vla_fold_norm_weight_host(orc.to_bf16(Wgu).ctypes.data, orc.to_bf16(g).ctypes.data, BF16, 2 * I, K,
                                                   Wf.ctypes.data) == 0
        y3 = empty((M, I), BF16)
        pkg.call("vla_glu_linear", to_dev(xs, BF16), dev(Wf), None, y3, BF16, BF16, M, I, K, code, 1e-5)
        sync()
        # exactly what the launch computes (unrounded normalised rows, weights folded and rounded once) ...
        n0 = orc.rms_norm(xs, None, 1e-5)
        Wfold = orc.from_bf16(Wf)
        model = fact(orc.linear(n0, Wfold[:I])) * orc.linear(n0, Wfold[I:])
        assert bf16_close(as_f32(y3, BF16), model)
        # ... which stays within bf16 rounding of norm-then-project with the unfolded weights
        n = orc.rms_norm(xs, g, 1e-5)
        want3 = fact(orc.linear(n, Wgu[:I])) * orc.linear(n, Wgu[I:])
        assert rel_err(as_f32(y3, BF16), want3) < 1e-2


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,S,n_lead,A,W", [(3, 50, 0, 32, 720), (2, 51, 1, 32, 1024), (3, 17, 1, 32, 1536), (1, 9, 0, 7, 200),
                                            (2, 5, 1, 32, 2560)])
def test_final_norm_inside_the_euler_launch(dtype, B, S, n_lead, A, W):
    """x_t += dt (W_out . norm(h) + b_out) in one launch, for the three final norms of the flow
    heads (RMSNorm with a weight, LayerNorm without affine then scale / shift, RMS statistics then
    scale / shift): against the oracle, and against the norm launch followed by the plain update."""
    r = np.random.default_rng(170 + W)
    h = (r.standard_normal((B, S, W)) * 2 + 0.3).astype(np.float32)
    g = (1 + 0.1 * r.standard_normal(W)).astype(np.float32)
    sc, sh = (0.2 * r.standard_normal(W)).astype(np.float32), (0.2 * r.standard_normal(W)).astype(np.float32)
    x_t = r.standard_normal((B, S - n_lead, A)).astype(np.float32)
    W_out = (0.05 * r.standard_normal((A, W))).astype(np.float32)
    b_out = r.standard_normal(A).astype(np.float32)
    if dtype == BF16:
        h, g = orc.round_bf16(h), orc.round_bf16(g)
    dt = -0.25
    M = B * S
    dh, dW, db = to_dev(h, dtype), dev(W_out), dev(b_out)
    rnd = orc.round_bf16 if dtype == BF16 else (lambda v: v)
    cases = {
        "rms": (lambda xd: pkg.call("vla_rmsnorm_euler_step", xd, dh, to_dev(g, dtype), 1e-6, dW, db, dtype, B, S, n_lead, A, W, dt),
                lambda y: pkg.call("vla_rms_norm", dh, to_dev(g, dtype), y, dtype, M, W, 1e-6),
                orc.rms_norm(h.reshape(M, W), g, 1e-6)),
        "adaln": (lambda xd: pkg.call("vla_adanorm_euler_step", xd, dh, dev(sc), dev(sh), 1, 1e-5, dW, db, dtype, B, S, n_lead, A, W, dt),
                  lambda y: pkg.call("vla_adaln", dh, dev(sc), dev(sh), y, dtype, M, W, 1e-5),
                  orc.adaln(h.reshape(M, W), sc, sh, 1e-5)),
        "adarms": (lambda xd: pkg.call("vla_adanorm_euler_step", xd, dh, dev(sc), dev(sh), 0, 1e-6, dW, db, dtype, B, S, n_lead, A, W, dt),
                   lambda y: pkg.call("vla_adarms", dh, dev(sc), dev(sh), y, dtype, M, W, 1e-6),
                   orc.adarms(h.reshape(M, W), sc, sh, 1e-6)),
    }
    for name, (fused, norm, hn_want) in cases.items():
        xd = dev(x_t)
        fused(xd)
        y = empty((M, W), dtype)
        norm(y)
        xd2 = dev(x_t)
        pkg.call("vla_euler_step", xd2, y, dW, db, dtype, B, S, n_lead, A, W, dt)
        sync()
        hn = rnd(hn_want).reshape(B, S, W)[:, n_lead:]
        v = orc.linear(hn.reshape(-1, W), W_out, b_out).reshape(B, S - n_lead, A)
        want = x_t + dt * v
        got, chain = host(xd), host(xd2)
        # the row statistics are summed in another order than the stand-alone norm's: with bf16 rows a
        # last-place difference of the scale can move single elements to the neighbouring bf16 value
        tol = FP32_TOL if dtype == F32 else 2e-3
        assert rel_err(got, want) < tol, (name, rel_err(got, want))
        assert rel_err(got, chain) < tol, (name, rel_err(got, chain))


# ------------------------------------------------------------------ attention
CASES = [
    # name, B, S, Hq, Hkv, D, P, mask kind, pad
    ("smolvla-causal", 2, 50, 15, 5, 64, 241, "causal", (230, 240)),
    ("smolvla-bidir", 1, 50, 15, 5, 64, 241, "none", (0, 0)),
    ("smolvla-cross", 2, 50, 15, 5, 64, 241, "cross", (200, 240)),
    ("pi0", 2, 51, 8, 1, 256, 816, "pi0", (0, 0)),
    ("gr00t-cross", 3, 17, 32, 32, 48, 296, "cross", (0, 0)),
    ("gr00t-self", 3, 17, 32, 32, 48, 0, "none", (0, 0)),
    ("bitvla-decode", 2, 1, 20, 5, 128, 515, "cross", (0, 0)),
    ("bitvla-prefill", 1, 130, 20, 5, 128, 0, "none", (0, 0)),
    # at most 32 query rows per kv head: the register-direct kernel, with every mask kind
    ("short-causal", 2, 10, 6, 2, 64, 100, "causal", (90, 97)),
    ("short-pi0", 1, 4, 8, 1, 128, 75, "pi0", (0, 0)),
    ("short-ragged", 5, 3, 4, 4, 48, 37, "cross", (30, 33)),
]


def _mask(kind, P, S, pad):
    if kind == "causal":
        return orc.mask_smolvla_full(P, S, pad[0], pad[1]), pkg.VLA_MASK_CAUSAL_SUFFIX, P + S
    if kind == "pi0":
        return orc.mask_pi0_full(P, S), pkg.VLA_MASK_PI0_STATE, P + S
    if kind == "cross":
        return orc.mask_smolvla_prefix_only(P, S, pad[0], pad[1]), pkg.VLA_MASK_NONE, P
    m = np.zeros((S, P + S), np.float32)
    m[:, pad[0]:pad[1]] = -np.inf
    return m, pkg.VLA_MASK_NONE, P + S


@pytest.mark.parametrize("B,S,H,T", [(64, 17, 32, 296), (33, 17, 32, 296), (40, 5, 32, 130), (64, 17, 32, 320)])
def test_streaming_cross_attention_matches_oracle_and_direct_kernel(tune, B, S, H, T):
    # GR00T's cross blocks at batch: 48-wide heads, at most 32 query rows per head, at least 1024
    # (batch, head) pairs -- the streaming form (K / V^T through a per-wavefront LDS ring, a
    # wavefront walking several pairs).  Against the oracle on a sample of observations, and bit
    # for bit against the register-direct kernel on all of them.  Pair counts that are not a
    # multiple of the wavefront count, key counts that end inside a 64-key stretch and one that
    # fills the cache rows exactly; stale cache contents past n_keys are poisoned.
    D = 48
    r = np.random.default_rng(B * 1000 + T)
    t_max = (T + 63) // 64 * 64
    Q = orc.round_bf16(r.standard_normal((B, S, H, D)).astype(np.float32))
    K = orc.round_bf16(r.standard_normal((B, T, H, D)).astype(np.float32))
    V = orc.round_bf16(r.standard_normal((B, T, H, D)).astype(np.float32))
    kc = torch.full((B, H, t_max, D), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    vc = torch.full((B, H, D, t_max), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, BF16), to_dev(V, BF16), BF16, B, H, D, t_max, 0, T)
    scale = 1.0 / math.sqrt(D)
    outs = {}
    for name in ("stream", "direct"):
        if name == "direct":
            tune.set("VLA_ATTN_NO_STREAM", "1")
            tune.set("VLA_ATTN_SPLIT", "0")  # one key slice, as the streaming form walks the keys (fewer than 2048 pairs would be sliced)
        out = empty((B, S, H * D), BF16)
        pkg.call("vla_attn_prefix_suffix", to_dev(Q, BF16), kc, vc, out, BF16, B, S, H, H, D, t_max, T, scale, pkg.VLA_MASK_NONE, T,
                 0, 0, None)
        sync()
        outs[name] = host(out)
    assert np.array_equal(outs["stream"], outs["direct"])
    got = orc.from_bf16(outs["stream"].view(np.uint16))
    mask = np.zeros((S, T), np.float32)
    for b in (0, B // 2, B - 1):
        want = orc.attention(Q[b], K[b], V[b], mask, scale)
        assert np.isfinite(got[b]).all()
        assert bf16_close(got[b], want) and rel_err(got[b], want) < 1e-2


@pytest.mark.parametrize("dtype,kernel", [(F32, "auto"), (BF16, "auto"), (BF16, "direct"), (BF16, "staged"), (BF16, "one-slice")],
                         ids=["f32", "bf16", "bf16-direct", "bf16-staged", "bf16-one-slice"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_attention_against_oracle(tune, dtype, kernel, case):
    name, B, S, Hq, Hkv, D, P, kind, pad = case
    if kernel == "direct":
        # the register-direct kernel is the default up to 32 query rows per kv head; beyond
        # that it walks 32-row blocks, exercised here on the cases that normally take the LDS kernel
        if not (D <= 128 and 32 < (Hq // Hkv) * S <= 256):
            pytest.skip("covered by the default dispatch")
        tune.set("VLA_ATTN_DIRECT_ROWS", "256")
    if kernel in ("staged", "one-slice"):
        # 64-wide bf16 heads beyond 32 rows default to the direct-to-LDS variant of the LDS
        # kernel (two key slices per row tile with 3+ key tiles); the
        # register-staged variant and the unsliced one on the same cases
        if not (D == 64 and (Hq // Hkv) * S > 32):
            pytest.skip("covered by the default dispatch")
        tune.set("VLA_ATTN_DL" if kernel == "staged" else "VLA_ATTN_SLICES", "0" if kernel == "staged" else "1")
    r = np.random.default_rng(106)
    mask, mkind, T = _mask(kind, P, S, pad)
    t_max = (T + 63) // 64 * 64
    Q = r.standard_normal((B, S, Hq, D)).astype(np.float32)
    K = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    if dtype == BF16:
        Q, K, V = orc.round_bf16(Q), orc.round_bf16(K), orc.round_bf16(V)
    # stale cache contents past n_keys must not matter: poison them
    kc = torch.full((B, Hkv, t_max, D), float("nan"), device="cuda")
    vc = torch.full((B, Hkv, D, t_max), float("nan"), device="cuda")
    if dtype == BF16:
        kc, vc = kc.to(torch.bfloat16).view(torch.int16), vc.to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, dtype), to_dev(V, dtype), dtype, B, Hkv, D, t_max, 0, T)
    scale = 1.0 / math.sqrt(D)
    out = empty((B, S, Hq * D), dtype)
    pkg.call("vla_attn_prefix_suffix", to_dev(Q, dtype), kc, vc, out, dtype, B, S, Hq, Hkv, D, t_max, T, scale, mkind, P,
             pad[0], pad[1], None)
    out_m = empty((B, S, Hq * D), dtype)
    pkg.call("vla_attn_prefix_suffix", to_dev(Q, dtype), kc, vc, out_m, dtype, B, S, Hq, Hkv, D, t_max, T, scale,
             pkg.VLA_MASK_NONE, 0, 0, 0, dev(mask))
    sync()
    want = np.stack([orc.attention(Q[b], K[b], V[b], mask, scale) for b in range(B)])
    got, got_m = as_f32(out, dtype), as_f32(out_m, dtype)
    assert np.isfinite(got).all()
    if dtype == F32:
        assert rel_err(got, want) < FP32_TOL, rel_err(got, want)
        assert rel_err(got_m, want) < FP32_TOL
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
    else:
        assert bf16_close(got, want) and bf16_close(got_m, want)
        assert rel_err(got, want) < 1e-2
        # split-precision probabilities: same storage, P.V product within output rounding
        out_p2 = empty((B, S, Hq * D), dtype)
        pkg.call("vla_attn_prefix_suffix", to_dev(Q, dtype), kc, vc, out_p2, pkg.VLA_DT_BF16_P2, B, S, Hq, Hkv, D, t_max, T,
                 scale, mkind, P, pad[0], pad[1], None)
        sync()
        got_p2 = as_f32(out_p2, dtype)
        assert bf16_close(got_p2, want) and rel_err(got_p2, want) < 4e-3
        assert rel_err(got_p2, want) <= rel_err(got, want) * 1.05
    # generated mask and mask-as-data run the same arithmetic
    assert np.array_equal(host(out), host(out_m))


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_attention_cache_rows_of_any_multiple_of_8(dtype, case):
    """The cache row length only has to be a multiple of 8 keys: with the tightest t_max the last
    32-key block reaches past the end of every V^T row, and what a kernel reads for those keys
    must stay inside the allocation and out of the result."""
    name, B, S, Hq, Hkv, D, P, kind, pad = case
    r = np.random.default_rng(107)
    mask, mkind, T = _mask(kind, P, S, pad)
    t_max = (T + 7) // 8 * 8
    Q = r.standard_normal((B, S, Hq, D)).astype(np.float32)
    K = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    if dtype == BF16:
        Q, K, V = orc.round_bf16(Q), orc.round_bf16(K), orc.round_bf16(V)
    kc = torch.full((B, Hkv, t_max, D), float("nan"), device="cuda")
    vc = torch.full((B, Hkv, D, t_max), float("nan"), device="cuda")
    if dtype == BF16:
        kc, vc = kc.to(torch.bfloat16).view(torch.int16), vc.to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, dtype), to_dev(V, dtype), dtype, B, Hkv, D, t_max, 0, T)
    scale = 1.0 / math.sqrt(D)
    out = empty((B, S, Hq * D), dtype)
    pkg.call("vla_attn_prefix_suffix", to_dev(Q, dtype), kc, vc, out, dtype, B, S, Hq, Hkv, D, t_max, T, scale, mkind, P,
             pad[0], pad[1], None)
    sync()
    want = np.stack([orc.attention(Q[b], K[b], V[b], mask, scale) for b in range(B)])
    got = as_f32(out, dtype)
    assert np.isfinite(got).all()
    if dtype == F32:
        assert rel_err(got, want) < FP32_TOL, rel_err(got, want)
    else:
        assert bf16_close(got, want) and rel_err(got, want) < 1e-2


@pytest.mark.parametrize("split", [1, 2, 5, 8, 64])
def test_attention_direct_kernel_key_slices_merge(tune, split):
    # Few query rows: any slicing of the keys across wavefronts (merged by the second
    # kernel) gives the same result as the oracle.
    r = np.random.default_rng(120 + split)
    B, S, Hq, Hkv, D, T = 2, 5, 6, 2, 64, 333
    t_max = 336
    Q = orc.round_bf16(r.standard_normal((B, S, Hq, D)).astype(np.float32))
    K = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    V = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    kc = torch.full((B, Hkv, t_max, D), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    vc = torch.full((B, Hkv, D, t_max), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, BF16), to_dev(V, BF16), BF16, B, Hkv, D, t_max, 0, T)
    tune.set("VLA_ATTN_SPLIT", str(split))
    out = empty((B, S, Hq * D), BF16)
    pkg.call("vla_attn_prefix_suffix", to_dev(Q, BF16), kc, vc, out, BF16, B, S, Hq, Hkv, D, t_max, T, 0.125,
             pkg.VLA_MASK_CAUSAL_SUFFIX, T - S, 100, 120, None)
    sync()
    mask = orc.mask_smolvla_full(T - S, S, 100, 120)
    want = np.stack([orc.attention(Q[b], K[b], V[b], mask, 0.125) for b in range(B)])
    got = as_f32(out, BF16)
    assert np.isfinite(got).all() and bf16_close(got, want) and rel_err(got, want) < 1e-2


@pytest.mark.parametrize("split", [12, 16, 19])
def test_attention_merge_launch_with_many_key_slices(tune, split):
    # The merge launch is specialised for up to 16 slices (every load of a row requested at once) and loops over
    # the slices beyond that: both forms against the oracle, on a key range long enough for 19 slices of two blocks.
    r = np.random.default_rng(140 + split)
    B, S, Hq, Hkv, D, T = 1, 3, 4, 2, 64, 1200
    t_max = 1216
    Q = orc.round_bf16(r.standard_normal((B, S, Hq, D)).astype(np.float32))
    K = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    V = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    kc = torch.full((B, Hkv, t_max, D), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    vc = torch.full((B, Hkv, D, t_max), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, BF16), to_dev(V, BF16), BF16, B, Hkv, D, t_max, 0, T)
    tune.set("VLA_ATTN_SPLIT", str(split))
    out = empty((B, S, Hq * D), BF16)
    pkg.call("vla_attn_prefix_suffix", to_dev(Q, BF16), kc, vc, out, BF16, B, S, Hq, Hkv, D, t_max, T, 0.125,
             pkg.VLA_MASK_CAUSAL_SUFFIX, T - S, 100, 120, None)
    sync()
    mask = orc.mask_smolvla_full(T - S, S, 100, 120)
    want = np.stack([orc.attention(Q[b], K[b], V[b], mask, 0.125) for b in range(B)])
    got = as_f32(out, BF16)
    assert np.isfinite(got).all() and bf16_close(got, want) and rel_err(got, want) < 1e-2


@pytest.mark.parametrize("B,S,Hq,Hkv,T", [(8, 1, 20, 5, 519), (1, 1, 20, 5, 513), (3, 2, 8, 2, 519), (1, 1, 28, 4, 1000), (3, 2, 8, 2, 300), (2, 1, 4, 4, 97),
                                          (8, 1, 20, 5, 33)])
def test_attention_decode_slices_merged_by_the_last_to_arrive(tune, B, S, Hq, Hkv, T):
    # 128-wide heads, a few rows per kv head (single-token decode): the keys are sliced over
    # single-wavefront workgroups and the slice that arrives last merges them inside the launch.
    # Same tolerance against the oracle as the one-workgroup form, repeatable bit for bit
    # (the counters return to zero), and close to that form.
    D, t_max = 128, (T + 15) // 16 * 16 + 16
    r = np.random.default_rng(1000 * B + T)
    Q = orc.round_bf16(r.standard_normal((B, S, Hq, D)).astype(np.float32))
    K = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    V = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    kc = torch.full((B, Hkv, t_max, D), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    vc = torch.full((B, Hkv, D, t_max), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, BF16), to_dev(V, BF16), BF16, B, Hkv, D, t_max, 0, T)
    scale = 1.0 / np.sqrt(D)

    def run():
        out = empty((B, S, Hq * D), BF16)
        pkg.call("vla_attn_prefix_suffix", to_dev(Q, BF16), kc, vc, out, pkg.VLA_DT_BF16_P2, B, S, Hq, Hkv, D, t_max, T, scale,
                 pkg.VLA_MASK_NONE, T, 0, 0, None)
        sync()
        return as_f32(out, BF16)

    got = [run() for _ in range(3)]
    tune.set("VLA_ATTN_NO_ARRIVE", "1")
    ref = run()
    mask = np.zeros((S, T), np.float32)
    want = np.stack([orc.attention(Q[b], K[b], V[b], mask, scale) for b in range(B)]).reshape(B, S, Hq * D)
    assert np.isfinite(got[0]).all() and np.array_equal(got[0], got[1]) and np.array_equal(got[0], got[2])
    assert bf16_close(got[0], want) and rel_err(got[0], want) < 1e-2
    assert bf16_close(ref, want) and rel_err(got[0], ref) < 1e-2


@pytest.mark.parametrize("B", [1, 4])
def test_attention_wide_heads_key_slices_and_partial_formats(tune, B):
    # pi0's 256-wide MQA heads: with few workgroups the keys are walked in slices whose partial
    # outputs travel as fp16 (normalised per slice) to a merge launch.  Unsliced, fp32 partials
    # and fp16 partials all meet the oracle; the fp16 partials cost less than the output rounding.
    r = np.random.default_rng(130 + B)
    S, Hq, Hkv, D, P = 51, 8, 1, 256, 816
    T, t_max = P + S, 896
    Q = orc.round_bf16(r.standard_normal((B, S, Hq, D)).astype(np.float32))
    K = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    V = orc.round_bf16(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    kc = torch.full((B, Hkv, t_max, D), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    vc = torch.full((B, Hkv, D, t_max), float("nan"), device="cuda").to(torch.bfloat16).view(torch.int16)
    pkg.call("vla_kv_append", kc, vc, to_dev(K, BF16), to_dev(V, BF16), BF16, B, Hkv, D, t_max, 0, T)
    mask = orc.mask_pi0_full(P, S)
    want = np.stack([orc.attention(Q[b], K[b], V[b], mask, 1.0 / 16) for b in range(B)])
    got = {}
    for name, env in (("sliced-fp16", {}), ("sliced-fp32", {"VLA_ATTN_PART_F32": "1"}), ("unsliced", {"VLA_ATTN_SPLIT": "1"})):
        for k in ("VLA_ATTN_PART_F32", "VLA_ATTN_SPLIT"):
            tune.clear(k)
        for k, v in env.items():
            tune.set(k, v)
        out = empty((B, S, Hq * D), BF16)
        pkg.call("vla_attn_prefix_suffix", to_dev(Q, BF16), kc, vc, out, BF16, B, S, Hq, Hkv, D, t_max, T, 1.0 / 16,
                 pkg.VLA_MASK_PI0_STATE, P, 0, 0, None)
        sync()
        got[name] = as_f32(out, BF16)
        assert np.isfinite(got[name]).all() and bf16_close(got[name], want) and rel_err(got[name], want) < 1e-2, name
    assert rel_err(got["sliced-fp16"], want) <= rel_err(got["unsliced"], want) * 1.25 + 1e-4
    assert rel_err(got["sliced-fp16"], got["sliced-fp32"]) < 1e-2


def test_attention_special_cases_fp32():
    # all-zero Q -> mean of the visible V rows; permuting keys changes nothing
    r = np.random.default_rng(107)
    B, S, Hq, Hkv, D, T = 1, 5, 6, 2, 64, 100
    t_max = 128
    K = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    kc, vc = empty((B, Hkv, t_max, D), F32), empty((B, Hkv, D, t_max), F32)
    pkg.call("vla_kv_append", kc, vc, dev(K), dev(V), F32, B, Hkv, D, t_max, 0, T)
    out = empty((B, S, Hq * D), F32)
    pkg.call("vla_attn_prefix_suffix", dev(np.zeros((B, S, Hq, D), np.float32)), kc, vc, out, F32, B, S, Hq, Hkv, D,
             t_max, T, 0.125, pkg.VLA_MASK_NONE, T, 10, 30, None)
    sync()
    keep = [t for t in range(T) if not 10 <= t < 30]
    got = host(out).reshape(S, Hq, D)
    for h in range(Hq):
        assert np.allclose(got[2, h], V[0, keep, h // 3].mean(0), atol=1e-6)
    Q = r.standard_normal((B, S, Hq, D)).astype(np.float32)
    perm = r.permutation(T)
    outs = []
    for Kx, Vx in ((K, V), (K[:, perm], V[:, perm])):
        pkg.call("vla_kv_append", kc, vc, dev(Kx), dev(Vx), F32, B, Hkv, D, t_max, 0, T)
        o = empty((B, S, Hq * D), F32)
        pkg.call("vla_attn_prefix_suffix", dev(Q), kc, vc, o, F32, B, S, Hq, Hkv, D, t_max, T, 0.125,
                 pkg.VLA_MASK_NONE, T, 0, 0, None)
        sync()
        outs.append(host(o))
    assert rel_err(outs[1], outs[0]) < FP32_TOL


# -------------------------------------------------------------------- ternary
def test_act_quant_bit_exact():
    r = np.random.default_rng(108)
    M, K = 67, 2560
    x = orc.round_bf16((r.standard_normal((M, K)) * 3).astype(np.float32))
    x[3] = 0.0  # amax floor
    x[4, :8] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -127.0, 3.5]
    x[4, 8:] = 0.0  # scale exactly 1: ties go to even
    x = orc.round_bf16(x)
    q = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    rs = torch.zeros(M, dtype=torch.int32, device="cuda")
    pkg.call("vla_act_quant_bf16", dev(orc.to_bf16(x)), q, s, rs, M, K)
    q2 = torch.zeros_like(q)
    s2 = torch.zeros_like(s)
    pkg.call("bitvla_act_quant", dev(orc.to_bf16(x)), q2, s2, M, K)
    sync()
    wq, ws = orc.act_quant(x)
    assert np.array_equal(host(q), wq) and np.array_equal(host(s), ws)
    assert np.array_equal(host(rs), wq.astype(np.int32).sum(1))
    assert np.array_equal(host(q2), wq) and np.array_equal(host(s2), ws)
    assert list(wq[4, :8]) == [127, 0, 2, 2, 0, -2, -127, 4]


def _pack_plain(t):
    N, K = t.shape
    out = np.empty(pkg.lib().vla_ternary_packed_words(N, K), np.uint32)
    assert pkg.lib().vla_ternary_pack_host(t.ctypes.data, N, K, out.ctypes.data) == 0
    return out


@pytest.mark.parametrize("M,N,K,ws_num", [(600, 3840, 2560, 3), (517, 640, 2560, 1), (1, 2560, 2560, 1), (8, 3840, 2560, 6),
                                          (256, 1152, 1152 + 128, 1)])
def test_ternary_gemm_accumulators_and_epilogue_bit_exact(M, N, K, ws_num):
    # Inputs drawn the way the reference's GEMM check draws them
    # (tests/bitvla_gemm_check.cu:81-88): mt19937(1234 + N + M), A in [-127,127],
    # raw weight bytes (code 0 -> -2 included), s = 40 + rng%100, ws = 0.01 + 0.001*(rng%50).
    raw = mt19937_raw(1234 + N + M, M * K + N * K // 4 + M + ws_num)
    A = ((raw[:M * K] % 255).astype(np.int32) - 127).astype(np.int8).reshape(M, K)
    ladder = (raw[M * K:M * K + N * K // 4] % 256).astype(np.uint8)
    s = (40.0 + (raw[M * K + N * K // 4:M * K + N * K // 4 + M] % 100)).astype(np.float32)
    ws = (0.01 + 0.001 * (raw[-ws_num:] % 50).astype(np.float32)).astype(np.float32)
    Wt = orc.unpack_ladder_int2(ladder, N, K)
    packed = np.empty(pkg.lib().vla_ternary_packed_words(N, K), np.uint32)
    assert pkg.lib().vla_ternary_repack_ladder_host(ladder.ctypes.data, N, K, packed.ctypes.data) == 0
    acc = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    rowsum = dev(A.astype(np.int32).sum(1).astype(np.int32))
    pkg.call("vla_ternary_gemm", dev(A), dev(packed), out, acc, dev(s), rowsum, dev(ws), ws_num, M, N, K)
    sync()
    want_acc = orc.ternary_gemm_i32(A, Wt)
    assert np.array_equal(host(acc), want_acc)
    assert np.array_equal(host(out, np.uint16), orc.ternary_epilogue(want_acc, s, ws))
    if (N, K, ws_num) in ((3840, 2560, 3), (640, 2560, 1), (2560, 2560, 1)):
        out2 = torch.zeros_like(out)
        pkg.call("bitlinear_int8xint2_m", dev(A), dev(packed), out2, dev(s), dev(ws), M, N, K)
        sync()
        assert np.array_equal(host(out2), host(out))


@pytest.mark.parametrize("tile", [128, 256, 16])
@pytest.mark.parametrize("M,N,K", [(300, 288, 256), (515, 640, 384), (64, 48, 128)])
def test_ternary_gemm_large_tile_kernels_bit_exact(tune, tile, M, N, K):
    # The large-M kernels (weights read straight from the fragment-major layout), pinned
    # by VLA_TERNARY_TILE (16 = the 16x16x64 kernel), on ragged M and N: same int32
    # accumulators and bf16 epilogue.
    r = np.random.default_rng(tile + M)
    A = r.integers(-127, 128, (M, K)).astype(np.int8)
    ladder = r.integers(0, 256, N * K // 4).astype(np.uint8)
    s = (40.0 + r.integers(0, 100, M)).astype(np.float32)
    s[::7] = (127.0 / np.abs(r.standard_normal(s[::7].size) * 3 + 1e-3)).astype(np.float32)  # arbitrary mantissas
    if M > 400:  # scales near the exponent limits take the full-range division path
        s[5], s[100], s[300] = 1e-25, 3e22, 7.5e-21
    ws_num = 3 if N % 3 == 0 else 1
    ws = (0.01 + 0.001 * r.integers(0, 50, ws_num)).astype(np.float32)
    Wt = orc.unpack_ladder_int2(ladder, N, K)
    packed = np.empty(pkg.lib().vla_ternary_packed_words(N, K), np.uint32)
    assert pkg.lib().vla_ternary_repack_ladder_host(ladder.ctypes.data, N, K, packed.ctypes.data) == 0
    acc = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    rowsum = dev(A.astype(np.int32).sum(1).astype(np.int32))
    tune.set("VLA_TERNARY_TILE", str(tile))
    pkg.call("vla_ternary_gemm", dev(A), dev(packed), out, acc, dev(s), rowsum, dev(ws), ws_num, M, N, K)
    sync()
    want_acc = orc.ternary_gemm_i32(A, Wt)
    assert np.array_equal(host(acc), want_acc)
    assert np.array_equal(host(out, np.uint16), orc.ternary_epilogue(want_acc, s, ws))


def test_ternary_gemm_prefill_shape_all_tilings_agree(tune):
    # BitVLA prefill QKV at full size (M = 8 x 512 tokens): the shape-selected kernel and
    # both pinned tilings give identical accumulators and outputs; a sample of rows is
    # checked against the oracle.
    M, N, K, ws_num = 4096, 3840, 2560, 6
    r = np.random.default_rng(4096)
    A = r.integers(-127, 128, (M, K)).astype(np.int8)
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    s = (40.0 + r.integers(0, 100, M)).astype(np.float32)
    ws = (0.01 + 0.001 * r.integers(0, 50, ws_num)).astype(np.float32)
    dA, dW, ds, dws = dev(A), dev(_pack_plain(t)), dev(s), dev(ws)
    rowsum = dev(A.astype(np.int32).sum(1).astype(np.int32))
    res = []
    for tile in (None, 64, 128, 256, 16):
        if tile is None:
            tune.clear("VLA_TERNARY_TILE")
        else:
            tune.set("VLA_TERNARY_TILE", str(tile))
        acc = torch.zeros((M, N), dtype=torch.int32, device="cuda")
        out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
        pkg.call("vla_ternary_gemm", dA, dW, out, acc, ds, rowsum, dws, ws_num, M, N, K)
        sync()
        res.append((acc, out))
    for acc, out in res[1:]:
        assert torch.equal(acc, res[0][0]) and torch.equal(out, res[0][1])
    rows = np.r_[0:8, 255:258, 2047:2050, 4088:4096]
    want_acc = orc.ternary_gemm_i32(A[rows], t)
    assert np.array_equal(host(res[0][0])[rows], want_acc)
    assert np.array_equal(host(res[0][1], np.uint16)[rows], orc.ternary_epilogue(want_acc, s[rows], ws))


@pytest.mark.parametrize("M,N,K,ws_num", [(1, 3840, 2560, 6), (8, 3840, 2560, 6), (32, 3840, 2560, 6),
                                          (5, 48, 128, 3), (3, 640, 6912, 1)])
def test_ternary_gemv_decode_rows_bit_exact(M, N, K, ws_num):
    # At most 32 rows (single-token decode): the split-K GEMV kernel gives the oracle's
    # accumulators and epilogue, and, with a residual, the bits of GEMM followed by add.
    # Ragged N (not a multiple of 32), a K of one 128-slice and the long-K variant included.
    r = np.random.default_rng(900 + M)
    A = r.integers(-127, 128, (M, K)).astype(np.int8)
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    s = (127.0 / np.abs(r.standard_normal(M) * 3 + 1e-3)).astype(np.float32)
    ws = (0.01 + 0.001 * r.integers(0, 50, ws_num)).astype(np.float32)
    res = orc.to_bf16(r.standard_normal((M, N)).astype(np.float32))
    dA, dW, ds, dws = dev(A), dev(_pack_plain(t)), dev(s), dev(ws)
    rowsum = dev(A.astype(np.int32).sum(1).astype(np.int32))
    acc = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    pkg.call("vla_ternary_gemm", dA, dW, out, acc, ds, rowsum, dws, ws_num, M, N, K)
    h = dev(res)
    pkg.call("vla_ternary_gemm_add", dA, dW, h, h, ds, rowsum, dws, ws_num, M, N, K)  # in place, as the engine calls it
    want_sum = torch.zeros_like(out)
    pkg.call("bitvla_add_bf16", out, dev(res), want_sum, M * N)
    sync()
    want_acc = orc.ternary_gemm_i32(A, t)
    assert np.array_equal(host(acc), want_acc)
    assert np.array_equal(host(out, np.uint16), orc.ternary_epilogue(want_acc, s, ws))
    assert np.array_equal(host(h), host(want_sum))


@pytest.mark.parametrize("M,N,K,tile", [(300, 288, 256, 64), (300, 288, 256, 128), (515, 640, 384, 256), (300, 288, 256, 16),
                                        (515, 640, 384, 16)])
def test_ternary_gemm_add_matches_gemm_then_add(tune, M, N, K, tile):
    r = np.random.default_rng(M + tile)
    A = r.integers(-127, 128, (M, K)).astype(np.int8)
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    s = (40.0 + r.integers(0, 100, M)).astype(np.float32)
    ws = np.float32([0.02])
    res = orc.to_bf16(r.standard_normal((M, N)).astype(np.float32))
    dA, dW, ds, dws = dev(A), dev(_pack_plain(t)), dev(s), dev(ws)
    rowsum = dev(A.astype(np.int32).sum(1).astype(np.int32))
    tune.set("VLA_TERNARY_TILE", str(tile))
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    pkg.call("vla_ternary_gemm", dA, dW, out, None, ds, rowsum, dws, 1, M, N, K)
    fused = torch.zeros_like(out)
    pkg.call("vla_ternary_gemm_add", dA, dW, fused, dev(res), ds, rowsum, dws, 1, M, N, K)
    want = torch.zeros_like(out)
    pkg.call("bitvla_add_bf16", out, dev(res), want, M * N)
    sync()
    assert np.array_equal(host(fused), host(want))


@pytest.mark.parametrize("M,K", [(8, 2560), (37, 720), (4, 4096), (300, 2560), (129, 720), (70, 4096), (9, 6912), (3, 16384)])
def test_rmsnorm_act_quant_fused_is_the_pair(M, K):
    r = np.random.default_rng(K + M)
    x = orc.to_bf16((r.standard_normal((M, K)) * 3).astype(np.float32))
    w = orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32))
    hn = torch.zeros((M, K), dtype=torch.int16, device="cuda")
    q1, s1, r1 = (torch.zeros((M, K), dtype=torch.int8, device="cuda"), torch.zeros(M, device="cuda"),
                  torch.zeros(M, dtype=torch.int32, device="cuda"))
    q2, s2, r2 = torch.zeros_like(q1), torch.zeros_like(s1), torch.zeros_like(r1)
    pkg.call("bitvla_rmsnorm_bf16", dev(x), dev(w), hn, 1e-5, M, K)
    pkg.call("vla_act_quant_bf16", hn, q1, s1, r1, M, K)
    pkg.call("vla_rmsnorm_act_quant_bf16", dev(x), dev(w), q2, s2, r2, 1e-5, M, K)
    sync()
    if K <= 4096:  # longer rows: the two paths sum the squares in different orders, so only the oracle check below applies
        assert torch.equal(q1, q2) and torch.equal(s1, s2) and torch.equal(r1, r2)
    assert np.array_equal(host(r2), host(q2).astype(np.int32).sum(1))
    # and the pair follows the oracle
    n = orc.round_bf16(orc.rms_norm(orc.from_bf16(x), orc.from_bf16(w), 1e-5))
    qo, so = orc.act_quant(n)
    assert np.mean(host(q2) != qo) < 2e-3 and np.allclose(host(s2), so, rtol=1e-2)
    assert pkg.lib().vla_rmsnorm_act_quant_bf16(0, 0, 0, 0, 0, ctypes.c_float(1e-5), 1, 8, 0) == pkg.VLA_K_ERR_ARG
    # a norm weight that is not 16-byte aligned takes element loads: same bits
    wpad = torch.zeros(K + 8, dtype=torch.int16, device="cuda")
    wpad[1:K + 1] = dev(w)
    q3, s3, r3 = torch.zeros_like(q1), torch.zeros_like(s1), torch.zeros_like(r1)
    pkg.call("vla_rmsnorm_act_quant_bf16", dev(x), wpad[1:K + 1], q3, s3, r3, 1e-5, M, K)
    sync()
    assert torch.equal(q3, q2) and torch.equal(s3, s2) and torch.equal(r3, r2)


@pytest.mark.parametrize("M,N,K,ws_num", [(1, 3840, 2560, 3), (8, 3840, 2560, 3), (8, 2560, 2560, 1), (3, 48, 128, 3),
                                          (5, 640, 4096, 1), (7, 100, 1024, 1)])
def test_rmsnorm_ternary_gemv_one_launch_is_the_chain(M, N, K, ws_num):
    # Decode rows: norm + quantisation inside the GEMV launch gives the bits of
    # vla_rmsnorm_act_quant_bf16 -> vla_ternary_gemm_add, with and without the residual
    # (written in place, as the engine's O projection does).  Two calls in a row on
    # different rows: nothing of the first survives in the second.
    r = np.random.default_rng(77 * M + K)
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    ws = (0.01 + 0.001 * r.integers(0, 50, ws_num)).astype(np.float32)
    w = orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32))
    dW, dws, dw = dev(_pack_plain(t)), dev(ws), dev(w)
    for rep in range(2):
        x = orc.to_bf16((r.standard_normal((M, K)) * (3 if rep == 0 else 0.2)).astype(np.float32))
        res = orc.to_bf16(r.standard_normal((M, N)).astype(np.float32))
        q, sc, rs = (torch.zeros((M, K), dtype=torch.int8, device="cuda"), torch.zeros(M, device="cuda"),
                     torch.zeros(M, dtype=torch.int32, device="cuda"))
        pkg.call("vla_rmsnorm_act_quant_bf16", dev(x), dw, q, sc, rs, 1e-5, M, K)
        want, want_res = torch.zeros((M, N), dtype=torch.int16, device="cuda"), dev(res)
        pkg.call("vla_ternary_gemm", q, dW, want, None, sc, rs, dws, ws_num, M, N, K)
        pkg.call("vla_ternary_gemm_add", q, dW, want_res, want_res, sc, rs, dws, ws_num, M, N, K)
        got, got_res = torch.zeros_like(want), dev(res)
        pkg.call("vla_rmsnorm_ternary_gemv", dev(x), dw, 1e-5, dW, got, None, dws, ws_num, M, N, K)
        pkg.call("vla_rmsnorm_ternary_gemv", dev(x), dw, 1e-5, dW, got_res, got_res, dws, ws_num, M, N, K)
        sync()
        assert torch.equal(got, want) and torch.equal(got_res, want_res)
    # and the chain follows the oracle: norm -> bf16 -> quantise -> int32 GEMM -> epilogue
    n = orc.round_bf16(orc.rms_norm(orc.from_bf16(x), orc.from_bf16(w), 1e-5))
    qo, so = orc.act_quant(n)
    ref = orc.from_bf16(orc.ternary_epilogue(orc.ternary_gemm_i32(qo, t), so, ws))
    assert rel_err(orc.from_bf16(host(got, np.uint16)), ref) < 2e-2


@pytest.mark.parametrize("B,Hq,Hkv,D,K,ws_num", [(8, 20, 5, 128, 2560, 6), (1, 20, 5, 128, 2560, 6), (3, 4, 2, 64, 256, 2),
                                                 (5, 2, 2, 32, 128, 1)])
def test_rmsnorm_ternary_gemv_rope_append_one_launch_is_the_chain(B, Hq, Hkv, D, K, ws_num):
    # One appended token per batch row: norm + quantisation + QKV GEMV + split + RoPE + cache
    # append in one launch (paired weight rows) gives the bits of the three-launch chain, in Q
    # and in the written cache slot, and touches nothing else of the cache.
    r = np.random.default_rng(31 * B + D)
    N, t_max, pos = (Hq + 2 * Hkv) * D, 64, 37
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    ws = (0.01 + 0.001 * r.integers(0, 50, ws_num)).astype(np.float32)
    w = orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32))
    x = orc.to_bf16((r.standard_normal((B, K)) * 2).astype(np.float32))
    cos, sin = orc.rope_tables(np.int32([pos]), D, 10000.0)
    packed = _pack_plain(t)
    paired = np.empty_like(packed)
    assert pkg.lib().vla_ternary_pair_rope_rows_host(packed.ctypes.data, Hq, Hkv, D, K, paired.ctypes.data) == 0
    dws, dw, dx, dcos, dsin = dev(ws), dev(w), dev(x), dev(cos.astype(np.float32)), dev(sin.astype(np.float32))
    fill = r.integers(0, 65536, (2, B, Hkv, t_max * D)).astype(np.uint16)
    kc1, vc1, kc2, vc2 = dev(fill[0]), dev(fill[1]), dev(fill[0]), dev(fill[1])
    q1 = torch.zeros((B, Hq * D), dtype=torch.int16, device="cuda")
    q2 = torch.zeros_like(q1)
    qkv = torch.zeros((B, N), dtype=torch.int16, device="cuda")
    pkg.call("vla_rmsnorm_ternary_gemv", dx, dw, 1e-5, dev(packed), qkv, None, dws, ws_num, B, N, K)
    pkg.call("vla_qkv_split_rope_append", qkv, dcos, dsin, q1, kc1, vc1, pkg.VLA_DT_BF16, B, 1, Hq, Hkv, D, t_max, pos)
    pkg.call("vla_rmsnorm_ternary_gemv_rope_append", dx, dw, 1e-5, dev(paired), dws, ws_num, dcos, dsin, q2, kc2, vc2, B, Hq, Hkv,
             D, K, t_max, pos)
    sync()
    assert torch.equal(q1, q2) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    assert not np.array_equal(host(kc2, np.uint16), fill[0]) and not np.array_equal(host(vc2, np.uint16), fill[1])
    lib, f, p = pkg.lib(), ctypes.c_float(1e-5), qkv.data_ptr()
    bad = lambda *a: lib.vla_rmsnorm_ternary_gemv_rope_append(p, p, f, p, p, a[0], p, p, p, p, p, a[1], a[2], a[3], a[4], a[5], 64, a[6], 0)
    assert bad(1, 9, 2, 2, 32, 128, 0) == pkg.VLA_K_ERR_SHAPE      # rows
    assert bad(1, 4, 2, 2, 48, 128, 0) == pkg.VLA_K_ERR_SHAPE      # head width not whole 32-row blocks
    assert bad(4, 4, 2, 2, 32, 128, 0) == pkg.VLA_K_ERR_SHAPE      # scale group of 48 columns cuts a head
    assert bad(1, 4, 2, 2, 32, 128, 64) == pkg.VLA_K_ERR_SHAPE     # slot past the cache
    assert bad(1, 0, 2, 2, 32, 128, 0) == pkg.VLA_K_OK


@pytest.mark.parametrize("M,N,K", [(8, 2560, 6912), (1, 2560, 6912), (5, 96, 768), (3, 64, 4096)])
def test_sqrelu_rmsnorm_ternary_gemv_one_launch_is_the_chain(M, N, K):
    # The FFN's second half on decode rows: relu(gate)^2 * up -> sub-norm -> quantisation -> down
    # projection + residual in one launch against the three stand-alone launches; and the long
    # rows alone (no activation) through vla_rmsnorm_ternary_gemv.
    r = np.random.default_rng(13 * M + K)
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    ws = np.float32([0.017])
    w = orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32))
    gu = orc.to_bf16((r.standard_normal((M, 2 * K)) * 1.5).astype(np.float32))
    res = orc.to_bf16(r.standard_normal((M, N)).astype(np.float32))
    dW, dws, dw, dgu = dev(_pack_plain(t)), dev(ws), dev(w), dev(gu)
    act = torch.zeros((M, K), dtype=torch.int16, device="cuda")
    q, sc, rs = (torch.zeros((M, K), dtype=torch.int8, device="cuda"), torch.zeros(M, device="cuda"),
                 torch.zeros(M, dtype=torch.int32, device="cuda"))
    pkg.call("gate_up_fused_sqrelu_mul_bf16", dgu, act, M, K)
    pkg.call("vla_rmsnorm_act_quant_bf16", act, dw, q, sc, rs, 1e-5, M, K)
    want = dev(res)
    pkg.call("vla_ternary_gemm_add", q, dW, want, want, sc, rs, dws, 1, M, N, K)
    got, got2 = dev(res), dev(res)
    pkg.call("vla_sqrelu_rmsnorm_ternary_gemv", dgu, dw, 1e-5, dW, got, got, dws, 1, M, N, K)
    pkg.call("vla_rmsnorm_ternary_gemv", act, dw, 1e-5, dW, got2, got2, dws, 1, M, N, K)
    sync()
    assert torch.equal(got, got2)
    if K <= 4096:
        assert torch.equal(got, want)
    else:
        # rows longer than 4096: the stand-alone norm + quantisation shares a row among four
        # wavefronts and adds the squares in another order, so a scale can differ in its last
        # bit and a few int8 codes with it
        g, wv = as_f32(got, BF16), as_f32(want, BF16)
        assert np.mean(g != wv) < 0.05 and rel_err(g, wv) < 1e-2
    assert pkg.lib().vla_sqrelu_rmsnorm_ternary_gemv(dgu.data_ptr(), dw.data_ptr(), ctypes.c_float(1e-5), dW.data_ptr(),
                                                     got.data_ptr(), 0, dws.data_ptr(), 1, 9, N, K, 0) == pkg.VLA_K_ERR_SHAPE


@pytest.mark.parametrize("M,K", [(8, 6912), (300, 6912), (5, 768), (37, 4096), (2, 8192)])
def test_sqrelu_rmsnorm_act_quant_one_launch_is_the_pair(M, K):
    # relu(gate)^2 * up -> sub-norm -> quantisation in one launch (the activation never written)
    # against gate_up_fused_sqrelu_mul_bf16 followed by vla_rmsnorm_act_quant_bf16: same bits.
    r = np.random.default_rng(7 * M + K)
    gu = dev(orc.to_bf16((r.standard_normal((M, 2 * K)) * 1.5).astype(np.float32)))
    w = dev(orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32)))
    act = torch.zeros((M, K), dtype=torch.int16, device="cuda")
    q1, s1, r1 = (torch.zeros((M, K), dtype=torch.int8, device="cuda"), torch.zeros(M, device="cuda"),
                  torch.zeros(M, dtype=torch.int32, device="cuda"))
    q2, s2, r2 = torch.zeros_like(q1), torch.zeros_like(s1), torch.zeros_like(r1)
    pkg.call("gate_up_fused_sqrelu_mul_bf16", gu, act, M, K)
    pkg.call("vla_rmsnorm_act_quant_bf16", act, w, q1, s1, r1, 1e-5, M, K)
    pkg.call("vla_sqrelu_rmsnorm_act_quant_bf16", gu, w, q2, s2, r2, 1e-5, M, K)
    sync()
    assert torch.equal(q1, q2) and torch.equal(s1, s2) and torch.equal(r1, r2)
    assert np.array_equal(host(r2), host(q2).astype(np.int32).sum(1))
    lib, f = pkg.lib(), ctypes.c_float(1e-5)
    p = [t.data_ptr() for t in (gu, w, q2, s2, r2)]
    assert lib.vla_sqrelu_rmsnorm_act_quant_bf16(0, p[1], p[2], p[3], p[4], f, M, K, 0) == pkg.VLA_K_ERR_ARG
    assert lib.vla_sqrelu_rmsnorm_act_quant_bf16(p[0], p[1], p[2], p[3], p[4], f, 1, 8200, 0) == pkg.VLA_K_ERR_SHAPE
    assert lib.vla_sqrelu_rmsnorm_act_quant_bf16(p[0], p[1], p[2], p[3], p[4], f, 1, 100, 0) == pkg.VLA_K_ERR_SHAPE
    assert lib.vla_sqrelu_rmsnorm_act_quant_bf16(p[0] + 2, p[1], p[2], p[3], p[4], f, 1, 64, 0) == pkg.VLA_K_ERR_SHAPE
    assert lib.vla_sqrelu_rmsnorm_act_quant_bf16(p[0], p[1], p[2], p[3], p[4], f, 0, K, 0) == pkg.VLA_K_OK


def test_rmsnorm_ternary_gemv_rejects_what_it_cannot_hold():
    lib, f = pkg.lib(), ctypes.c_float(1e-5)
    buf = torch.zeros(16 * 8192, dtype=torch.int16, device="cuda")
    p = buf.data_ptr()
    assert lib.vla_rmsnorm_ternary_gemv(p, p, f, p, p, 0, p, 1, 9, 64, 256, 0) == pkg.VLA_K_ERR_SHAPE   # rows
    assert lib.vla_rmsnorm_ternary_gemv(p, p, f, p, p, 0, p, 1, 4, 64, 8192, 0) == pkg.VLA_K_ERR_SHAPE  # row length
    assert lib.vla_rmsnorm_ternary_gemv(p, p, f, p, p, 0, p, 1, 4, 64, 200, 0) == pkg.VLA_K_ERR_SHAPE
    assert lib.vla_rmsnorm_ternary_gemv(p, p, f, p, p, 0, p, 3, 4, 64, 256, 0) == pkg.VLA_K_ERR_SHAPE   # N % ws_num
    assert lib.vla_rmsnorm_ternary_gemv(0, p, f, p, p, 0, p, 1, 4, 64, 256, 0) == pkg.VLA_K_ERR_ARG
    assert lib.vla_rmsnorm_ternary_gemv(p, p, f, p, p, 0, p, 1, 0, 64, 256, 0) == pkg.VLA_K_OK


def test_ternary_pipeline_matches_cpu_twin():
    # act-quant + ternary GEMM + epilogue against the reference's CPU formulation
    # (fp32 fake-quant GEMM, src/models/bitvla.cpp:173-176): same number up to bf16 rounding.
    r = np.random.default_rng(109)
    M, N, K = 40, 640, 2560
    x = orc.round_bf16(r.standard_normal((M, K)).astype(np.float32))
    W = (0.02 * r.standard_normal((N, K))).astype(np.float32)
    t, am = orc.weight_quant_ternary(W)
    q = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    rs = torch.zeros(M, dtype=torch.int32, device="cuda")
    pkg.call("vla_act_quant_bf16", dev(orc.to_bf16(x)), q, s, rs, M, K)
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    pkg.call("vla_ternary_gemm", q, dev(_pack_plain(t)), out, None, s, rs, dev(np.float32([am])), 1, M, N, K)
    sync()
    want = orc.bit_linear_f32(x, t, am)
    got = orc.from_bf16(host(out, np.uint16))
    assert bf16_close(got, want) and rel_err(got, want) < 5e-3


# ------------------------------------------------------- BitVLA LM context
class _LmLayer(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in (
        "attn_norm_w", "attn_sub_norm_w", "ffn_norm_w", "ffn_sub_norm_w", "q_packed", "q_ws", "k_packed", "k_ws", "v_packed",
        "v_ws", "o_packed", "o_ws", "gate_up_packed", "gate_up_ws", "down_packed", "down_ws")]


def test_bitvla_lm_context_forward_follows_the_oracle():
    # init / set_layer / set_output_norm / forward / free with the reference's argument meaning:
    # two full layers (attention and squared-ReLU GLU halves) over 37 tokens against the CPU
    # restatement of run_layer; plus the error returns (sequence too long, unbound layer).
    import oracle.chunk as orc_chunk
    lib = pkg.lib()
    H, n_q, n_kv, D, F, L, seq, eps, base = 256, 4, 2, 64, 384, 2, 37, 1e-5, 500000.0
    r = np.random.default_rng(0xB17)
    keep, layers_o = [], []

    def tern(N, K, n_ws):
        t = r.choice(np.int8([-1, 0, 0, 1]), (N, K))
        ws = (0.02 + 0.01 * r.random(n_ws)).astype(np.float32)
        dp, dws = dev(_pack_plain(t)), dev(ws)
        keep.extend([dp, dws])
        return (t, ws), dp.data_ptr(), dws.data_ptr()

    def norm(K):
        wv = orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32))
        d = dev(wv)
        keep.append(d)
        return orc.from_bf16(wv), d.data_ptr()

    assert lib.bitvla_lm_hip_init(H, n_q, n_kv, D, F, L, base, eps, 0) is None        # no sequence
    assert lib.bitvla_lm_hip_init(200, n_q, n_kv, D, F, L, base, eps, 48) is None      # K not a multiple of 128
    ctx = lib.bitvla_lm_hip_init(H, n_q, n_kv, D, F, L, base, eps, 48)
    assert ctx
    x = orc.to_bf16(r.standard_normal((seq, H)).astype(np.float32))
    d_in, d_out = dev(x), torch.zeros((seq, H), dtype=torch.int16, device="cuda")
    on_o, on_p = norm(H)
    lib.bitvla_lm_hip_set_output_norm(ctx, on_p)
    assert lib.bitvla_lm_hip_forward(ctx, d_in.data_ptr(), d_out.data_ptr(), seq, None) == -1   # layers not bound
    for l in range(L):
        st, lo = _LmLayer(), {}
        for name, K in (("attn_norm", H), ("sub_norm", n_q * D), ("ffn_norm", H), ("ffn_sub_norm", F)):
            lo[name], p = norm(K)
            setattr(st, {"sub_norm": "attn_sub_norm_w"}.get(name, name + "_w"), p)
        for name, N, K, n_ws in (("q", n_q * D, H, 1), ("k", n_kv * D, H, 1), ("v", n_kv * D, H, 1), ("o", H, n_q * D, 1),
                                 ("gate_up", 2 * F, H, 2), ("down", H, F, 1)):
            lo[name], pp, pw = tern(N, K, n_ws)
            setattr(st, name + "_packed", pp)
            setattr(st, name + "_ws", pw)
        lib.bitvla_lm_hip_set_layer(ctx, l, ctypes.byref(st))
        layers_o.append(lo)
    assert lib.bitvla_lm_hip_forward(ctx, d_in.data_ptr(), d_out.data_ptr(), 49, None) == -1    # longer than max_seq
    assert lib.bitvla_lm_hip_forward(ctx, d_in.data_ptr(), d_out.data_ptr(), seq, None) == 0
    sync()
    got = orc.from_bf16(host(d_out, np.uint16))
    want = orc_chunk.bitvla_lm_forward(orc.from_bf16(x), layers_o, on_o, n_q, n_kv, D, eps, base)
    # a one-ulp difference before a quantisation can flip an int8 code, so a few elements may sit
    # outside the per-element bar; the bulk and the worst case are both bounded
    bad = np.abs(got - want) > 1e-2 + 2e-2 * np.abs(want)
    assert bad.mean() < 5e-3 and rel_err(got, want) < 3e-2, (bad.mean(), rel_err(got, want))
    # a second forward on a shorter sequence reuses the workspace
    assert lib.bitvla_lm_hip_forward(ctx, d_in.data_ptr(), d_out.data_ptr(), 5, None) == 0
    sync()
    want5 = orc_chunk.bitvla_lm_forward(orc.from_bf16(x[:5]), layers_o, on_o, n_q, n_kv, D, eps, base)
    assert rel_err(orc.from_bf16(host(d_out, np.uint16))[:5], want5) < 3e-2
    lib.bitvla_lm_hip_free(ctx)
    lib.bitvla_lm_hip_free(None)


def test_gate_up_squared_relu_bit_exact():
    import oracle.chunk as orc_chunk
    r = np.random.default_rng(77)
    for seq, ffn in ((5, 384), (3, 20)):   # vector and scalar paths
        gu = orc.to_bf16((r.standard_normal((seq, 2 * ffn)) * 3).astype(np.float32))
        out = torch.zeros((seq, ffn), dtype=torch.int16, device="cuda")
        pkg.call("gate_up_fused_sqrelu_mul_bf16", dev(gu), out, seq, ffn)
        sync()
        assert np.array_equal(host(out, np.uint16), orc.to_bf16(orc_chunk.sqrelu_mul(orc.from_bf16(gu), ffn)))


# ------------------------------------------------------- BitVLA layer helpers
def test_bitvla_layout_helpers_and_softmax():
    r = np.random.default_rng(110)
    S, H, hd, n_kv = 37, 20, 128, 5
    x = r.integers(0, 65536, (S, H * hd)).astype(np.uint16)
    t = torch.zeros((H, S, hd), dtype=torch.int16, device="cuda")
    pkg.call("bitvla_transpose_sNhd_to_NshHd_bf16", dev(x), t, S, H, hd)
    back = torch.zeros((S, H * hd), dtype=torch.int16, device="cuda")
    pkg.call("bitvla_transpose_NshHd_to_sNhd_bf16", t, back, H, S, hd)
    rep = torch.zeros((H, S, hd), dtype=torch.int16, device="cuda")
    pkg.call("bitvla_repeat_kv_bf16", t[:n_kv].contiguous(), rep, H, n_kv, S, hd)
    ids = np.int32([5, 5, 0, 36])
    gat = torch.zeros((4, H * hd), dtype=torch.int16, device="cuda")
    pkg.call("bitvla_gather_rows_bf16", dev(x), gat, dev(ids), 4, H * hd)
    sync()
    want_t = orc.transpose_sHd_to_Hsd(x, H)
    assert np.array_equal(host(t, np.uint16), want_t)
    assert np.array_equal(host(back, np.uint16), x)
    assert np.array_equal(host(rep, np.uint16), orc.repeat_kv(want_t[:n_kv], H))
    assert np.array_equal(host(gat, np.uint16), orc.gather_rows(x, ids))
    sc = orc.to_bf16((r.standard_normal((40, 519)) * 8).astype(np.float32))
    sd = dev(sc)
    pkg.call("bitvla_softmax_scaled_bf16", sd, 0.0883883, 40, 519)
    a, b = dev(orc.to_bf16(r.standard_normal(1000).astype(np.float32))), dev(orc.to_bf16(r.standard_normal(1000).astype(np.float32)))
    c = torch.zeros(1000, dtype=torch.int16, device="cuda")
    pkg.call("bitvla_add_bf16", a, b, c, 1000)
    sync()
    want = orc.from_bf16(orc.softmax_scaled_bf16(sc, 0.0883883))
    got = orc.from_bf16(host(sd, np.uint16))
    assert np.abs(got - want).max() <= 2 ** -8 * max(want.max(), 1e-3)
    assert np.array_equal(host(c, np.uint16), orc.to_bf16(orc.from_bf16(host(a, np.uint16)) + orc.from_bf16(host(b, np.uint16))))


# ---------------------------------------------------------- flow-matching glue
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_embed_suffix_and_euler_step(out_dtype):
    r = np.random.default_rng(111)
    B, S, n_lead, A, W = 3, 51, 1, 32, 1024
    x_t = r.standard_normal((B, S - n_lead, A)).astype(np.float32)
    W_in = (0.1 * r.standard_normal((W, A))).astype(np.float32)
    bias = r.standard_normal(W).astype(np.float32)
    lead = r.standard_normal((B, n_lead, W)).astype(np.float32)
    h = empty((B, S, W), out_dtype)
    pkg.call("vla_embed_suffix", dev(x_t), dev(W_in), dev(bias), dev(lead), h, out_dtype, B, S, n_lead, A, W)
    sync()
    want = np.concatenate([lead, (orc.linear(x_t.reshape(-1, A), W_in, bias)).reshape(B, S - n_lead, W)], axis=1)
    got = as_f32(h, out_dtype)
    assert rel_err(got, want) < (FP32_TOL if out_dtype == F32 else 8e-3)
    # with an activation on the projected rows (lead rows are copied as they are), and the
    # state-token rows written over a buffer afterwards
    h2 = empty((B, S, W), out_dtype)
    pkg.call("vla_embed_suffix_act", dev(x_t), dev(W_in), dev(bias), dev(lead), h2, out_dtype, B, S, n_lead, A, W, pkg.VLA_ACT_SILU)
    h3 = empty((B, S, W), out_dtype)
    pkg.call("vla_set_lead_rows", dev(lead), h3, out_dtype, B, S, n_lead, W)
    sync()
    want2 = want.copy()
    want2[:, n_lead:] = orc.silu(want[:, n_lead:])
    assert rel_err(as_f32(h2, out_dtype), want2) < (FP32_TOL if out_dtype == F32 else 8e-3)
    got3 = as_f32(h3, out_dtype)
    assert not got3[:, n_lead:].any() and rel_err(got3[:, :n_lead], lead) < (1e-7 if out_dtype == F32 else 8e-3)
    W_out = (0.05 * r.standard_normal((A, W))).astype(np.float32)
    b_out = r.standard_normal(A).astype(np.float32)
    xd = dev(x_t)
    pkg.call("vla_euler_step", xd, h, dev(W_out), dev(b_out), out_dtype, B, S, n_lead, A, W, -0.1)
    sync()
    v = orc.linear(got[:, n_lead:].reshape(-1, W), W_out, b_out).reshape(B, S - n_lead, A)
    assert rel_err(host(xd), x_t - 0.1 * v) < FP32_TOL
