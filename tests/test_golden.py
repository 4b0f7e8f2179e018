"""Committed golden data: the reference-held known-answer vectors
(tests/golden/reference_vectors.json) against the oracle, the oracle against its own
committed outputs (tests/golden/path_fixtures.npz, written by make_fixtures.py), and -- on
a GPU -- the HIP path against the same fixtures through the C ABI."""
import importlib.util
import json
import math
import os

import numpy as np
import pytest

import oracle as orc
from conftest import mt19937_raw

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")


def _vectors():
    with open(os.path.join(GOLD, "reference_vectors.json")) as f:
        return json.load(f)


def _fixtures():
    return np.load(os.path.join(GOLD, "path_fixtures.npz"))


def test_reference_known_answer_vectors_hold_for_the_oracle():
    v = _vectors()
    rh = v["rotate_half"]
    assert np.array_equal(orc.rotate_half(np.float32(rh["input"])), np.float32(rh["output"]))
    tab = v["ternary_code_table"]
    word = sum(c << (2 * i) for i, c in enumerate(tab["codes"]))  # codes 0..3 in values 0, 4, 8, 12 of a slot (byte 0)
    dec = orc.decode_i2s_to_i8s(np.uint32(word))
    assert [int(dec[4 * j]) for j in range(4)] == tab["values"]
    slot = v["ladder_slot_bit_positions"]
    for idx, sh in zip(slot["value_index"], slot["bit_shift"]):
        dec = orc.decode_i2s_to_i8s(np.uint32(3 << sh))  # code 3 (+1) in one position, code 0 (-2) elsewhere
        assert dec[idx] == 1 and sum(int(x == 1) for x in dec) == 1
    aq = v["act_quant"]
    q, s = orc.act_quant(np.float32([aq["row"]]))
    assert list(q[0]) == aq["q"] and s[0] == aq["scale"]
    amax = 4.0  # a row whose scale is 127/4: entries t*4/127 land on t exactly
    row = np.float32([amax] + [t * amax / 127.0 for t in aq["ties_times_scale"]])
    q, _ = orc.act_quant(row[None])
    assert list(q[0][1:]) == aq["ties_rounded"]
    rec = v["gemm_check_recipe"]
    assert int(mt19937_raw(5489, 1)[0]) == rec["mt19937_default_seed_first_output"]
    tp = v["timesteps_proj"]
    out0, out250 = orc.timesteps_proj(0), orc.timesteps_proj(250)
    assert np.allclose(out0[:128], tp["t0_cos_half"], atol=1e-6) and np.allclose(out0[128:], tp["t0_sin_half"], atol=1e-6)
    assert abs(out250[0] - tp["t250_channel0"]) < 1e-5 and abs(tp["t250_channel0"] - math.cos(250.0)) < 1e-12


def test_oracle_reproduces_its_committed_fixtures_bit_for_bit():
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLD, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh, stored = mod.build(), _fixtures()
    assert sorted(fresh) == sorted(stored.files)
    for k in fresh:
        assert np.array_equal(np.asarray(fresh[k]), stored[k]), k


@pytest.mark.gpu
def test_hip_path_against_committed_fixtures():
    import torch
    from util import dev, host, pkg, rel_err
    fx = _fixtures()
    F32, BF16 = pkg.VLA_DT_F32, pkg.VLA_DT_BF16
    # attention, fp32 and bf16, mask generated in the kernel
    S, Hq, Hkv, D, P, p0, p1 = [int(x) for x in fx["attn_geom"]]
    T, t_max = P + S, (P + S + 63) // 64 * 64
    for dt, want, tol in ((F32, fx["attn_out"], 1e-5), (BF16, fx["attn_out_bf16_inputs"], 1e-2)):
        conv = (lambda a: dev(np.ascontiguousarray(a, np.float32))) if dt == F32 else (lambda a: dev(orc.to_bf16(a)))
        tdt = torch.float32 if dt == F32 else torch.int16
        kc = torch.zeros((1, Hkv, t_max, D), dtype=tdt, device="cuda")
        vc = torch.zeros((1, Hkv, D, t_max), dtype=tdt, device="cuda")
        pkg.call("vla_kv_append", kc, vc, conv(fx["attn_k"]), conv(fx["attn_v"]), dt, 1, Hkv, D, t_max, 0, T)
        out = torch.zeros((1, S, Hq * D), dtype=tdt, device="cuda")
        pkg.call("vla_attn_prefix_suffix", conv(fx["attn_q"]), kc, vc, out, dt, 1, S, Hq, Hkv, D, t_max, T,
                 1.0 / math.sqrt(D), pkg.VLA_MASK_CAUSAL_SUFFIX, P, p0, p1, None)
        torch.cuda.synchronize()
        got = host(out) if dt == F32 else orc.from_bf16(host(out, np.uint16))
        assert rel_err(got.reshape(S, Hq * D), want.reshape(S, Hq * D)) < tol
        # gather returns the appended K bit for bit
        kb = torch.zeros((1, T, Hkv, D), dtype=tdt, device="cuda")
        vb = torch.zeros_like(kb)
        pkg.call("vla_kv_gather", kc, vc, kb, vb, dt, 1, Hkv, D, t_max, 0, T)
        torch.cuda.synchronize()
        assert torch.equal(kb[0], conv(fx["attn_k"]))
    # RoPE
    x = dev(fx["rope_x"].copy())
    n_tok, H, Dr = fx["rope_x"].shape
    pkg.call("vla_rope_neox", x, dev(fx["rope_cos"]), dev(fx["rope_sin"]), F32, n_tok, n_tok, H, Dr)
    torch.cuda.synchronize()
    assert rel_err(host(x), fx["rope_out"]) < 1e-6
    # ternary: host quantiser and packer, act-quant, exact accumulators, epilogue
    W, t = fx["tern_w"], fx["tern_t"]
    N, K = t.shape
    tq = np.empty_like(t)
    am = np.zeros(1, np.float32)
    assert pkg.lib().vla_ternary_quant_host(np.ascontiguousarray(W).ctypes.data, W.size, tq.ctypes.data, am.ctypes.data) == 0
    assert np.array_equal(tq, t) and am[0] == fx["tern_absmean"][0]
    packed = np.empty(pkg.lib().vla_ternary_packed_words(N, K), np.uint32)
    assert pkg.lib().vla_ternary_repack_ladder_host(fx["tern_ladder"].ctypes.data, N, K, packed.ctypes.data) == 0
    M = fx["tern_x"].shape[0]
    q8 = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    s = torch.zeros(M, device="cuda")
    rs = torch.zeros(M, dtype=torch.int32, device="cuda")
    pkg.call("vla_act_quant_bf16", dev(orc.to_bf16(fx["tern_x"])), q8, s, rs, M, K)
    acc = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    pkg.call("vla_ternary_gemm", q8, dev(packed), out, acc, s, rs, dev(fx["tern_absmean"]), 1, M, N, K)
    torch.cuda.synchronize()
    assert np.array_equal(host(q8), fx["tern_q8"]) and np.array_equal(host(s), fx["tern_s"])
    assert np.array_equal(host(acc), fx["tern_acc"]) and np.array_equal(host(out, np.uint16), fx["tern_out"])
    # RMSNorm
    y = torch.zeros(fx["norm_x"].shape, device="cuda")
    Mn, Kn = fx["norm_x"].shape
    pkg.call("vla_rms_norm", dev(fx["norm_x"]), dev(fx["norm_w"]), y, F32, Mn, Kn, 1e-5)
    torch.cuda.synchronize()
    assert rel_err(host(y), fx["norm_out"]) < 1e-6
    # the widened layer pieces: gated FFN through the GLU epilogue, biased GELU FFN, adaRMS, gated residual
    x, Wg, Wu, Wd = fx["ffn_x"], fx["ffn_wg"], fx["ffn_wu"], fx["ffn_wd"]
    M, K = x.shape
    I = Wg.shape[0]
    Wgu = dev(np.concatenate([Wg, Wu], 0))
    for act, want in ((pkg.VLA_ACT_SILU, fx["ffn_glu_silu"]), (pkg.VLA_ACT_GELU, fx["ffn_glu_gelu"])):
        mid = torch.zeros((M, I), device="cuda")
        y = torch.zeros((M, K), device="cuda")
        pkg.call("vla_glu_linear", dev(x), Wgu, None, mid, F32, F32, M, I, K, act, -1.0)
        pkg.call("vla_linear", mid, dev(Wd), None, None, y, F32, F32, M, K, I)
        torch.cuda.synchronize()
        assert rel_err(host(y), want) < 1e-5
    mid = torch.zeros((M, I), device="cuda")
    y = torch.zeros((M, K), device="cuda")
    pkg.call("vla_linear_act", dev(x), dev(Wg), dev(fx["ffn_b1"]), None, mid, F32, F32, M, I, K, pkg.VLA_ACT_GELU)
    pkg.call("vla_linear", mid, dev(Wd), dev(fx["ffn_b2"]), None, y, F32, F32, M, K, I)
    ya = torch.zeros((M, K), device="cuda")
    pkg.call("vla_adarms", dev(x), dev(fx["ada_scale"]), dev(fx["ada_shift"]), ya, F32, M, K, 1e-6)
    yg = torch.zeros((M, K), device="cuda")
    pkg.call("vla_linear_gated", dev(x), dev(fx["gated_w"]), None, dev(fx["gated_gate"]), dev(x), yg, F32, F32, M, K, K)
    torch.cuda.synchronize()
    assert rel_err(host(y), fx["ffn_gelu"]) < 1e-5 and rel_err(host(ya), fx["ada_out"]) < 1e-6
    assert rel_err(host(yg), fx["gated_out"]) < 1e-5
