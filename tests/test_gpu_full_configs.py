"""The BASELINE configurations at the batch sizes and depths that bench.py times.

Kernel selection follows the batch (key slices, partial formats, tile shapes), so the dispatch
that produces the reported numbers is the dispatch checked here: every configuration runs at
its full depth and its benchmark batch through vla_predict_batch, and the first and the last
observation of the batch are held to the CPU oracle -- both to the oracle that rounds where the
GPU stores bf16 and to the pure fp32 oracle, which is what "bf16 within 2e-2 relative / 1e-2
absolute of the CPU reference on the action-chunk output" refers to.

BitVLA (config 4) re-quantises every activation to int8, which turns a one-ulp bf16 difference
into a different integer code now and then; through 30 layers the chunk output of the *oracle
itself* moves by more than the bf16 bar when one input in a hundred changes by one ulp.  Two
tests therefore: per layer, teacher-forced (each layer is fed the oracle's input for that layer),
the per-element bar holds; end to end the bar is derived in the test from the oracle's own
sensitivity, measured on the same weights and observation.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle as orc
from oracle import chunk as orc_chunk
from util import dev, host, one_ulp_noise, pkg

pytestmark = pytest.mark.gpu

from vla_cpp_amd import checkpoint as ckpt  # noqa: E402
from vla_cpp_amd import ffi  # noqa: E402
from test_gpu_chunk import bf16_close, load, make_obs  # noqa: E402


def _check_first_and_last(cfg, w, obs, got):
    for b in (0, len(obs) - 1):
        want_e = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=False)
        assert np.isfinite(got[b]).all()
        assert bf16_close(got[b], want_e), (b, np.abs(got[b] - want_e).max())
        assert bf16_close(got[b], want), (b, np.abs(got[b] - want).max())


@pytest.mark.timeout(600)
def test_config1_smolvla_16_layers_batch_32(tmp_path):
    cfg = ckpt.smolvla_config(n_layers=16, dtype="bf16", suffix_mask=0)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 21)
    r = np.random.default_rng(2100)
    obs = [make_obs(cfg, r, n_views=3) for _ in range(32)]
    m = load(tmp_path, cfg, w, "cfg1_b32")
    got = m.predict_batch(obs).reshape(32, 50, 32)
    _check_first_and_last(cfg, w, obs, got)
    again = m.predict_batch(obs).reshape(32, 50, 32)  # the captured graph
    assert np.array_equal(again, got)
    m.close()


@pytest.mark.timeout(900)
def test_config2_pi0_18_layers_batch_16(tmp_path):
    cfg = ckpt.pi0_config(n_layers=18)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 22)
    r = np.random.default_rng(2200)
    obs = [make_obs(cfg, r, n_views=3) for _ in range(16)]
    m = load(tmp_path, cfg, w, "cfg2_b16")
    got = m.predict_batch(obs).reshape(16, 50, 32)
    _check_first_and_last(cfg, w, obs, got)
    assert np.array_equal(m.predict_batch(obs).reshape(16, 50, 32), got)
    # batch 1: seven key slices instead of four -- the other dispatch the bench line reports
    solo = m.predict(obs[0]).reshape(50, 32)
    want = orc_chunk.flow_expert_chunk(cfg, w, obs[0], emulate_bf16=False)
    assert bf16_close(solo, want), np.abs(solo - want).max()
    m.close()


@pytest.mark.timeout(600)
def test_config3_gr00t_16_blocks_batch_64(tmp_path):
    cfg = ckpt.gr00t_config(n_layers=16)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 23)
    r = np.random.default_rng(2300)
    obs = [make_obs(cfg, r, n_views=2) for _ in range(64)]
    m = load(tmp_path, cfg, w, "cfg3_b64")
    got = m.predict_batch(obs).reshape(64, 16, 32)
    _check_first_and_last(cfg, w, obs, got)
    assert np.array_equal(m.predict_batch(obs).reshape(64, 16, 32), got)
    m.close()


@pytest.mark.timeout(900)
def test_config4_bitvla_30_layers_batch_8_against_the_oracles_own_sensitivity(tmp_path):
    cfg = ckpt.bitvla_config(n_layers=30)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 24)
    r = np.random.default_rng(2400)
    obs = [make_obs(cfg, r, n_views=1) for _ in range(8)]
    for o in obs:
        o["img_emb"] = orc.round_bf16(o["img_emb"])
    m = load(tmp_path, cfg, w, "cfg4_b8", ladder_pack=orc.pack_ladder_int2)
    got = m.predict_batch(obs).reshape(8, 7, 32)
    assert np.array_equal(m.predict_batch(obs).reshape(8, 7, 32), got)
    # batch 1 at full depth, the reference's own operating point: its decode attention is dispatched
    # differently (key slices merged in the launch by the slice that arrives last instead of inside a workgroup)
    got1 = m.predict_batch(obs[:1]).reshape(1, 7, 32)
    assert np.array_equal(m.predict_batch(obs[:1]).reshape(1, 7, 32), got1)
    m.close()
    # the oracle's sensitivity: the same observation with 1 % of its image embeddings one bf16 ulp away
    want0, _ = orc_chunk.bitvla_chunk(cfg, w, obs[0])
    pert = dict(obs[0], img_emb=one_ulp_noise(obs[0]["img_emb"], r))
    wantp, _ = orc_chunk.bitvla_chunk(cfg, w, pert)
    noise_max, noise_mean = np.abs(wantp - want0).max(), np.abs(wantp - want0).mean()
    assert noise_max > 0

    def outside(a, ref):  # share of outputs outside the literal bf16 bar, 2e-2 relative / 1e-2 absolute
        return float(np.mean(np.abs(a - ref) > 1e-2 + 2e-2 * np.abs(ref)))

    noise_share = outside(wantp, want0)
    for name, b, g in (("b=0 of 8", 0, got[0]), ("b=7 of 8", 7, got[7]), ("batch 1", 0, got1[0])):
        want = want0 if b == 0 else orc_chunk.bitvla_chunk(cfg, w, obs[b])[0]
        err = np.abs(g - want)
        share = outside(g, want)
        print("cfg4 %s: |gpu-oracle| max %.4f mean %.4f, %.1f %% outside the literal bar ; oracle under 1-ulp input noise max %.4f "
              "mean %.4f, %.1f %% outside ; |want| max %.3f"
              % (name, err.max(), err.mean(), 100 * share, noise_max, noise_mean, 100 * noise_share, np.abs(want).max()))
        # measured: the GPU sits closer to the oracle (max 0.033, mean 0.009) than the oracle
        # to itself under the probe (max 0.035, mean 0.009)
        assert err.max() <= 1.5 * noise_max + 1e-2 and err.mean() <= 1.5 * noise_mean + 2e-3, (name, err.max(), err.mean(), noise_max, noise_mean)
        # the literal bar on the chunk itself: no more outputs leave it than leave it when the oracle's
        # own input moves by one bf16 ulp (1.5x, plus one output of the 224)
        assert share <= 1.5 * noise_share + 1.0 / g.size, (name, share, noise_share)
    # the same observation alone and inside the batch agree within the bf16 bar of the path's stages
    assert np.abs(got1[0] - got[0]).max() <= 1.5 * noise_max + 1e-2


class _LmLayer(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in (
        "attn_norm_w", "attn_sub_norm_w", "ffn_norm_w", "ffn_sub_norm_w", "q_packed", "q_ws", "k_packed", "k_ws", "v_packed",
        "v_ws", "o_packed", "o_ws", "gate_up_packed", "gate_up_ws", "down_packed", "down_ws")]


def _pack(t):
    N, K = t.shape
    out = np.zeros(pkg.lib().vla_ternary_packed_words(N, K), np.uint32)
    assert pkg.lib().vla_ternary_pack_host(np.ascontiguousarray(t).ctypes.data, N, K, out.ctypes.data) == 0
    return out


def _bf_dev(a):
    return dev(orc.to_bf16(np.ascontiguousarray(a, np.float32)))


def _bf_host(t):
    return orc.from_bf16(host(t, np.uint16))


@pytest.mark.timeout(900)
def test_config4_bitvla_30_layers_teacher_forced_stage_by_stage():
    # BitNet b1.58 2B layer geometry (width 2560, 20 / 5 heads of 128, FFN 6912), 30 distinct
    # layers, 96 tokens.  Every stage of run_layer (src/kernels/bitvla/bitvla_lm_cuda.cu:422-520)
    # is run on the GPU from the ORACLE's input to that stage, so no stage ever sees a GPU-made
    # input and nothing compounds.  Between two quantisation points the arithmetic is integer:
    # those stages must reproduce the oracle bit for bit.  The floating-point stages (the four
    # norms and RoPE + attention) are held to the per-element bar 2e-2 relative / 1e-2 absolute.
    # Then the whole layer runs through the context API (bitvla_lm_hip_*), where the stages feed
    # each other and an int8 code can flip on a one-ulp difference: its distance to the oracle
    # is bounded by the oracle's own distance to itself under one-ulp input noise.
    lib = pkg.lib()
    H, n_q, n_kv, D, F, L, seq, eps, base = 2560, 20, 5, 128, 6912, 30, 96, 1e-5, 500000.0
    hq, hkv = n_q * D, n_kv * D
    r = np.random.default_rng(0xB30)
    ctx = lib.bitvla_lm_hip_init(H, n_q, n_kv, D, F, 1, base, eps, seq)
    assert ctx
    on = orc.to_bf16((1 + 0.1 * r.standard_normal(H)).astype(np.float32))
    d_on = dev(on)
    lib.bitvla_lm_hip_set_output_norm(ctx, d_on.data_ptr())
    cos_t, sin_t = orc.rope_tables(np.arange(seq, dtype=np.int32), D, base)
    d_cos, d_sin = dev(cos_t), dev(sin_t)
    rb = orc.round_bf16
    x = rb(r.standard_normal((seq, H)).astype(np.float32))
    t_max = 128
    i8 = lambda K: torch.zeros((seq, K), dtype=torch.int8, device="cuda")
    bfz = lambda K: torch.zeros((seq, K), dtype=torch.int16, device="cuda")
    sc, rs = torch.zeros(seq, dtype=torch.float32, device="cuda"), torch.zeros(seq, dtype=torch.int32, device="cuda")
    worst_float, worst_layer, worst_ratio = 0.0, 0.0, 0.0

    def norm_stage(xin, wname, lo, wdev):
        out = bfz(xin.shape[1])
        pkg.call("bitvla_rmsnorm_bf16", _bf_dev(xin), wdev[wname], out, eps, seq, xin.shape[1])
        want = rb(orc.rms_norm(xin, lo[wname], eps))
        got = _bf_host(out)
        assert bf16_close(got, want), (wname, np.abs(got - want).max())
        return want, float(np.abs(got - want).max())

    def exact_linear(xn, name, lo, wdev, n_ws, residual=None):
        """act-quant + ternary GEMM (+ residual) from the oracle's normalised rows: bit-exact."""
        K = xn.shape[1]
        t, ws = lo[name]
        q8 = i8(K)
        pkg.call("vla_act_quant_bf16", _bf_dev(xn), q8, sc, rs, seq, K)
        out = bfz(t.shape[0])
        if residual is None:
            pkg.call("vla_ternary_gemm", q8, wdev[name][0], out, None, sc, rs, wdev[name][1], n_ws, seq, t.shape[0], K)
        else:
            pkg.call("vla_ternary_gemm_add", q8, wdev[name][0], out, _bf_dev(residual), sc, rs, wdev[name][1], n_ws, seq, t.shape[0], K)
        q, s = orc.act_quant(xn)
        y = orc.from_bf16(orc.ternary_epilogue(orc.ternary_gemm_i32(q, t), s, np.asarray(ws, np.float32)))
        want = y if residual is None else rb(residual + y)
        torch.cuda.synchronize()
        assert np.array_equal(orc.to_bf16(want), host(out, np.uint16)), name
        return want

    for l in range(L):
        st, lo, wdev = _LmLayer(), {}, {}
        for name, K in (("attn_norm", H), ("sub_norm", hq), ("ffn_norm", H), ("ffn_sub_norm", F)):
            wv = orc.to_bf16((1 + 0.1 * r.standard_normal(K)).astype(np.float32))
            wdev[name] = dev(wv)
            lo[name] = orc.from_bf16(wv)
            setattr(st, {"sub_norm": "attn_sub_norm_w"}.get(name, name + "_w"), wdev[name].data_ptr())
        for name, N, K, n_ws in (("q", hq, H, 1), ("k", hkv, H, 1), ("v", hkv, H, 1), ("o", H, hq, 1), ("gate_up", 2 * F, H, 2),
                                 ("down", H, F, 1)):
            t = r.choice(np.int8([-1, 0, 0, 1]), (N, K))
            ws = (0.02 * np.sqrt(2 / np.pi) * r.uniform(0.9, 1.1, n_ws)).astype(np.float32)
            wdev[name] = (dev(_pack(t)), dev(ws))
            lo[name] = (t, ws)
            setattr(st, name + "_packed", wdev[name][0].data_ptr())
            setattr(st, name + "_ws", wdev[name][1].data_ptr())

        # ---- attention half, stage by stage from the oracle's inputs
        hn, e = norm_stage(x, "attn_norm", lo, wdev)
        worst_float = max(worst_float, e)
        q = exact_linear(hn, "q", lo, wdev, 1).reshape(seq, n_q, D)
        k = exact_linear(hn, "k", lo, wdev, 1).reshape(seq, n_kv, D)
        v = exact_linear(hn, "v", lo, wdev, 1).reshape(seq, n_kv, D)
        dq, dk = _bf_dev(q), _bf_dev(k)
        pkg.call("vla_rope_neox", dq, d_cos, d_sin, pkg.VLA_DT_BF16, seq, seq, n_q, D)
        pkg.call("vla_rope_neox", dk, d_cos, d_sin, pkg.VLA_DT_BF16, seq, seq, n_kv, D)
        kc = torch.zeros((1, n_kv, t_max, D), dtype=torch.int16, device="cuda")
        vc = torch.zeros((1, n_kv, D, t_max), dtype=torch.int16, device="cuda")
        pkg.call("vla_kv_append", kc, vc, dk, _bf_dev(v), pkg.VLA_DT_BF16, 1, n_kv, D, t_max, 0, seq)
        att_d = bfz(hq)
        pkg.call("vla_attn_prefix_suffix", dq, kc, vc, att_d, pkg.VLA_DT_BF16_P2, 1, seq, n_q, n_kv, D, t_max, seq,
                 1.0 / np.sqrt(D), pkg.VLA_MASK_NONE, seq, 0, 0, None)
        qo, ko = rb(orc.rope_neox(q, cos_t, sin_t)), rb(orc.rope_neox(k, cos_t, sin_t))
        att = rb(orc.attention(qo, ko, v, None, 1.0 / np.sqrt(D))).reshape(seq, hq)
        torch.cuda.synchronize()
        assert bf16_close(_bf_host(dq).reshape(qo.shape), qo) and bf16_close(_bf_host(dk).reshape(ko.shape), ko)
        got_att = _bf_host(att_d)
        assert bf16_close(got_att, att), (l, np.abs(got_att - att).max())
        worst_float = max(worst_float, float(np.abs(got_att - att).max()))
        sn, e = norm_stage(att, "sub_norm", lo, wdev)
        worst_float = max(worst_float, e)
        h1 = exact_linear(sn, "o", lo, wdev, 1, residual=x)
        # ---- squared-ReLU GLU half
        fn, e = norm_stage(h1, "ffn_norm", lo, wdev)
        worst_float = max(worst_float, e)
        gu = exact_linear(fn, "gate_up", lo, wdev, 2)
        act_d = bfz(F)
        pkg.call("gate_up_fused_sqrelu_mul_bf16", _bf_dev(gu), act_d, seq, F)
        act = orc_chunk.sqrelu_mul(gu, F)
        torch.cuda.synchronize()
        assert np.array_equal(host(act_d, np.uint16), orc.to_bf16(act))
        fs, e = norm_stage(act, "ffn_sub_norm", lo, wdev)
        worst_float = max(worst_float, e)
        h2 = exact_linear(fs, "down", lo, wdev, 1, residual=h1)
        want = rb(orc.rms_norm(h2, orc.from_bf16(on), eps))
        # the staged oracle above is the oracle's own layer
        assert np.array_equal(want, orc_chunk.bitvla_lm_forward(x, [lo], orc.from_bf16(on), n_q, n_kv, D, eps, base))

        # ---- the whole layer through the context API against the oracle's own sensitivity
        lib.bitvla_lm_hip_set_layer(ctx, 0, ctypes.byref(st))
        d_out = bfz(H)
        assert lib.bitvla_lm_hip_forward(ctx, _bf_dev(x).data_ptr(), d_out.data_ptr(), seq, None) == 0
        torch.cuda.synchronize()
        got = _bf_host(d_out)
        noisy = orc_chunk.bitvla_lm_forward(one_ulp_noise(x, r), [lo], orc.from_bf16(on), n_q, n_kv, D, eps, base)
        d_gpu, d_self = np.abs(got - want), np.abs(noisy - want)
        bar = 1e-2 + 2e-2 * np.abs(want)
        ratio = d_gpu.mean() / d_self.mean()
        worst_layer, worst_ratio = max(worst_layer, float(d_gpu.max())), max(worst_ratio, float(ratio))
        assert d_gpu.mean() <= 1.5 * d_self.mean() and (d_gpu > bar).mean() <= 1.5 * (d_self > bar).mean() + 1e-3, (
            l, d_gpu.mean(), d_self.mean(), (d_gpu > bar).mean(), (d_self > bar).mean())
        x = want  # teacher forcing: the next layer's input is the oracle's
    print("teacher-forced BitVLA: float stages worst |gpu - oracle| %.4f; whole layers worst |diff| %.4f, "
          "worst mean-distance ratio to the oracle's one-ulp self-distance %.2f" % (worst_float, worst_layer, worst_ratio))
    lib.bitvla_lm_hip_free(ctx)
