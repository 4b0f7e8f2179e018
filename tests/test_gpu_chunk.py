"""Whole action-chunk parity through the model-level C ABI (vla_model_load /
vla_predict / vla_predict_batch) against the chunk oracle, one test per BASELINE
configuration family.

Tolerances: fp32 (config 0) 1e-5 relative on the chunk output; bf16 configs
2e-2 relative / 1e-2 absolute on the chunk output.
"""
import os

import numpy as np
import pytest

import oracle as orc
from oracle import chunk as orc_chunk
from util import one_ulp_noise, pkg, rel_err

pytestmark = pytest.mark.gpu

from vla_cpp_amd import checkpoint as ckpt  # noqa: E402
from vla_cpp_amd import ffi  # noqa: E402


def bf16_close(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) <= 1e-2 + 2e-2 * np.abs(want)))


def make_obs(cfg, r, n_views, n_lang=None, bf16_inputs=False):
    A = cfg["max_action_dim"]
    n_act = cfg["n_suffix"] - (0 if cfg["arch"] in ("smolvla", "bitvla", "pi05") else 1 + cfg.get("num_future", 0) * cfg.get("head_io", 0))
    img = r.standard_normal((n_views * cfg["n_img"], cfg["hidden"])).astype(np.float32)
    if cfg["arch"] == "smolvla":
        img /= np.sqrt(cfg["hidden"])  # the prefix builder scales image rows by sqrt(hidden)
    obs = dict(img_emb=img, n_views=n_views, noise=r.standard_normal((n_act, A)).astype(np.float32))
    if cfg.get("vocab", 0) > 0:
        n_lang = cfg["n_lang"] if n_lang is None else n_lang
        obs["lang"] = r.integers(0, cfg["vocab"], n_lang).astype(np.int32)
    if cfg.get("max_state_dim", 0) > 0:
        obs["state"] = r.standard_normal(cfg["max_state_dim"]).astype(np.float32)
    return obs


def load(tmp_path, cfg, w, name, **kw):
    path = os.path.join(str(tmp_path), name + ".vlaw")
    ckpt.write_synthetic(path, cfg, w, **kw)
    return ffi.Model(path)


@pytest.mark.parametrize("suffix_mask,n_lang", [(0, 48), (1, 48), (1, 37)])
def test_config0_smolvla_single_layer_fp32(tmp_path, suffix_mask, n_lang):
    cfg = ckpt.smolvla_config(n_layers=1, dtype="f32", suffix_mask=suffix_mask)
    w = ckpt.synth_weights(cfg, seed=0x5EED)
    r = np.random.default_rng(200 + suffix_mask + n_lang)
    obs = make_obs(cfg, r, n_views=3, n_lang=n_lang)
    m = load(tmp_path, cfg, w, "cfg0")
    got = m.predict(obs).reshape(50, 32)
    c = m.config()
    assert (c.n_q_heads, c.n_kv_heads, c.head_dim, c.n_suffix, c.num_steps) == (15, 5, 64, 50, 10)
    want = orc_chunk.flow_expert_chunk(cfg, w, obs)
    assert rel_err(got, want) < 1e-5, rel_err(got, want)
    st = m.stats()
    assert st.ms_total > 0
    # the same handle, a second observation: the resident cache is rebuilt, not reused
    obs2 = make_obs(cfg, r, n_views=3, n_lang=n_lang)
    got2 = m.predict(obs2).reshape(50, 32)
    assert rel_err(got2, orc_chunk.flow_expert_chunk(cfg, w, obs2)) < 1e-5
    m.close()


@pytest.mark.parametrize("n_layers,batch", [(4, 1), (16, 3)])
def test_config1_smolvla_stack_bf16(tmp_path, n_layers, batch):
    cfg = ckpt.smolvla_config(n_layers=n_layers, dtype="bf16", suffix_mask=0)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 1)
    r = np.random.default_rng(210 + n_layers)
    obs = [make_obs(cfg, r, n_views=3) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "cfg1")
    got = m.predict_batch(obs).reshape(batch, 50, 32)
    for b in range(batch):
        want_e = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
        assert bf16_close(got[b], want_e), np.abs(got[b] - want_e).max()
        if b == 0:
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=False)
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
    # batch elements are independent: element 0 alone gives the same chunk
    solo = m.predict(obs[0]).reshape(50, 32)
    assert np.array_equal(solo, got[0])
    m.close()


def test_config1_reference_causal_mask_and_language_padding(tmp_path):
    cfg = ckpt.smolvla_config(n_layers=4, dtype="bf16", suffix_mask=1)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 2)
    r = np.random.default_rng(220)
    obs = make_obs(cfg, r, n_views=2, n_lang=30)
    m = load(tmp_path, cfg, w, "cfg1c")
    got = m.predict(obs).reshape(50, 32)
    assert bf16_close(got, orc_chunk.flow_expert_chunk(cfg, w, obs, emulate_bf16=True))
    m.close()


@pytest.mark.parametrize("n_layers,batch", [(3, 2), (18, 1)])
def test_config2_pi0_mqa_bf16(tmp_path, n_layers, batch):
    cfg = ckpt.pi0_config(n_layers=n_layers)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 3)
    r = np.random.default_rng(230)
    obs = [make_obs(cfg, r, n_views=3) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "cfg2")
    got = m.predict_batch(obs).reshape(batch, 50, 32)
    for b in range(batch):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
        assert bf16_close(got[b], want), np.abs(got[b] - want).max()
        if b == 0:  # and the pure fp32 CPU reference, which is what the tolerance is quoted against
            want32 = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=False)
            assert bf16_close(got[b], want32), np.abs(got[b] - want32).max()
    m.close()


def test_config2_pi0_in_the_references_default_fp32(tmp_path):
    # pi0's default activation type in the reference is F32 (src/models/pi0.cpp:90, 174-176):
    # 256-wide heads in fp32, held to 1e-5 like config 0
    cfg = ckpt.pi0_config(n_layers=3, dtype="f32")
    w = ckpt.synth_weights(cfg, seed=0x5EED + 8)
    r = np.random.default_rng(231)
    obs = [make_obs(cfg, r, n_views=2) for _ in range(2)]
    m = load(tmp_path, cfg, w, "cfg2_f32")
    got = m.predict_batch(obs).reshape(2, 50, 32)
    for b in range(2):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b])
        assert rel_err(got[b], want) < 1e-5, rel_err(got[b], want)
    m.close()


@pytest.mark.parametrize("n_layers,batch", [(4, 2), (16, 1)])
def test_config3_gr00t_dit_bf16(tmp_path, n_layers, batch):
    cfg = ckpt.gr00t_config(n_layers=n_layers)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 4)
    r = np.random.default_rng(240)
    obs = [make_obs(cfg, r, n_views=2) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "cfg3")
    got = m.predict_batch(obs).reshape(batch, 16, 32)
    for b in range(batch):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
        assert bf16_close(got[b], want), np.abs(got[b] - want).max()
        if b == 0:  # and the pure fp32 CPU reference, which is what the tolerance is quoted against
            want32 = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=False)
            assert bf16_close(got[b], want32), np.abs(got[b] - want32).max()
    m.close()


@pytest.mark.parametrize("fold_mb,batch", [("0", 2), (None, 33)])
def test_gr00t_blocks_with_and_without_the_folded_modulation(tmp_path, monkeypatch, fold_mb, batch):
    # The per-step folded adaLN operands are a memory-for-launches trade with a budget
    # (VLA_ADALN_FOLD_MB): over it the blocks run adaln + projection as two launches.  Batch 33
    # takes the self blocks' one-launch front half (eight observations per workgroup, the last
    # group with one).  Both against the oracle.
    if fold_mb is not None:
        monkeypatch.setenv("VLA_ADALN_FOLD_MB", fold_mb)
    cfg = ckpt.gr00t_config(n_layers=4)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 77)
    r = np.random.default_rng(377)
    obs = [make_obs(cfg, r, n_views=1) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "gr00t_fold")
    got = m.predict_batch(obs).reshape(batch, 16, 32)
    for b in (0, batch - 1):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
        assert bf16_close(got[b], want), np.abs(got[b] - want).max()
    m.close()


@pytest.mark.parametrize("dtype,n_layers,batch", [("f32", 2, 1), ("bf16", 4, 2), ("bf16", 16, 1)])
def test_gr00t_with_the_dit_heads_own_input_and_output_mlps(tmp_path, dtype, n_layers, batch):
    # The real GR00T N1.5 head (src/models/gr00tn1d5.cpp:366-381): state token from encode_state,
    # 32 learned future tokens, 16 action tokens from encode_action (step sinusoid, learned
    # positions), 49 tokens through DiT blocks with their FFN, velocity = decode(proj_out(h)).
    cfg = ckpt.gr00t_head_io_config(n_layers=n_layers, dtype=dtype, ffn_dim=1024 if n_layers < 16 else 6144)
    if dtype == "f32":
        cfg.update(head_dim=64, n_q_heads=8, n_kv_heads=8, expert_h=512, dit_out_dim=256, dec_hidden=256, state_hidden=256)  # fp32 heads of 48 are not built
    w = ckpt.synth_weights(cfg, seed=0x5EED + 31)
    r = np.random.default_rng(310 + n_layers)
    obs = [make_obs(cfg, r, n_views=2) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "gr00t_io")
    got = m.predict_batch(obs).reshape(batch, 16, 32)
    assert m.config().n_suffix == 49
    for b in range(batch):
        if dtype == "f32":
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b])
            assert rel_err(got[b], want) < 1e-5, rel_err(got[b], want)
        else:
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
            if b == 0:
                want32 = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=False)
                assert bf16_close(got[b], want32), np.abs(got[b] - want32).max()
    # the state really enters through encode_state: another state, another chunk
    other = dict(obs[0], state=obs[0]["state"] + 1.0)
    assert np.abs(m.predict(other).reshape(16, 32) - got[0]).max() > 1e-4
    m.close()


@pytest.mark.parametrize("arch,dtype,n_layers,ffn_dim,batch", [
    ("smolvla", "f32", 2, 256, 1),      # silu gate, fp32: 1e-5
    ("smolvla", "bf16", 4, 2048, 2),    # the expert's real FFN width, pre-norm inside the gate/up launch
    ("pi0", "bf16", 2, 4096, 1),        # gelu gate
    ("gr00t", "bf16", 4, 6144, 2),      # LayerNorm -> ffn_gelu with biases
])
def test_whole_layers_with_the_ffn_half(tmp_path, arch, dtype, n_layers, ffn_dim, batch):
    """The layers with their FFN half (not part of the BASELINE configurations, whose layers
    stop after attention + Wo): post-attention norm, gated or plain FFN, residual."""
    if arch == "smolvla":
        cfg = ckpt.smolvla_config(n_layers=n_layers, dtype=dtype, suffix_mask=1)
    elif arch == "pi0":
        cfg = ckpt.pi0_config(n_layers=n_layers)
    else:
        cfg = ckpt.gr00t_config(n_layers=n_layers)
    cfg["ffn_dim"] = ffn_dim
    w = ckpt.synth_weights(cfg, seed=0x5EED + 9)
    r = np.random.default_rng(290 + ffn_dim)
    obs = [make_obs(cfg, r, n_views=2) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "ffn_" + arch)
    n_act = cfg["n_suffix"] - (0 if arch == "smolvla" else 1)
    got = m.predict_batch(obs).reshape(batch, n_act, 32)
    for b in range(batch):
        if dtype == "f32":
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b])
            assert rel_err(got[b], want) < 1e-5, rel_err(got[b], want)
        else:
            # the bar is against the fp32 oracle.  The bf16-emulating oracle rounds where the
            # two-launch path rounds (normalised activations), the fused launches round elsewhere
            # (folded weights): both are bf16-noisy estimates of the same chunk (the emulating
            # oracle itself sits 0.008 from the fp32 one here), so between them only the mean
            # error and twice the bar are held.
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b])
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
            emu = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
            d = np.abs(got[b] - emu)
            assert d.mean() < 4e-3 and np.all(d <= 2e-2 + 4e-2 * np.abs(emu)), (d.mean(), d.max())
    # without the FFN weights the same observation gives a different chunk: the half is really run
    cfg0 = dict(cfg, ffn_dim=0)
    assert not np.allclose(orc_chunk.flow_expert_chunk(cfg0, w, obs[0], emulate_bf16=dtype != "f32"), got[0], atol=1e-3)
    m.close()


@pytest.mark.parametrize("arch,dtype,batch", [("smolvla", "f32", 1), ("smolvla", "bf16", 3), ("pi0", "bf16", 2)])
def test_suffix_embedding_with_the_action_time_mlp(tmp_path, arch, dtype, batch):
    """The suffix embedding through its real action-time MLP (the BASELINE configurations use
    W_in x + b + time embedding): the library folds the first two projections into one matrix
    and a per-step bias, the oracle follows the reference's order."""
    cfg = ckpt.smolvla_config(n_layers=2, dtype=dtype, suffix_mask=1) if arch == "smolvla" else ckpt.pi0_config(n_layers=2)
    cfg["time_mlp"] = 1
    cfg["ffn_dim"] = 256
    w = ckpt.synth_weights(cfg, seed=0x5EED + 11)
    r = np.random.default_rng(300 + batch)
    obs = [make_obs(cfg, r, n_views=2) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "tmlp_" + arch)
    got = m.predict_batch(obs).reshape(batch, 50, 32)
    for b in range(batch):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=dtype != "f32")
        if dtype == "f32":
            assert rel_err(got[b], want) < 1e-5, rel_err(got[b], want)
        else:
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
    w0 = {k: v for k, v in w.items() if not k.startswith("act.W_at") and not k.startswith("act.b_at")}
    assert not np.allclose(orc_chunk.flow_expert_chunk(cfg, w0, obs[0], emulate_bf16=dtype != "f32"), got[0], atol=1e-3)
    m.close()


@pytest.mark.parametrize("dtype,n_layers,ffn_dim,batch", [
    ("f32", 2, 256, 1),      # fp32: 1e-5
    ("bf16", 3, 0, 2),       # attention half only
    ("bf16", 4, 4096, 2),    # the expert's real FFN width
])
def test_pi05_adarms_layers(tmp_path, dtype, n_layers, ffn_dim, batch):
    """pi0.5 (src/models/pi05.cpp:208-283, 610-631): adaRMS norms whose scale, shift and gate
    come from the flow time, gated residuals, a suffix of action tokens only, no suffix mask."""
    cfg = ckpt.pi05_config(n_layers=n_layers, dtype=dtype)
    cfg["ffn_dim"] = ffn_dim
    if dtype == "f32":
        cfg["head_dim"] = 128  # 256-wide heads are built for bf16 only
    w = ckpt.synth_weights(cfg, seed=0x5EED + 13)
    r = np.random.default_rng(310 + ffn_dim)
    obs = [make_obs(cfg, r, n_views=2, n_lang=57) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "pi05")
    got = m.predict_batch(obs).reshape(batch, 50, 32)
    for b in range(batch):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=dtype != "f32")
        if dtype == "f32":
            assert rel_err(got[b], want) < 1e-5, rel_err(got[b], want)
        else:
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
    # the modulation is live: a chunk computed with all gates at zero is a different chunk
    w0 = {k: (np.zeros_like(v) if "ada_" in k else v) for k, v in w.items()}
    assert not np.allclose(orc_chunk.flow_expert_chunk(cfg, w0, obs[0], emulate_bf16=dtype != "f32"), got[0], atol=1e-3)
    m.close()


@pytest.mark.parametrize("n_layers,every,interleave,n_lang,batch", [
    (8, 2, 1, 21, 2),     # N1.6 / N1.7 defaults: text on layers 0, 4; image on 2, 6; self on odd layers
    (6, 1, 1, 33, 1),     # text on every cross layer
    (4, 2, 0, 21, 2),     # no interleave: all layers cross, text on 0, image on 1, 2, 3
    (4, 2, 1, 0, 1),      # no text rows: the text layers read the image rows
    (32, 2, 1, 64, 1),    # the full depth
])
def test_gr00t_n1d6_alternating_text_and_image_cross_layers(tmp_path, n_layers, every, interleave, n_lang, batch):
    """AlternateVLDiT (src/models/gr00tn1d6.cpp:445-467, src/models/gr00tn1d7.cpp:565-590): the cross
    layers' resident K/V come from the text rows or the image rows of the backbone features."""
    cfg = ckpt.gr00t_n1d6_config(n_layers=n_layers, attend_text_every_n=every, dit_interleave=interleave)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 17)
    r = np.random.default_rng(320 + n_layers)
    obs = [make_obs(cfg, r, n_views=2, n_lang=n_lang) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "n1d6")
    got = m.predict_batch(obs).reshape(batch, 16, 32)
    for b in range(batch):
        want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
        assert bf16_close(got[b], want), np.abs(got[b] - want).max()
    if n_lang:
        # the text rows are really used: other tokens, another chunk
        other = dict(obs[0], lang=(obs[0]["lang"] + 1) % cfg["vocab"])
        assert not np.allclose(orc_chunk.flow_expert_chunk(cfg, w, other, emulate_bf16=True), got[0], atol=1e-3)
    m.close()


@pytest.mark.parametrize("variant,dtype,n_layers,batch", [("n1_6", "bf16", 8, 2), ("n1_6", "f32", 4, 1), ("n1_7", "bf16", 8, 1),
                                                         ("n1_6", "bf16", 32, 1)])
def test_gr00t_n1d6_head_as_its_gguf_loads_it(tmp_path, variant, dtype, n_layers, batch):
    """N1.6 / N1.7 with the head's own MLPs (src/models/gr00tn1d6.cpp:436-479, src/models/gr00tn1d7.cpp:
    556-600): vlln on the backbone rows (N1.6), hh = [state; actions] without future tokens, cross
    layers alternating text / image rows, velocity = decode(proj_out(h)) on the action rows."""
    cfg = ckpt.gr00t_n1d6_head_config(n_layers=n_layers, dtype=dtype, ffn_dim=1024 if n_layers < 32 else 6144, variant=variant)
    if dtype == "f32":
        cfg.update(head_dim=64, n_q_heads=8, n_kv_heads=8, expert_h=512, dit_out_dim=256, dec_hidden=256, state_hidden=256)  # fp32 heads of 48 are not built
    w = ckpt.synth_weights(cfg, seed=0x5EED + 41)
    r = np.random.default_rng(340 + n_layers)
    obs = [make_obs(cfg, r, n_views=2, n_lang=19) for _ in range(batch)]
    m = load(tmp_path, cfg, w, "n1d6_head")
    AH, A = (50, 128) if variant == "n1_6" else (40, 132)
    got = m.predict_batch(obs).reshape(batch, AH, A)
    assert m.config().n_suffix == 1 + AH
    for b in range(batch):
        if dtype == "f32":
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b])
            assert rel_err(got[b], want) < 1e-5, rel_err(got[b], want)
        else:
            want = orc_chunk.flow_expert_chunk(cfg, w, obs[b], emulate_bf16=True)
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
    if variant == "n1_6":
        # vlln is applied: with identity weights the chunk is another one
        w2 = dict(w)
        w2["prefix.vlln_w"], w2["prefix.vlln_b"] = np.ones_like(w["prefix.vlln_w"]), np.zeros_like(w["prefix.vlln_b"])
        assert not np.allclose(orc_chunk.flow_expert_chunk(cfg, w2, obs[0], emulate_bf16=dtype == "bf16"), got[0], atol=1e-3)
    m.close()


@pytest.mark.parametrize("from_fp32,ffn_dim", [(False, 0), (True, 0), (False, 768), (True, 6912)])
def test_config4_bitvla_ternary_append(tmp_path, from_fp32, ffn_dim):
    # ffn_dim > 0: the layers also run their squared-ReLU GLU half (768: the down projection of
    # the decode rows takes the one-launch activation + norm + GEMV; 6912, the model's width: activation + norm + quantisation in one launch, then the GEMV)
    cfg = ckpt.bitvla_config(n_layers=2)
    if ffn_dim:
        cfg["ffn_dim"] = ffn_dim
    w = ckpt.synth_weights(cfg, seed=0x5EED + 5)
    r = np.random.default_rng(250)
    obs = [make_obs(cfg, r, n_views=1) for _ in range(2)]
    m = load(tmp_path, cfg, w, "cfg4", ladder_pack=None if from_fp32 else orc.pack_ladder_int2)
    got = m.predict_batch(obs).reshape(2, 7, 32)
    for b in range(2):
        want, _ = orc_chunk.bitvla_chunk(cfg, w, obs[b], from_fp32=from_fp32)
        if ffn_dim == 0:
            assert bf16_close(got[b], want), np.abs(got[b] - want).max()
        else:
            # Two more quantisations and a squaring per layer: a one-ulp bf16 difference can flip
            # int8 codes, so the per-element bar does not apply end to end (it does stage by stage:
            # test_gpu_full_configs.py).  The bound is the oracle's own distance to itself when
            # 1 % of its bf16 inputs move by one ulp, measured here on the same weights.
            noisy, _ = orc_chunk.bitvla_chunk(cfg, w, dict(obs[b], img_emb=one_ulp_noise(obs[b]["img_emb"], r)), from_fp32=from_fp32)
            d_self, d_gpu = np.abs(noisy - want), np.abs(got[b] - want)
            assert d_gpu.max() <= 1.5 * d_self.max() + 1e-2 and d_gpu.mean() <= 1.5 * d_self.mean() + 2e-3, (
                d_gpu.max(), d_gpu.mean(), d_self.max(), d_self.mean())
    m.close()


def test_graph_replays_match_the_eager_chunk(tmp_path):
    # The first chunk of a shape runs eagerly, the second is captured into a HIP graph,
    # later ones replay it.  Every replay, with other eager work and synchronisations in
    # between, must reproduce the eager result bit for bit.
    import torch
    cfg = ckpt.smolvla_config(n_layers=4, dtype="bf16", suffix_mask=1)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 6)
    r = np.random.default_rng(270)
    obs_a, obs_b = make_obs(cfg, r, n_views=2, n_lang=30), make_obs(cfg, r, n_views=2, n_lang=48)
    m = load(tmp_path, cfg, w, "graph")
    eager_a = m.predict(obs_a)
    eager_b = m.predict(obs_b)  # other padding range: launches change, the graph must follow
    for i in range(3):
        assert np.array_equal(m.predict(obs_a), eager_a), "replay %d of observation A" % i
        torch.zeros(1 << 20, device="cuda").sum().item()  # unrelated eager work + sync
        assert np.array_equal(m.predict(obs_b), eager_b), "replay %d of observation B" % i
    assert bf16_close(eager_a.reshape(50, 32), orc_chunk.flow_expert_chunk(cfg, w, obs_a, emulate_bf16=True))
    # several chunks in one call: the last one is what fetch returns
    m.prefill_batch([obs_a])
    m.denoise_async(3, None)
    assert np.array_equal(m.fetch(), eager_a)
    m.close()
    cfg4 = ckpt.bitvla_config(n_layers=2)
    w4 = ckpt.synth_weights(cfg4, seed=0x5EED + 7)
    obs4 = make_obs(cfg4, r, n_views=1)
    m4 = load(tmp_path, cfg4, w4, "graph4", ladder_pack=orc.pack_ladder_int2)
    first = m4.predict(obs4)
    for i in range(3):
        assert np.array_equal(m4.predict(obs4), first)
    m4.close()


def test_bad_inputs_are_argument_errors_not_crashes(tmp_path):
    cfg = ckpt.smolvla_config(n_layers=1, dtype="f32")
    w = ckpt.synth_weights(cfg)
    m = load(tmp_path, cfg, w, "bad")
    r = np.random.default_rng(260)
    obs = make_obs(cfg, r, n_views=1)
    obs["lang"] = np.int32([cfg["vocab"] + 5] * 4)  # out-of-vocabulary ids (smolvla.cpp:1582-1589)
    with pytest.raises(RuntimeError, match="-1"):
        m.predict(obs)
    obs = make_obs(cfg, r, n_views=9)
    with pytest.raises(RuntimeError, match="-1"):
        m.predict(obs)
    m.close()
    with pytest.raises(RuntimeError):
        ffi.Model(os.path.join(str(tmp_path), "missing.vlaw"))
    # a file whose tensors do not match its own configuration fails at load, whichever tensor it is
    for name, cut in (("ex.0.Wo", (slice(None), slice(0, -16))), ("vlm.0.Wkv", (slice(0, -64), slice(None))), ("act.W_out", (slice(0, -1), slice(None))),
                      ("ex.0.ln", (slice(0, -8),))):
        w2 = dict(w)
        w2[name] = np.ascontiguousarray(w[name][cut])
        with pytest.raises(RuntimeError):
            load(tmp_path, cfg, w2, "misshapen")
    cfg4 = ckpt.bitvla_config(n_layers=1)
    w4 = ckpt.synth_weights(cfg4, seed=1)
    w4["lm.0.Wo.t"] = w4["lm.0.Wo.t"][:-32]
    for pack in (None, orc.pack_ladder_int2):
        with pytest.raises(RuntimeError):
            load(tmp_path, cfg4, w4, "misshapen4", ladder_pack=pack)
