"""Writer for "VLAW" checkpoints (the container libvla.so loads; layout in
host/checkpoint.h) and seeded synthetic weights for the benchmark configurations.

The reference loads GGUF files produced by its converters (scripts/*.py); with
no checkpoints or network here, every configuration is driven by seeded Gaussian
weights of the reference architectures' shapes.
"""
import struct

import numpy as np

_DT = {np.dtype(np.float32): "f32", np.dtype(np.int8): "i8", np.dtype(np.uint8): "u8", np.dtype(np.int32): "i32"}


def to_bf16_bits(x):
    """fp32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def bf16_round(x):
    return (to_bf16_bits(x).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(x))


class BF16:
    """Marks an fp32 array that is to be stored as bf16."""

    def __init__(self, values):
        self.values = np.ascontiguousarray(values, np.float32)


def write_vlaw(path, config, tensors):
    """config: dict of scalars/strings; tensors: dict name -> ndarray or BF16."""
    lines = ["K %s %s" % (k, v) for k, v in config.items()]
    blobs, off = [], 0
    for name, t in tensors.items():
        if isinstance(t, BF16):
            raw, dt, shape = to_bf16_bits(t.values).tobytes(), "bf16", t.values.shape
        else:
            t = np.ascontiguousarray(t)
            raw, dt, shape = t.tobytes(), _DT[t.dtype], t.shape
        lines.append("T %s %s %d %s %d %d" % (name, dt, len(shape), " ".join(str(d) for d in shape), off, len(raw)))
        pad = (-len(raw)) % 64
        blobs.append(raw + b"\0" * pad)
        off += len(raw) + pad
    header = ("\n".join(lines) + "\n").encode()
    with open(path, "wb") as f:
        f.write(b"VLAW0001")
        f.write(struct.pack("<Q", len(header)))
        f.write(header)
        f.write(b"\0" * ((-(16 + len(header))) % 64))
        for b in blobs:
            f.write(b)


# ------------------------------------------------------------------ configurations
def smolvla_config(n_layers=16, dtype="bf16", suffix_mask=0, num_steps=10):
    """SmolVLA-shape expert (src/models/smolvla.cpp:444-452, 604-630): VLM width 960,
    15 query / 5 KV heads of 64, expert width 720, 64 image tokens per view, 48 text
    tokens, 1 state token, 50 action tokens.  suffix_mask 0 = bidirectional suffix,
    1 = the reference's causal suffix block."""
    return dict(arch="smolvla", dtype=dtype, n_layers=n_layers, n_q_heads=15, n_kv_heads=5, head_dim=64, hidden=960,
                expert_h=720, n_img=64, n_lang=48, n_suffix=50, max_action_dim=32, max_state_dim=32,
                real_action_dim=32, real_state_dim=32, num_steps=num_steps, rms_eps=1e-5, rope_freq_base=10000.0,
                self_attn_every_n=2, min_period=4e-3, max_period=4.0, vocab=512, suffix_mask=suffix_mask, max_views=3)


def pi0_config(n_layers=18, dtype="bf16", num_steps=10):
    """pi0 shape (PaliGemma-2B prefix KV, 300M Gemma expert; src/models/pi0.cpp:250-298):
    MQA 8 / 1 heads of 256, backbone 2048, expert 1024, 256 image tokens per view,
    48 text tokens, suffix = 1 state + 50 action tokens."""
    return dict(arch="pi0", dtype=dtype, n_layers=n_layers, n_q_heads=8, n_kv_heads=1, head_dim=256, hidden=2048,
                expert_h=1024, n_img=256, n_lang=48, n_suffix=51, max_action_dim=32, max_state_dim=32,
                real_action_dim=32, real_state_dim=32, num_steps=num_steps, rms_eps=1e-6, rope_freq_base=10000.0,
                self_attn_every_n=1, min_period=4e-3, max_period=4.0, vocab=512, suffix_mask=2, max_views=3)


def pi05_config(n_layers=18, dtype="bf16", num_steps=10):
    """pi0.5 shape (src/models/pi05.cpp:292-328): the pi0 backbone and expert widths with
    adaRMS norms conditioned on the flow time, no state token (suffix = 50 action tokens,
    the state travels as text) and up to 200 text tokens."""
    c = pi0_config(n_layers, dtype, num_steps)
    c.update(arch="pi05", n_lang=200, n_suffix=50, suffix_mask=0)
    return c


def gr00t_config(n_layers=16, dtype="bf16", num_steps=4, n_suffix=17):
    """GR00T N1.5 DiT head (src/modules/dit_head.h:38-45): width 1536, 32 heads of 48,
    cross-attention on even layers onto 148 backbone tokens per view of width 2048,
    self-attention on odd layers; 1 state + 16 action tokens."""
    return dict(arch="gr00t_n1d5", dtype=dtype, n_layers=n_layers, n_q_heads=32, n_kv_heads=32, head_dim=48,
                hidden=2048, expert_h=1536, n_img=148, n_lang=0, n_suffix=n_suffix, max_action_dim=32,
                max_state_dim=64, real_action_dim=32, real_state_dim=64, num_steps=num_steps, rms_eps=1e-5,
                norm_out_eps=1e-6, rope_freq_base=10000.0, vocab=0, suffix_mask=0, max_views=2)


def gr00t_head_io_config(n_layers=16, dtype="bf16", num_steps=4, ffn_dim=6144):
    """GR00T N1.5 with the DiT head's own input / output MLPs (src/models/gr00tn1d5.cpp:281, 366-381;
    src/modules/action_expert.cpp:41-59; src/modules/dit_head.cpp:139-147): the sequence is
    1 state token (encode_state) + 32 learned future tokens + 16 action tokens (encode_action with
    the step's sinusoid and learned positions), every block has its FFN, and the velocity is
    decode(proj_out(h)) on the action rows."""
    c = gr00t_config(n_layers, dtype, num_steps, n_suffix=1 + 32 + 16)
    c.update(head_io=1, num_future=32, dit_out_dim=1024, dec_hidden=1024, state_hidden=1024, ffn_dim=ffn_dim,
             num_buckets=1000, max_pos=1024)
    return c


def gr00t_n1d6_config(n_layers=32, dtype="bf16", num_steps=4, n_suffix=17, attend_text_every_n=2, dit_interleave=1):
    """GR00T N1.6 / N1.7 DiT head (AlternateVLDiT, src/models/gr00tn1d6.cpp:85-86, 445-467;
    src/models/gr00tn1d7.cpp:75, 565-590): the N1.5 block, 32 layers, whose cross layers
    alternate between the text rows (layer % (2 attend_text_every_n) == 0) and the image rows
    of the backbone features; up to 64 text rows (an embedding lookup stands in for them)."""
    c = gr00t_config(n_layers, dtype, num_steps, n_suffix)
    c.update(arch="gr00t_n1d6", n_lang=64, vocab=512, attend_text_every_n=attend_text_every_n, dit_interleave=dit_interleave)
    return c


def gr00t_n1d6_head_config(n_layers=32, dtype="bf16", num_steps=4, ffn_dim=6144, variant="n1_6"):
    """GR00T N1.6 / N1.7 as the reference loads them from GGUF (src/models/gr00tn1d6.cpp:75-126,
    294-298, 436-467; src/models/gr00tn1d7.cpp:60-100, 556-590): the alternating head with its own
    input / output MLPs, no future tokens (the sequence is 1 state + action_horizon rows), and
    vlln, an affine LayerNorm on the backbone rows.  N1.6: horizon 50, 128 action / state values;
    N1.7: horizon 40, 132, and vlln inside the backbone (a VL self-attention stack follows it), so not on this path."""
    AH, A = (50, 128) if variant == "n1_6" else (40, 132)
    c = gr00t_n1d6_config(n_layers, dtype, num_steps, n_suffix=1 + AH)
    c.update(head_io=1, num_future=0, dit_out_dim=1024, dec_hidden=1024, state_hidden=1024, ffn_dim=ffn_dim,
             num_buckets=1000, max_pos=1024, max_action_dim=A, real_action_dim=A, max_state_dim=A, real_state_dim=A,
             vlln=1 if variant == "n1_6" else 0, vlln_eps=1e-5, variant=variant)
    return c


def bitvla_config(n_layers=30):
    """BitVLA / BitNet b1.58 2B shape (src/models/bitvla.cpp:121-122): width 2560,
    20 query / 5 KV heads of 128, RoPE base 5e5; prefix 256 image + 256 text tokens,
    7 action tokens appended one at a time."""
    return dict(arch="bitvla", dtype="bf16", n_layers=n_layers, n_q_heads=20, n_kv_heads=5, head_dim=128, hidden=2560,
                n_img=256, n_lang=256, n_suffix=7, max_action_dim=32, real_action_dim=32, rms_eps=1e-5,
                rope_freq_base=500000.0, vocab=512)


def _is_self(cfg, l):
    if cfg["arch"] in ("pi0", "pi05"):
        return True
    if cfg["arch"] == "smolvla":
        return l % cfg["self_attn_every_n"] == 0
    return l % 2 == 1 and bool(cfg.get("dit_interleave", 1))  # gr00t: cross on even layers


def synth_weights(cfg, seed=0x5EED):
    """Seeded weights: matrices N(0, 0.02), norm weights 1 + N(0, 0.05), biases
    N(0, 0.02); values of bf16 models are bf16-representable.  Returns a dict of
    fp32 arrays (ternary BitVLA projections as int8 {-1,0,1} plus a scale)."""
    r = np.random.default_rng(seed)
    bf = cfg["dtype"] == "bf16"
    rnd = bf16_round if bf else (lambda x: np.asarray(x, np.float32))
    mat = lambda n, k, s=0.02: rnd((s * r.standard_normal((n, k))).astype(np.float32))
    vec = lambda n, s=0.02: (s * r.standard_normal(n)).astype(np.float32)
    nrm = lambda n: rnd((1.0 + 0.05 * r.standard_normal(n)).astype(np.float32))
    w = {}
    arch = cfg["arch"]
    D, Hq, Hkv = cfg["head_dim"], cfg["n_q_heads"], cfg["n_kv_heads"]
    qd, kvd, Wv = Hq * D, Hkv * D, cfg["hidden"]
    A = cfg["max_action_dim"]
    if arch == "bitvla":
        H = Wv
        w["prefix.E_lang"] = r.standard_normal((cfg["vocab"], H)).astype(np.float32)
        w["act.emb"] = r.standard_normal((cfg["n_suffix"], H)).astype(np.float32)
        w["act.norm"] = bf16_round((1.0 + 0.05 * r.standard_normal(H)).astype(np.float32))
        w["act.W_out"] = (0.02 * r.standard_normal((A, H))).astype(np.float32)
        w["act.b_out"] = vec(A)
        for l in range(cfg["n_layers"]):
            p = "lm.%d." % l
            w[p + "attn_norm"] = bf16_round((1.0 + 0.05 * r.standard_normal(H)).astype(np.float32))
            w[p + "sub_norm"] = bf16_round((1.0 + 0.05 * r.standard_normal(H)).astype(np.float32))
            # ternary with P(0) = 0.5, P(+-1) = 0.25; one absmean-like fp32 scale per source tensor
            w[p + "Wqkv.t"] = r.choice(np.int8([-1, 0, 0, 1]), size=(qd + 2 * kvd, H)).astype(np.int8)
            # absmean of N(0, 0.02) weights is 0.02*sqrt(2/pi); +-10% per source tensor
            w[p + "Wqkv.ws"] = (0.02 * np.sqrt(2 / np.pi) * r.uniform(0.9, 1.1, 3)).astype(np.float32)
            w[p + "Wo.t"] = r.choice(np.int8([-1, 0, 0, 1]), size=(H, qd)).astype(np.int8)
            w[p + "Wo.ws"] = (0.02 * np.sqrt(2 / np.pi) * r.uniform(0.9, 1.1, 1)).astype(np.float32)
            F = cfg.get("ffn_dim", 0)
            if F > 0:  # the squared-ReLU GLU half of run_layer (bitvla_lm_cuda.cu:488-520): [gate; up] rows, down
                w[p + "ffn_norm"] = bf16_round((1.0 + 0.05 * r.standard_normal(H)).astype(np.float32))
                w[p + "ffn_sub_norm"] = bf16_round((1.0 + 0.05 * r.standard_normal(F)).astype(np.float32))
                w[p + "Wgu.t"] = r.choice(np.int8([-1, 0, 0, 1]), size=(2 * F, H)).astype(np.int8)
                w[p + "Wgu.ws"] = (0.02 * np.sqrt(2 / np.pi) * r.uniform(0.9, 1.1, 2)).astype(np.float32)
                w[p + "Wd.t"] = r.choice(np.int8([-1, 0, 0, 1]), size=(H, F)).astype(np.int8)
                w[p + "Wd.ws"] = (0.02 * np.sqrt(2 / np.pi) * r.uniform(0.9, 1.1, 1)).astype(np.float32)
        return w
    W = cfg["expert_h"]
    if cfg.get("vocab", 0) > 0:
        # N1.6: the rows stand for backbone features at the text positions, O(1) like the image rows
        w["prefix.E_lang"] = (r.standard_normal((cfg["vocab"], Wv)) / (1.0 if arch == "gr00t_n1d6" else np.sqrt(Wv))).astype(np.float32)
    if cfg.get("vlln", 0):
        w["prefix.vlln_w"] = (1.0 + 0.1 * r.standard_normal(Wv)).astype(np.float32)
        w["prefix.vlln_b"] = vec(Wv, 0.1)
    if arch == "smolvla":
        w["prefix.Wstate"] = (0.1 * r.standard_normal((Wv, cfg["max_state_dim"]))).astype(np.float32)
        w["prefix.bstate"] = vec(Wv, 0.1)
    elif arch != "pi05":
        w["act.W_sp"] = (0.1 * r.standard_normal((W, cfg["max_state_dim"]))).astype(np.float32)
        w["act.b_sp"] = vec(W, 0.1)
    if cfg.get("head_io", 0):
        del w["act.W_sp"], w["act.b_sp"]
        Hs, Hd, O, NF = cfg["state_hidden"], cfg["dec_hidden"], cfg["dit_out_dim"], cfg["num_future"]
        f32m = lambda n, k, s_: (s_ * r.standard_normal((n, k))).astype(np.float32)
        w["aex.se_l1W"], w["aex.se_l1b"] = f32m(Hs, cfg["max_state_dim"], 0.1), vec(Hs, 0.1)
        w["aex.se_l2W"], w["aex.se_l2b"] = f32m(W, Hs, 1.0 / np.sqrt(Hs)), vec(W, 0.1)
        w["aex.ae_W1"], w["aex.ae_b1"] = f32m(W, A, 0.1), vec(W, 0.1)
        w["aex.ae_W2"], w["aex.ae_b2"] = f32m(W, 2 * W, 1.0 / np.sqrt(2 * W)), vec(W, 0.1)
        w["aex.ae_W3"], w["aex.ae_b3"] = f32m(W, W, 1.0 / np.sqrt(W)), vec(W, 0.1)
        w["aex.pos_embd"] = f32m(cfg.get("max_pos", 64), W, 0.02)
        if NF > 0:
            w["aex.future_tokens"] = f32m(NF, W, 0.5)
        w["aex.po1W"], w["aex.po1b"] = f32m(2 * W, W, 0.02), vec(2 * W)
        w["aex.po2W"], w["aex.po2b"] = mat(O, W), vec(O)
        w["aex.ad_l1W"], w["aex.ad_l1b"] = mat(Hd, O), vec(Hd)
        w["aex.ad_l2W"], w["aex.ad_l2b"] = f32m(A, Hd, 0.02), vec(A)
    else:
        w["act.W_in"] = (0.1 * r.standard_normal((W, A))).astype(np.float32)
        w["act.b_in"] = vec(W, 0.1)
        w["act.W_out"] = (0.02 * r.standard_normal((A, W))).astype(np.float32)
        w["act.b_out"] = vec(A)
    # adaRMS modulation dense: rows [scale; shift; gate], the gate around 1 (pi05.cpp:208-224)
    ada_w = lambda: (0.5 * r.standard_normal((3 * W, W)) / np.sqrt(W)).astype(np.float32)
    ada_b = lambda: np.concatenate([vec(2 * W, 0.05), 1.0 + vec(W, 0.05)]).astype(np.float32)
    if arch == "pi05":
        w["te.W_tin"] = (r.standard_normal((W, W)) / np.sqrt(W)).astype(np.float32)
        w["te.b_tin"] = vec(W, 0.1)
        w["te.W_tout"] = (r.standard_normal((W, W)) / np.sqrt(W)).astype(np.float32)
        w["te.b_tout"] = vec(W, 0.1)
        w["act.ada_final_w"] = ada_w()
        w["act.ada_final_b"] = ada_b()
    elif arch not in ("gr00t_n1d5", "gr00t_n1d6"):
        w["act.norm"] = nrm(W)
        if cfg.get("time_mlp", 0):  # action_time_mlp_in / _out of the suffix embedding
            w["act.W_at1"] = (r.standard_normal((W, 2 * W)) / np.sqrt(2 * W)).astype(np.float32)
            w["act.b_at1"] = vec(W, 0.1)
            w["act.W_at2"] = (r.standard_normal((W, W)) / np.sqrt(W)).astype(np.float32)
            w["act.b_at2"] = vec(W, 0.1)
    else:
        w["te.l1W"] = (0.05 * r.standard_normal((W, 256))).astype(np.float32)
        w["te.l1b"] = vec(W)
        w["te.l2W"] = (0.02 * r.standard_normal((W, W))).astype(np.float32)
        w["te.l2b"] = vec(W)
    for l in range(cfg["n_layers"]):
        p, v = "ex.%d." % l, "vlm.%d." % l
        self_l = _is_self(cfg, l)
        if arch in ("gr00t_n1d5", "gr00t_n1d6"):
            w[p + "adaln_w"] = mat(2 * W, W)
            w[p + "adaln_b"] = vec(2 * W)
            if self_l:
                w[p + "Wqkv"] = mat(qd + 2 * kvd, W)
                w[p + "bqkv"] = vec(qd + 2 * kvd)
            else:
                w[p + "Wq"] = mat(qd, W)
                w[p + "bq"] = vec(qd)
                w[v + "Wkv"] = mat(2 * kvd, Wv)
                w[v + "bkv"] = vec(2 * kvd)
            w[p + "Wo"] = mat(W, qd)
            w[p + "bo"] = vec(W)
            if cfg.get("ffn_dim", 0) > 0:  # ffn_gelu of the DiT block
                w[p + "W1"] = mat(cfg["ffn_dim"], W)
                w[p + "b1"] = vec(cfg["ffn_dim"])
                w[p + "W2"] = mat(W, cfg["ffn_dim"])
                w[p + "b2"] = vec(W)
            continue
        if arch == "pi05":
            w[p + "ada_in_w"], w[p + "ada_in_b"] = ada_w(), ada_b()
            if cfg.get("ffn_dim", 0) > 0:
                w[p + "ada_post_w"], w[p + "ada_post_b"] = ada_w(), ada_b()
        else:
            w[p + "ln"] = nrm(W)
        w[v + "ln"] = nrm(Wv)
        w[v + "Wkv"] = mat(2 * kvd, Wv)
        if self_l:
            w[p + "Wqkv"] = mat(qd + 2 * kvd, W)
        else:
            w[p + "Wq"] = mat(qd, W)
            w[p + "Wk_x"] = mat(kvd, kvd, 0.05)
            w[p + "Wv_x"] = mat(kvd, kvd, 0.05)
        w[p + "Wo"] = mat(W, qd)
        if cfg.get("ffn_dim", 0) > 0:  # post-attention norm, [gate; up] rows, down
            if arch != "pi05":
                w[p + "ln2"] = nrm(W)
            w[p + "Wgu"] = mat(2 * cfg["ffn_dim"], W)
            w[p + "Wd"] = mat(W, cfg["ffn_dim"])
    return w


_F32_NAMES = ("prefix.", "act.", "te.", "aex.")


def write_synthetic(path, cfg, weights, ladder_pack=None, plain_pack=None):
    """Write `weights` (from synth_weights) as a VLAW file.  BitVLA ternary tensors are
    stored ladder-packed ("*.i2" + "*.ws") when ladder_pack (a function
    int8 [N,K] -> uint8 bytes) is given, in the gfx950 word order ("*.p2" + "*.ws") when
    plain_pack is given, else as dequantised fp32 the loader re-quantises."""
    bf = cfg["dtype"] == "bf16"
    out = {}
    for name, t in weights.items():
        if name.endswith(".t"):
            base = name[:-2]
            if ladder_pack is not None:
                out[base + ".i2"] = np.ascontiguousarray(ladder_pack(t), np.uint8)
                out[base + ".ws"] = weights[base + ".ws"]
            elif plain_pack is not None:
                out[base + ".p2"] = np.ascontiguousarray(plain_pack(t), np.uint8)
                out[base + ".ws"] = weights[base + ".ws"]
            else:
                # fp32 weights whose absmean quantisation gives back (t, scale): t * scale
                # has mean |w| = scale * P(nonzero); store exactly that product per source tensor.
                out[base] = _dequant_sources(cfg, base, t, weights[base + ".ws"])
            continue
        if name.endswith(".ws"):
            continue
        small = name.startswith(_F32_NAMES) or name.endswith((".bqkv", ".bq", ".bo", ".bkv", ".adaln_b", ".b1", ".b2", ".ada_in_w", ".ada_in_b",
                                                            ".ada_post_w", ".ada_post_b"))
        if cfg["arch"] == "bitvla" and name.endswith(("attn_norm", "sub_norm", "ffn_norm")):
            out[name] = BF16(t)
        elif bf and not small:
            out[name] = BF16(t)
        else:
            out[name] = np.ascontiguousarray(t, np.float32)
    if cfg["arch"] == "bitvla" and "act.norm" in out:
        out["act.norm"] = np.ascontiguousarray(weights["act.norm"], np.float32)
    write_vlaw(path, cfg, out)


def _dequant_sources(cfg, base, t, ws):
    kvd = cfg["n_kv_heads"] * cfg["head_dim"]
    parts = [cfg["hidden"], kvd, kvd] if base.endswith("Wqkv") else ([t.shape[0] // 2] * 2 if base.endswith("Wgu") else [t.shape[0]])
    out = np.empty(t.shape, np.float32)
    row = 0
    for n, s in zip(parts, ws):
        out[row:row + n] = t[row:row + n].astype(np.float32) * np.float32(s)
        row += n
    return out
