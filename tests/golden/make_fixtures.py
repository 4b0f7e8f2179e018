"""Writes tests/golden/path_fixtures.npz: seeded inputs and the CPU oracle's outputs for small
cases of every kernel on the path.  The fixtures pin the oracle against silent drift (the
CPU suite recomputes them bit for bit) and give the GPU suite expectations that do not
depend on building the oracle on the GPU box.

    python tests/golden/make_fixtures.py

Inputs come from numpy's PCG64 with the seeds below; nothing from the reference is imported
or executed (its algorithm is restated in oracle/)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as orc  # noqa: E402


def build():
    out = {}
    # --- attention: GQA, causal suffix with a padded prefix range (SmolVLA mask recipe)
    r = np.random.default_rng(0xA77)
    S, Hq, Hkv, D, P, pad = 7, 6, 2, 64, 90, (80, 86)
    T = P + S
    Q = r.standard_normal((S, Hq, D)).astype(np.float32)
    K = r.standard_normal((T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((T, Hkv, D)).astype(np.float32)
    mask = orc.mask_smolvla_full(P, S, pad[0], pad[1])
    out.update(attn_q=Q, attn_k=K, attn_v=V, attn_geom=np.int32([S, Hq, Hkv, D, P, pad[0], pad[1]]),
               attn_out=orc.attention(Q, K, V, mask, 1.0 / np.sqrt(D)).astype(np.float32))
    # the same case with bf16-rounded operands (what the bf16 kernels see)
    Qb, Kb, Vb = orc.round_bf16(Q), orc.round_bf16(K), orc.round_bf16(V)
    out["attn_out_bf16_inputs"] = orc.attention(Qb, Kb, Vb, mask, 1.0 / np.sqrt(D)).astype(np.float32)
    # --- RoPE (NeoX) on [tokens, heads, D] with explicit positions
    r = np.random.default_rng(0x20FE)
    x = r.standard_normal((5, 3, 64)).astype(np.float32)
    pos = np.int32([0, 1, 7, 241, 290])
    cos, sin = orc.rope_tables(pos, 64, 10000.0)
    out.update(rope_x=x, rope_pos=pos, rope_cos=cos, rope_sin=sin, rope_out=orc.rope_neox(x, cos, sin))
    # --- ternary path: quantise, pack (ladder), act-quant, int32 GEMM, epilogue
    r = np.random.default_rng(0x7E2)
    N, Kt, M = 64, 256, 9
    W = (0.02 * r.standard_normal((N, Kt))).astype(np.float32)
    t, absmean = orc.weight_quant_ternary(W)
    xa = orc.round_bf16((r.standard_normal((M, Kt)) * 2).astype(np.float32))
    q8, s = orc.act_quant(xa)
    acc = orc.ternary_gemm_i32(q8, t)
    out.update(tern_w=W, tern_t=t, tern_absmean=np.float32([absmean]), tern_ladder=orc.pack_ladder_int2(t),
               tern_x=xa, tern_q8=q8, tern_s=s, tern_acc=acc,
               tern_out=orc.ternary_epilogue(acc, s, np.float32([absmean])))
    # --- RMSNorm and the fused QKV + RoPE + append layout (one self-attention layer's producer)
    r = np.random.default_rng(0x11E)
    h = r.standard_normal((6, 96)).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(96)).astype(np.float32)
    out.update(norm_x=h, norm_w=w, norm_out=orc.rms_norm(h, w, 1e-5))
    # --- the widened layer pieces: gated FFN (silu and gelu), biased GELU FFN, adaRMS, gated residual
    r = np.random.default_rng(0xFF4)
    x = r.standard_normal((6, 96)).astype(np.float32)
    Wg, Wu = (0.1 * r.standard_normal((128, 96))).astype(np.float32), (0.1 * r.standard_normal((128, 96))).astype(np.float32)
    Wd = (0.1 * r.standard_normal((96, 128))).astype(np.float32)
    b1, b2 = (0.1 * r.standard_normal(128)).astype(np.float32), (0.1 * r.standard_normal(96)).astype(np.float32)
    sc, sh = (0.2 * r.standard_normal(96)).astype(np.float32), (0.2 * r.standard_normal(96)).astype(np.float32)
    gate = (1 + 0.2 * r.standard_normal(96)).astype(np.float32)
    Wo = (0.1 * r.standard_normal((96, 96))).astype(np.float32)
    out.update(ffn_x=x, ffn_wg=Wg, ffn_wu=Wu, ffn_wd=Wd, ffn_b1=b1, ffn_b2=b2,
               ffn_glu_silu=orc.ffn_glu(x, Wg, Wu, Wd, orc.silu), ffn_glu_gelu=orc.ffn_glu(x, Wg, Wu, Wd, orc.gelu),
               ffn_gelu=orc.ffn_gelu(x, Wg, b1, Wd, b2),
               ada_scale=sc, ada_shift=sh, ada_out=orc.adarms(x, sc, sh, 1e-6),
               gated_w=Wo, gated_gate=gate, gated_out=(x + orc.linear(x, Wo) * gate).astype(np.float32))
    return out


if __name__ == "__main__":
    fx = build()
    path = os.path.join(HERE, "path_fixtures.npz")
    np.savez_compressed(path, **fx)
    print(path, os.path.getsize(path), "bytes,", len(fx), "arrays")
