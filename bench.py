#!/usr/bin/env python3
"""Benchmark of the action-expert attention hot path on one MI355X.

One "step" is one denoise step (every expert layer: pre-norm, fused QKV + RoPE +
KV append, masked prefix+suffix attention, Wo + residual, then the Euler update)
over one batch of synthetic observations whose prefix KV is already resident in
HBM; for the BitVLA workload a step is one appended action token through every
layer.  Launched through the model-level C ABI (vla_denoise_steps_async).

Timed region: exactly K steps on one stream, bracketed by device synchronisation, in
steady state -- before it, three whole chunks always run (the first eagerly, the second
is captured into a HIP graph, the third replays it) and then the W warm-up steps.

Per-kernel figures are measured live, in the step's own sequence: after the timed region
one more chunk runs with a HIP event recorded after every launch on the launch stream
(vla_profile_begin / vla_profile_end), so a kernel's time is taken with the caches as
its predecessors left them and includes the gap to the launch before it.  The events'
own cost (the marked chunk minus a replayed one, per mark) is subtracted.

Prints ONE JSON line (a few KB) with the contract fields plus
  roofline      the kernel the path's HBM target is set on: the attention launch that reads the
                most prefix K/V at this workload (algorithmic K/V bytes / its duration in the step)
  roofline_dominant  the launch site with the largest share of the step's time, when that is
                another kernel (share_of_step says how much), on its own roofline
  roofline_ternary_prefill  the BitVLA prefill QKV GEMM (int8 MFMA roofline)
  cpu_baseline  the CPU oracle (restated reference op sequence, with the reference's
                per-step concat copies, fp32 SIMD-style accumulation) timed on this host
                with the reference's thread rule and timing recipe
  us_per_action_chunk_with_prefix  one chunk plus the once-per-observation prefix K/V build
  config.workloads  one compact entry per BASELINE configuration and batch size: us per
                step, chunk p50, chunk with the prefix build, launches per step, the roofline
                of the launch with the largest share {kernel, frac, avg_us, traffic} and, when
                that is not it, of the largest prefix-K/V read (roofline_kv)
--verbose adds the per-launch-site tables (kernels, prefill_kernels, other_configs).
"""
import argparse
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3, "i8": 5000.0}


def workloads():
    from vla_cpp_amd import checkpoint as ck
    return {
        "cfg0_smolvla_1layer_f32_b1": dict(cfg=ck.smolvla_config(1, "f32", 0), B=1, views=3),
        "cfg1_smolvla_16layer_bf16_b1": dict(cfg=ck.smolvla_config(16, "bf16", 0), B=1, views=3),
        "cfg1_smolvla_16layer_bf16_b32": dict(cfg=ck.smolvla_config(16, "bf16", 0), B=32, views=3),
        "cfg2_pi0_18layer_bf16_b1": dict(cfg=ck.pi0_config(18), B=1, views=3),
        "cfg2_pi0_18layer_bf16_b16": dict(cfg=ck.pi0_config(18), B=16, views=3),
        "cfg3_gr00t_16dit_bf16_b1": dict(cfg=ck.gr00t_config(16), B=1, views=2),
        "cfg3_gr00t_16dit_bf16_b64": dict(cfg=ck.gr00t_config(16), B=64, views=2),
        # beyond the BASELINE configurations: the same stacks with the FFN half of every layer
        "whole_smolvla_16layer_bf16_b32": dict(cfg=dict(ck.smolvla_config(16, "bf16", 0), ffn_dim=2048), B=32, views=3),
        "whole_smolvla_16layer_bf16_b1": dict(cfg=dict(ck.smolvla_config(16, "bf16", 0), ffn_dim=2048), B=1, views=3),
        "whole_pi0_18layer_bf16_b16": dict(cfg=dict(ck.pi0_config(18), ffn_dim=4096), B=16, views=3),
        "whole_pi05_18layer_bf16_b16": dict(cfg=dict(ck.pi05_config(18), ffn_dim=4096), B=16, views=3),
        "whole_gr00t_16dit_bf16_b64": dict(cfg=dict(ck.gr00t_config(16), ffn_dim=6144), B=64, views=2),
        "whole_gr00t_n1d6_32dit_bf16_b64": dict(cfg=dict(ck.gr00t_n1d6_config(32), ffn_dim=6144), B=64, views=2),
        "cfg4_bitvla_30layer_b1": dict(cfg=ck.bitvla_config(30), B=1, views=1),
        "cfg4_bitvla_30layer_b8": dict(cfg=ck.bitvla_config(30), B=8, views=1),
        "whole_bitvla_30layer_b8": dict(cfg=dict(ck.bitvla_config(30), ffn_dim=6912), B=8, views=1),
    }


def make_obs(cfg, r, views):
    A = cfg["max_action_dim"]
    n_act = cfg["n_suffix"] - (0 if cfg["arch"] in ("smolvla", "bitvla", "pi05") else 1)
    img = r.standard_normal((views * cfg["n_img"], cfg["hidden"])).astype(np.float32)
    if cfg["arch"] == "smolvla":
        img /= np.sqrt(cfg["hidden"])
    obs = dict(img_emb=img, n_views=views, noise=r.standard_normal((n_act, A)).astype(np.float32))
    if cfg.get("vocab", 0) > 0:
        obs["lang"] = r.integers(0, cfg["vocab"], cfg["n_lang"]).astype(np.int32)
    if cfg.get("max_state_dim", 0) > 0:
        obs["state"] = r.standard_normal(cfg["max_state_dim"]).astype(np.float32)
    return obs


def plain_pack(t):
    """int8 ternary [N,K] -> gfx950 packed words (bytes) with the library's host packer."""
    import __graft_entry__ as entry
    lib = entry.load_package().lib()
    t = np.ascontiguousarray(t, np.int8)
    out = np.empty(lib.vla_ternary_packed_words(t.shape[0], t.shape[1]), np.uint32)
    rc = lib.vla_ternary_pack_host(t.ctypes.data, t.shape[0], t.shape[1], out.ctypes.data)
    assert rc == 0
    return out.view(np.uint8).reshape(-1)


def cpu_threads():
    """The reference's rule (src/arch.h:43-53): VLA_N_THREADS if set, else min(hardware threads, 16)."""
    e = os.environ.get("VLA_N_THREADS")
    if e and e.isdigit() and 0 < int(e) <= 1024:
        return int(e)
    return min(os.cpu_count() or 4, 16)


def time_events(fn, iters, warm=3):
    """Average device microseconds of one fn() call.  fn(i) launches on the current
    torch stream; `iters` calls are captured into one HIP graph and the graph is
    replayed between two events, so host launch overhead is not in the figure."""
    import torch
    # warm up on the stream the capture will use: the library keeps its scratch per (device,
    # stream) and may not allocate while a stream is being captured
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(warm):
            fn(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        for i in range(iters):
            fn(i)
    g.replay()
    torch.cuda.synchronize()
    reps = 5
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1000.0 / (iters * reps)


def kernel_breakdown(pkg, cfg, B, P):
    """(--isolated) Times every kernel of one step in isolation at the workload's shapes.
    Returns {name: dict(us, per_step, bound, work)} with work = algorithmic bytes
    (bound hbm) or flops (bound mfma) per launch."""
    import torch
    arch = cfg["arch"]
    dev = "cuda"
    bf = cfg["dtype"] == "bf16"
    dt = pkg.VLA_DT_BF16 if bf else pkg.VLA_DT_F32
    es = 2 if bf else 4
    tdt = torch.int16 if bf else torch.float32
    Hq, Hkv, D, L = cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["n_layers"]
    z = lambda *shape, dtype=tdt: torch.zeros(shape, dtype=dtype, device=dev)
    rnd = lambda *shape: (torch.randn(shape, device=dev).to(torch.bfloat16).view(torch.int16) if bf
                          else torch.randn(shape, device=dev))
    out = {}
    mfma = "bf16" if bf else "f32"

    def add(name, fn, per_step, bound, work, iters=32):
        out[name] = dict(us=time_events(fn, iters), per_step=per_step, bound=bound, work=work,
                         peak_key=("hbm" if bound == "hbm" else mfma))

    def kv_set(n, *shape):
        """n distinct caches (as the layers of the model are), so that consecutive
        launches do not re-read the same bytes out of the on-die caches."""
        return [rnd(*shape) for _ in range(n)]

    n_rot = max(2, min(L, 16))

    if arch == "bitvla":
        H, S = cfg["hidden"], 1
        M = B
        kvd = Hkv * D
        N = H + 2 * kvd
        t_max = (P + cfg["n_suffix"] + 63) // 64 * 64
        T = P + cfg["n_suffix"]
        h, hn = rnd(M, H), z(M, H)
        w1 = rnd(H)
        q8, s, rs = z(M, H, dtype=torch.int8), torch.ones(M, device=dev), z(M, dtype=torch.int32)
        wq = torch.randint(0, 2 ** 31 - 1, (N, H // 16), dtype=torch.int32, device=dev)
        wo = torch.randint(0, 2 ** 31 - 1, (H, H // 16), dtype=torch.int32, device=dev)
        ws = torch.full((6,), 0.016, device=dev)
        qkv, q, att = rnd(M, N), z(M, H), z(M, H)
        kcs, vcs = kv_set(n_rot, B, Hkv, t_max, D), kv_set(n_rot, B, Hkv, D, t_max)
        kc, vc = kcs[0], vcs[0]
        cos, sin = torch.ones(T, D // 2, device=dev), torch.zeros(T, D // 2, device=dev)
        scale = 1.0 / np.sqrt(D)
        # up to 8 rows the engine runs norm + quantisation inside the projection's launch; the
        # separate launches are then timed for comparison only (count 0)
        fused = M <= 8
        add("rmsnorm_act_quant", lambda i: pkg.call("vla_rmsnorm_act_quant_bf16", h, w1, q8, s, rs, 1e-5, M, H),
            0 if fused else 2 * L, "hbm", M * H * 3)
        add("ternary_qkv_gemv", lambda i: pkg.call("vla_ternary_gemm", q8, wq, qkv, None, s, rs, ws, 6, M, N, H),
            0 if fused else L, "hbm", N * H // 4 + M * H + 2 * M * N)
        if fused:
            add("norm_quant_ternary_qkv_gemv_rope_append",
                lambda i: pkg.call("vla_rmsnorm_ternary_gemv_rope_append", h, w1, 1e-5, wq, ws, 6, cos, sin, q, kc, vc, M, Hq, Hkv,
                                   D, H, t_max, P), L, "hbm", N * H // 4 + 2 * M * H + 2 * M * N)
            add("norm_quant_ternary_o_gemv_add", lambda i: pkg.call("vla_rmsnorm_ternary_gemv", att, w1, 1e-5, wo, h, h, ws, 1,
                                                                    M, H, H), L, "hbm", H * H // 4 + 2 * M * H + 4 * M * H)
        add("qkv_split_rope_append", lambda i: pkg.call("vla_qkv_split_rope_append", qkv, cos, sin, q, kc, vc, dt, M, 1, Hq,
                                                       Hkv, D, t_max, P), 0 if fused else L, "hbm", 2 * M * N * 2)
        add("attention_decode", lambda i: pkg.call("vla_attn_prefix_suffix", q, kcs[i % n_rot], vcs[i % n_rot], att,
                                                 pkg.VLA_DT_BF16_P2, B, 1, Hq, Hkv, D, t_max, T, scale, 0, T, 0, 0, None),
            L, "hbm", 2 * T * kvd * es * B)
        add("ternary_o_gemv_add", lambda i: pkg.call("vla_ternary_gemm_add", q8, wo, h, h, s, rs, ws, 1, M, H, H),
            0 if fused else L, "hbm", H * H // 4 + M * H + 4 * M * H)
        add("final_rms_norm", lambda i: pkg.call("bitvla_rmsnorm_bf16", h, w1, hn, 1e-5, M, H), 1, "hbm", 2 * M * H * 2)
        F = cfg.get("ffn_dim", 0)
        if F > 0:  # the squared-ReLU GLU half of every layer
            wgu = torch.randint(0, 2 ** 31 - 1, (2 * F, H // 16), dtype=torch.int32, device=dev)
            wd = torch.randint(0, 2 ** 31 - 1, (H, F // 16), dtype=torch.int32, device=dev)
            gu, actv, wf = rnd(M, 2 * F), rnd(M, F), rnd(F)
            q8f = z(M, F, dtype=torch.int8)
            if fused:
                add("norm_quant_ternary_gate_up_gemv", lambda i: pkg.call("vla_rmsnorm_ternary_gemv", h, w1, 1e-5, wgu, gu, None, ws, 2,
                                                                          M, 2 * F, H), L, "hbm", 2 * F * H // 4 + 2 * M * H + 4 * M * F)
            else:
                add("ternary_gate_up_gemm", lambda i: pkg.call("vla_ternary_gemm", q8, wgu, gu, None, s, rs, ws, 2, M, 2 * F, H), L,
                    "hbm", 2 * F * H // 4 + M * H + 4 * M * F)
            one = fused and F <= 4096  # activation, sub-norm, quantisation and down projection in one launch
            add("sqrelu_norm_quant_ternary_down_gemv_add",
                lambda i: pkg.call("vla_sqrelu_rmsnorm_ternary_gemv", gu, wf, 1e-5, wd, h, h, ws, 1, M, H, F), L if one else 0, "hbm",
                H * F // 4 + 4 * M * F + 4 * M * H)
            add("sqrelu_norm_act_quant", lambda i: pkg.call("vla_sqrelu_rmsnorm_act_quant_bf16", gu, wf, q8f, s, rs, 1e-5, M, F),
                0 if one else L, "hbm", 5 * M * F)
            add("sqrelu_mul", lambda i: pkg.call("gate_up_fused_sqrelu_mul_bf16", gu, actv, M, F), 0, "hbm", 6 * M * F)
            add("ffn_subnorm_act_quant", lambda i: pkg.call("vla_rmsnorm_act_quant_bf16", actv, wf, q8f, s, rs, 1e-5, M, F),
                0, "hbm", 3 * M * F)
            add("ternary_down_gemv_add", lambda i: pkg.call("vla_ternary_gemm_add", q8f, wd, h, h, s, rs, ws, 1, M, H, F),
                0 if one else L, "hbm", H * F // 4 + M * F + 4 * M * H)
        # the prefill-shaped fused QKV GEMM (one launch per layer per observation batch)
        Mp = B * P
        q8p, sp, rsp = z(Mp, H, dtype=torch.int8), torch.ones(Mp, device=dev), z(Mp, dtype=torch.int32)
        qkvp = z(Mp, N)
        add("ternary_qkv_gemm_prefill", lambda i: pkg.call("vla_ternary_gemm", q8p, wq, qkvp, None, sp, rsp, ws, 6, Mp, N, H),
            0, "mfma", 2.0 * Mp * N * H, iters=8)
        out["ternary_qkv_gemm_prefill"]["peak_key"] = "i8"
        return out

    W, S = cfg["expert_h"], cfg["n_suffix"]
    M = B * S
    qd, kvd = Hq * D, Hkv * D
    gr00t = arch in ("gr00t_n1d5", "gr00t_n1d6")
    self_layers = [l for l in range(L) if (True if arch in ("pi0", "pi05") else (l % 2 == 0 if arch == "smolvla" else l % 2 == 1))]
    n_self, n_cross = len(self_layers), L - len(self_layers)
    P_self = 0 if gr00t else P
    T_self = P_self + S
    t_self, t_cross = (T_self + 63) // 64 * 64, (P + 63) // 64 * 64
    h, hn = rnd(M, W), z(M, W)
    q, att = z(M, qd), rnd(M, qd)
    lnw = rnd(W)
    scv = torch.zeros(W, device=dev)
    Wqkv, Wq, Wo = rnd(qd + 2 * kvd, W), rnd(qd, W), rnd(W, qd)
    kcs_s, vcs_s = kv_set(n_rot, B, Hkv, t_self, D), kv_set(n_rot, B, Hkv, D, t_self)
    kc_s, vc_s = kcs_s[0], vcs_s[0]
    cos, sin = torch.ones(S, D // 2, device=dev), torch.zeros(S, D // 2, device=dev)
    rope = None if gr00t else cos
    scale = 1.0 / np.sqrt(D)
    A = cfg["max_action_dim"]
    pi05 = arch == "pi05"
    n_lead = 0 if arch in ("smolvla", "pi05") else 1
    xt = torch.zeros(B, S - n_lead, A, device=dev)
    W_in, b_in = torch.randn(W, A, device=dev), torch.zeros(W, device=dev)
    lead = torch.zeros(B, max(n_lead, 1), W, device=dev)
    W_out, b_out = torch.randn(A, W, device=dev) * 0.01, torch.zeros(A, device=dev)
    mask_kind = cfg["suffix_mask"]
    add("embed_suffix", lambda i: pkg.call("vla_embed_suffix", xt, W_in, b_in, lead if n_lead else None, h, dt, B, S, n_lead, A, W),
        1, "hbm", M * W * es)
    # bf16 RMS archs: the layer's pre-norm runs inside the projection launch (as the host
    # layer does); only the final norm is a launch of its own
    fused_norm = bf and not gr00t and not pi05 and W % 16 == 0
    if pi05:  # adaRMS before the projections, before the FFN and before the Euler step
        add("adarms", lambda i: pkg.call("vla_adarms", h, scv, scv, hn, dt, M, W, 1e-6), L + 1, "hbm", 2 * M * W * es)
    elif gr00t:
        add("adaln", lambda i: pkg.call("vla_adaln", h, scv, scv, hn, dt, M, W, 1e-5), L + 1, "hbm", 2 * M * W * es)
    else:
        add("rms_norm", lambda i: pkg.call("vla_rms_norm", h, lnw, hn, dt, M, W, 1e-5), 1 if fused_norm else L + 1, "hbm",
            2 * M * W * es)

    def proj(Wmat, has_kv, kc, vc, t_max, tok):
        if fused_norm:
            return lambda i: pkg.call("vla_rmsnorm_attn_qkv_rope", h, Wmat, None, dt, M, W, S, Hq, Hkv, has_kv, has_kv, D, rope,
                                      sin, q, kc, vc, t_max, tok, 1e-5)
        return lambda i: pkg.call("vla_attn_qkv_rope", hn, Wmat, None, dt, M, W, S, Hq, Hkv, has_kv, has_kv, D, rope,
                                  None if gr00t else sin, q, kc, vc, t_max, tok)

    if n_self:
        add("qkv_rope_append_self", proj(Wqkv, 1, kc_s, vc_s, t_self, P_self), n_self, "mfma", 2.0 * M * (qd + 2 * kvd) * W)
        add("attention_self", lambda i: pkg.call("vla_attn_prefix_suffix", q, kcs_s[i % n_rot], vcs_s[i % n_rot], att, dt, B, S, Hq, Hkv, D, t_self,
                                               T_self, scale, mask_kind, P_self, 0, 0, None),
            n_self, "hbm", 2 * T_self * kvd * es * B)
    if n_cross:
        kcs_c, vcs_c = kv_set(n_rot, B, Hkv, t_cross, D), kv_set(n_rot, B, Hkv, D, t_cross)
        kc_c, vc_c = kcs_c[0], vcs_c[0]
        add("q_rope_cross", proj(Wq, 0, kc_c, vc_c, t_cross, 0), n_cross, "mfma", 2.0 * M * qd * W)
        # N1.6 / N1.7: every attend_text_every_n-th cross layer reads the (short) text K/V instead
        n_txt = len([l for l in range(L) if l not in self_layers and l % (2 * cfg["attend_text_every_n"]) == 0]) \
            if arch == "gr00t_n1d6" else 0
        add("attention_cross", lambda i: pkg.call("vla_attn_prefix_suffix", q, kcs_c[i % n_rot], vcs_c[i % n_rot], att, dt, B, S, Hq, Hkv, D, t_cross,
                                                P, scale, 0, P, 0, 0, None),
            n_cross - n_txt, "hbm", 2 * P * kvd * es * B)
        if n_txt:
            Pt = cfg["n_lang"]
            add("attention_cross_text", lambda i: pkg.call("vla_attn_prefix_suffix", q, kcs_c[i % n_rot], vcs_c[i % n_rot], att, dt, B, S, Hq,
                                                         Hkv, D, t_cross, Pt, scale, 0, Pt, 0, 0, None),
                n_txt, "hbm", 2 * Pt * kvd * es * B)
    if pi05:
        gatev = torch.ones(W, device=dev)
        add("wo_gated_residual", lambda i: pkg.call("vla_linear_gated", att, Wo, None, gatev, h, h, dt, dt, M, W, qd), L, "mfma",
            2.0 * M * W * qd)
    else:
        add("wo_residual", lambda i: pkg.call("vla_linear", att, Wo, None, h, h, dt, dt, M, W, qd), L, "mfma", 2.0 * M * W * qd)
    I = cfg.get("ffn_dim", 0)
    if I > 0:  # the FFN half of every layer (workloads beyond the BASELINE configurations)
        mid = z(M, I)
        if gr00t:
            W1, W2, b1, b2 = rnd(I, W), rnd(W, I), torch.zeros(I, device=dev), torch.zeros(W, device=dev)
            out["adaln"]["per_step"] += L
            add("ffn_in_gelu", lambda i: pkg.call("vla_linear_act", hn, W1, b1, None, mid, dt, dt, M, I, W, pkg.VLA_ACT_GELU), L,
                "mfma", 2.0 * M * I * W)
            add("ffn_out_residual", lambda i: pkg.call("vla_linear", mid, W2, b2, h, h, dt, dt, M, W, I), L, "mfma", 2.0 * M * I * W)
        else:
            Wgu, Wd = rnd(2 * I, W), rnd(W, I)
            act = pkg.VLA_ACT_SILU if arch == "smolvla" else pkg.VLA_ACT_GELU
            if not fused_norm:
                out["adarms" if pi05 else "rms_norm"]["per_step"] += L
            add("ffn_gate_up", lambda i: pkg.call("vla_glu_linear", h if fused_norm else hn, Wgu, None, mid, dt, dt, M, I, W, act,
                                                  1e-5 if fused_norm else -1.0), L, "mfma", 4.0 * M * I * W)
            if pi05:
                add("ffn_down_gated_residual", lambda i: pkg.call("vla_linear_gated", mid, Wd, None, gatev, h, h, dt, dt, M, W, I), L,
                    "mfma", 2.0 * M * I * W)
            else:
                add("ffn_down_residual", lambda i: pkg.call("vla_linear", mid, Wd, None, h, h, dt, dt, M, W, I), L, "mfma",
                    2.0 * M * I * W)
    add("euler_step", lambda i: pkg.call("vla_euler_step", xt, hn, W_out, b_out, dt, B, S, n_lead, A, W, -0.1), 1, "hbm",
        M * W * es)
    return out


# HBM-side bytes per launch (L2 misses) measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on
# this command, each scaled by what the same counter reads for a plain 256 MiB device copy.
# Counters cannot be read from inside the process: the figures are those of the committed
# profile summaries, kept beside them as profiles/hbm_traffic.json (written by the same pass
# that writes the summaries); launch sites without a measurement report null.
def measured_traffic():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        return {}
    return {(w, k): int(v["bytes"]) for w, sites in doc.get("workloads", {}).items() for k, v in sites.items()}


MEASURED_TRAFFIC_BYTES = measured_traffic()


def prefix_tokens(cfg, views):
    if cfg["arch"] == "smolvla":
        return views * cfg["n_img"] + cfg["n_lang"] + 1
    if cfg["arch"] in ("pi0", "pi05"):
        return views * cfg["n_img"] + cfg["n_lang"]
    if cfg["arch"] == "bitvla":
        return cfg["n_img"] + cfg["n_lang"]
    return views * cfg["n_img"]


def algorithmic_work(cfg, B, P):
    """{launch-site label: (bound, algorithmic bytes or flops per launch, peak key)}: the per-unit
    figures of the path (K/V read once per launch, 2 M N K per projection) at this workload."""
    arch = cfg["arch"]
    bf = cfg["dtype"] == "bf16"
    es = 2 if bf else 4
    mf = "bf16" if bf else "f32"
    Hq, Hkv, D = cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd = Hq * D, Hkv * D
    w = {}
    if arch == "bitvla":
        H, n_act, F = cfg["hidden"], cfg["n_suffix"], cfg.get("ffn_dim", 0)
        N, M, Mp = H + 2 * kvd, B, B * P
        T = P + (n_act + 1) / 2.0  # keys seen by an appended token, averaged over the chunk
        w["step.token_embedding"] = ("hbm", 2 * M * H * 2, "hbm")
        w["step.norm_quant_qkv_gemv_rope_append"] = ("hbm", N * H // 4 + 2 * M * H + 2 * M * N, "hbm")
        w["step.attention"] = ("hbm", 2 * T * kvd * 2 * B, "hbm")
        w["step.norm_quant_o_gemv_add"] = ("hbm", H * H // 4 + 2 * M * H + 4 * M * H, "hbm")
        w["step.final_norm"] = ("hbm", 2 * M * H * 2, "hbm")
        w["step.action_head"] = ("hbm", n_act * M * H * 2, "hbm")
        w["prefill.norm_quant"] = ("hbm", 3 * Mp * H, "hbm")
        w["prefill.ternary_qkv_gemm"] = ("mfma", 2.0 * Mp * N * H, "i8")
        w["prefill.qkv_split_rope_append"] = ("hbm", 2 * Mp * N * 2, "hbm")
        w["prefill.attention"] = ("mfma", 4.0 * Hq * P * P * D * B, "bf16")
        w["prefill.ternary_o_gemm_add"] = ("mfma", 2.0 * Mp * H * H, "i8")
        if F:
            w["step.norm_quant_gate_up_gemv"] = ("hbm", 2 * F * H // 4 + 2 * M * H + 4 * M * F, "hbm")
            w["step.sqrelu_norm_quant_down_gemv_add"] = ("hbm", H * F // 4 + 4 * M * F + 4 * M * H, "hbm")
            w["step.sqrelu_norm_quant"] = ("hbm", 5 * M * F, "hbm")
            w["step.ternary_down_gemm_add"] = ("hbm", H * F // 4 + M * F + 4 * M * H, "hbm")
            w["prefill.ternary_gate_up_gemm"] = ("mfma", 4.0 * Mp * F * H, "i8")
            w["prefill.sqrelu_norm_quant"] = ("hbm", 5 * Mp * F, "hbm")
            w["prefill.ternary_down_gemm_add"] = ("mfma", 2.0 * Mp * H * F, "i8")
        return w
    W, Wv, S, A, I = cfg["expert_h"], cfg["hidden"], cfg["n_suffix"], cfg["max_action_dim"], cfg.get("ffn_dim", 0)
    M = B * S
    gr00t = arch in ("gr00t_n1d5", "gr00t_n1d6")
    P_self = 0 if gr00t else P
    n_lead = 0 if arch in ("smolvla", "pi05") else 1
    w["step.stage_noise"] = ("hbm", 2 * B * (S - n_lead) * A * 4, "hbm")
    w["step.embed_suffix"] = ("hbm", M * W * es, "hbm")
    for k in ("step.pre_norm", "step.final_norm", "step.ffn_norm"):
        w[k] = ("hbm", 2 * M * W * es, "hbm")
    w["step.qkv_rope_append_self"] = ("mfma", 2.0 * M * (qd + 2 * kvd) * W, mf)
    # a DiT self block's norm, projections and attention over its own S tokens in one launch
    w["step.norm_qkv_attention_self"] = ("mfma", 2.0 * M * (qd + 2 * kvd) * W + 4.0 * B * Hq * S * S * D, mf)
    w["step.q_rope_cross"] = ("mfma", 2.0 * M * qd * W, mf)
    w["step.attention_self"] = ("hbm", 2 * (P_self + S) * kvd * es * B, "hbm")
    w["step.attention_cross"] = ("hbm", 2 * P * kvd * es * B, "hbm")
    if arch == "gr00t_n1d6":
        w["step.attention_cross_text"] = ("hbm", 2 * cfg["n_lang"] * kvd * es * B, "hbm")
        w["step.attention_cross"] = ("hbm", 2 * (P - 0) * kvd * es * B, "hbm")
    w["step.wo_residual"] = ("mfma", 2.0 * M * W * qd, mf)
    w["step.ffn_gate_up"] = ("mfma", 4.0 * M * I * W, mf)
    w["step.ffn_down_residual"] = ("mfma", 2.0 * M * I * W, mf)
    w["step.ffn_gate_up_down"] = ("mfma", 6.0 * M * I * W, mf)
    w["step.ffn_in_out"] = ("mfma", 4.0 * M * I * W, mf)
    w["step.euler_step"] = ("hbm", M * W * es, "hbm")
    w["step.final_norm_euler_step"] = ("hbm", M * W * es, "hbm")
    w["prefill.prefix_norm"] = ("hbm", 2 * B * P * Wv * es, "hbm")
    w["prefill.prefix_kv_proj"] = ("mfma", 2.0 * B * P * 2 * kvd * Wv, mf)
    w["prefill.prefix_kv_proj_and_cross_reprojection"] = ("mfma", 2.0 * B * P * 2 * kvd * (Wv + kvd), mf)
    return w


def roofline_entry(label, us, work, workload=None):
    bound, amount, peak_key = work
    if bound == "hbm":
        achieved = amount / (us * 1e-6) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = amount / (us * 1e-6) / 1e12
        peak, unit = PEAK_TFLOPS[peak_key], "TFLOP/s" if peak_key != "i8" else "TOP/s"
    return dict(kernel=label, bound=bound, achieved=round(achieved, 3), peak=peak, unit=unit,
                frac=round(achieved / peak, 5), traffic=MEASURED_TRAFFIC_BYTES.get((workload, label)),
                avg_us=round(us, 3), algorithmic_work_per_launch=amount,
                timing="HIP events on the launch stream, in the step's own sequence, less the events' own cost")


def pct(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(round(q * (len(xs) - 1))))]


def cpu_baseline(cfg, w, obs, B):
    """The CPU oracle on a bounded sample: one observation, denoise steps only (the prefix K/V
    build is excluded, as on the GPU side), timed with the reference's recipe -- warm-ups, then
    repetitions, min / p50 / p90 (src/serving/vla-bench.cpp:159-195) -- on the reference's thread
    count (src/arch.h:43-53).  The per-step figure is scaled by the batch: observations are
    independent and the reference serves one at a time (src/serving/server.cpp:340-558)."""
    import oracle as orc
    from oracle import chunk as oc
    threads = cpu_threads()
    orc.set_num_threads(threads)
    orc.set_default_accumulation(False)  # fp32 accumulation with SIMD-style partial sums, not the parity oracle's double
    try:
        if cfg["arch"] == "bitvla":
            small = dict(cfg, n_layers=2)
            run = lambda: oc.bitvla_chunk(small, w, obs)
            scale_layers, n_units, what = cfg["n_layers"] / 2.0, cfg["n_suffix"], "appended token"
            budget = 12.0
            t0 = time.perf_counter()
            run()
            first = time.perf_counter() - t0
            reps = int(max(3, min(20, budget / max(first, 1e-3))))
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                run()
                ts.append(time.perf_counter() - t0)
            per = [t / n_units * scale_layers * 1e6 * B for t in ts]
            sample = ("restated CPU reference (not ggml, whose AVX-512 / AMX kernels would be several times faster): 1 observation, 2 of %d layers, prefix prefill + 7 tokens per run "
                      "(the prefill is included: the restated reference has no cache to skip it with), 1 warm-up + %d "
                      "repetitions, scaled by layers and batch %d" % (cfg["n_layers"], reps, B))
        else:
            n1, n2 = 1, 1 + cfg["num_steps"]
            run = lambda n: oc.flow_expert_chunk(dict(cfg, num_steps=n), w, obs, emulate_bf16=False)
            t0 = time.perf_counter()
            run(n2)
            first = time.perf_counter() - t0
            reps = int(max(3, min(20, 15.0 / max(first * 1.2, 1e-3))))
            for _ in range(2):
                run(n2)
            short, full = [], []
            for _ in range(reps):
                t0 = time.perf_counter()
                run(n1)
                short.append(time.perf_counter() - t0)
                t0 = time.perf_counter()
                run(n2)
                full.append(time.perf_counter() - t0)
            base = pct(short, 0.5)  # prefix build + one step
            per = [(t - base) / (n2 - n1) * 1e6 * B for t in full]
            what = "denoise step"
            sample = ("restated CPU reference (not ggml, whose AVX-512 / AMX kernels would be several times faster): 1 observation, (chunk of %d steps - chunk of 1 step) / %d, 3 warm-ups + "
                      "%d repetitions, scaled by batch %d" % (n2, n2 - n1, reps, B))
    finally:
        orc.set_default_accumulation(True)
    return dict(value=round(pct(per, 0.5), 1), unit="us per %s (batch of %d)" % (what, B), cores=threads, kind="port",
                min=round(min(per), 1), p50=round(pct(per, 0.5), 1), p90=round(pct(per, 0.9), 1), sample=sample)


def run_workload(name, spec, steps, warmup, with_cpu, tmpdir, isolated=False):
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    from vla_cpp_amd import checkpoint as ck
    from vla_cpp_amd import ffi
    cfg, B, views = spec["cfg"], spec["B"], spec["views"]
    w = ck.synth_weights(cfg, seed=0x5EED)
    path = os.path.join(tmpdir, name + ".vlaw")
    ck.write_synthetic(path, cfg, w, plain_pack=plain_pack if cfg["arch"] == "bitvla" else None)
    m = ffi.Model(path)
    r = np.random.default_rng(0x5EED)
    obs = [make_obs(cfg, r, views) for _ in range(B)]
    spc = cfg["n_suffix"] if cfg["arch"] == "bitvla" else cfg["num_steps"]  # steps per chunk
    m.prefill_batch(obs)  # allocates
    m.profile_begin()
    t0 = time.perf_counter()
    m.prefill_batch(obs)
    prefill_ms = (time.perf_counter() - t0) * 1e3
    prof_prefill = m.profile_end()
    stream = torch.cuda.current_stream().cuda_stream
    # steady state first: eager chunk, captured chunk, one replay -- whatever W is
    m.denoise_steps_async(3 * spc, stream)
    if warmup > 0:
        m.denoise_steps_async(warmup, stream)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    m.denoise_steps_async(steps, stream)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    dev_ms = e0.elapsed_time(e1)
    ms_per_step = max(dev_ms, wall_ms) / steps  # the host-inclusive figure when the host is the slower side
    # the reference bench's recipe on the GPU side as well: whole chunks one at a time,
    # 3 warm-ups, 20 repetitions, min / p50 / p90 (src/serving/vla-bench.cpp:159-195)
    reps = []
    for i in range(23):
        c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        c0.record()
        m.denoise_steps_async(spc, stream)
        c1.record()
        torch.cuda.synchronize()
        if i >= 3:
            reps.append(c0.elapsed_time(c1) * 1e3)
    chunk_us = dict(min=round(min(reps), 1), p50=round(pct(reps, 0.5), 1), p90=round(pct(reps, 0.9), 1), warmups=3, repetitions=20)
    # one more chunk with an event after every launch
    m.profile_begin()
    m.denoise_steps_async(spc, stream)
    prof = m.profile_end()
    P = prefix_tokens(cfg, views)
    work = algorithmic_work(cfg, B, P)
    # An event between two launches costs stream time of its own: the marked chunk takes longer
    # than a replayed one.  The difference, spread evenly over the marks, is taken off every
    # launch, so that the per-launch figures add up to the step as it was timed above.
    n_marks = sum(v["launches"] for v in prof.values())
    marked_us = sum(v["us"] * v["launches"] for v in prof.values())
    event_us = max(0.0, (marked_us - dev_ms * 1e3 / steps * spc) / max(n_marks, 1))
    prof = {k: dict(us=max(v["us"] - event_us, 0.05), launches=v["launches"], us_marked=v["us"]) for k, v in prof.items()}
    kernels, best, best_kv, best_t = {}, None, None, 0.0
    for label, v in sorted(prof.items()):
        per_step = v["launches"] / float(spc)
        k = dict(us=round(v["us"], 2), per_step=round(per_step, 3))
        if label in work:
            rf = roofline_entry(label, v["us"], work[label], name)
            k.update(bound=rf["bound"], frac=rf["frac"])
            if v["us"] * per_step > best_t:
                best, best_t = dict(rf, share_of_step=round(v["us"] * per_step / (ms_per_step * 1e3), 3)), v["us"] * per_step
            if label.startswith("step.attention") and (best_kv is None or work[label][1] > best_kv["algorithmic_work_per_launch"]):
                best_kv = rf
        kernels[label] = k
    res = dict(
        workload=name, batch=B, us_per_denoise_step=round(ms_per_step * 1e3, 2),
        us_per_action_chunk=round(ms_per_step * 1e3 * spc, 1), steps_per_chunk=spc, timed_steps=steps,
        action_chunk_us=chunk_us,
        device_us_per_step=round(dev_ms * 1e3 / steps, 2), host_us_per_step=round(wall_ms * 1e3 / steps, 2),
        prefix_kv_build_ms=round(prefill_ms, 2),
        # the reference's chunk is predict() = prefix + steps (src/model.cpp:200-296): the once-per-observation-batch
        # prefix K/V build (host staging, upload and projections, wall clock) plus one chunk (p50)
        us_per_action_chunk_with_prefix=round(prefill_ms * 1e3 + chunk_us["p50"], 1),
        sum_launch_us_per_step=round(sum(v["us"] * v["launches"] for v in prof.values()) / spc, 2),
        event_overhead_us_per_launch=round(event_us, 3),
        launches_per_step=round(sum(v["launches"] for v in prof.values()) / float(spc), 1),
        roofline=best, roofline_kv=best_kv, kernels=kernels,
        prefill_kernels={k: dict(us=round(v["us"], 2), launches=v["launches"]) for k, v in sorted(prof_prefill.items())},
    )
    if "prefill.ternary_qkv_gemm" in prof_prefill:
        res["roofline_ternary_prefill"] = roofline_entry("prefill.ternary_qkv_gemm", prof_prefill["prefill.ternary_qkv_gemm"]["us"],
                                                         work["prefill.ternary_qkv_gemm"], name)
    if isolated:
        kern = kernel_breakdown(pkg, cfg, B, P)
        res["kernels_isolated"] = {k: dict(us=round(v["us"], 2), per_step=v["per_step"]) for k, v in kern.items()}
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(cfg, w, obs[0], B)
    m.close()
    os.remove(path)
    return res, ms_per_step


BASELINE_WORKLOADS = ["cfg0_smolvla_1layer_f32_b1", "cfg1_smolvla_16layer_bf16_b1", "cfg1_smolvla_16layer_bf16_b32",
                      "cfg2_pi0_18layer_bf16_b1", "cfg2_pi0_18layer_bf16_b16", "cfg3_gr00t_16dit_bf16_b1",
                      "cfg3_gr00t_16dit_bf16_b64", "cfg4_bitvla_30layer_b1", "cfg4_bitvla_30layer_b8"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    # the headline workload: the largest single-GPU configuration of the BASELINE set, GR00T
    # N1.5-shape DiT at batch 64 -- the largest prefix-KV read per step (931 MB)
    ap.add_argument("--config", default="cfg3_gr00t_16dit_bf16_b64")
    ap.add_argument("--others", default="baseline",
                    help="'baseline' = every other BASELINE configuration (both batch sizes), 'all' = every workload, "
                         "'none', or a comma-separated list; reported under other_configs")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--isolated", action="store_true", help="also time every kernel alone (replayed, warm caches)")
    ap.add_argument("--verbose", action="store_true",
                    help="add the per-launch-site tables of every workload to the line (the default line keeps one compact entry per workload)")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="only run plain device copies of a known size (reference for the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU (the path shards over observations with no collectives); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if args.traffic_calibration:
        n = 64 << 20  # fp32 elements: each copy reads 256 MiB and writes 256 MiB
        src = torch.ones(n, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "device copy", "copies": 5, "bytes_read_per_copy": 4 * n, "bytes_written_per_copy": 4 * n}))
        return
    import __graft_entry__ as entry
    entry.load_package().lib()
    wl = workloads()
    if args.config not in wl:
        print("unknown --config; choose from: " + ", ".join(wl), file=sys.stderr)
        sys.exit(2)
    if args.others == "baseline":
        names = [n for n in BASELINE_WORKLOADS if n != args.config]
    elif args.others == "all":
        names = [n for n in wl if n != args.config]
    elif args.others == "none":
        names = []
    else:
        names = [n for n in args.others.split(",") if n and n != args.config]
    with tempfile.TemporaryDirectory() as tmp:
        main_res, ms_per_step = run_workload(args.config, wl[args.config], args.steps, args.warmup, not args.no_cpu, tmp,
                                             args.isolated)
        others = []
        for n in names:
            c = wl[n]["cfg"]
            spc = c["n_suffix"] if c["arch"] == "bitvla" else c["num_steps"]
            r, _ = run_workload(n, wl[n], 3 * spc, 0, False, tmp, args.isolated)  # whole chunks: graph replays only
            others.append(r)
    cfg = wl[args.config]["cfg"]

    def compact(r):
        """One short entry per workload: what the step costs and how its dominant launch sits on its roofline."""
        rf = r["roofline"] or {}
        e = {"us_per_denoise_step": r["us_per_denoise_step"], "us_per_action_chunk_p50": r["action_chunk_us"]["p50"],
             "us_per_action_chunk_with_prefix": r["us_per_action_chunk_with_prefix"], "prefix_kv_build_ms": r["prefix_kv_build_ms"],
             "launches_per_step": r["launches_per_step"],
             "roofline": {"kernel": rf.get("kernel"), "bound": rf.get("bound"), "frac": rf.get("frac"), "avg_us": rf.get("avg_us"),
                          "traffic": rf.get("traffic")}}
        kv = r.get("roofline_kv")
        if kv and kv.get("kernel") != rf.get("kernel"):
            e["roofline_kv"] = {"kernel": kv["kernel"], "frac": kv["frac"], "avg_us": kv["avg_us"], "traffic": kv["traffic"]}
        tp = r.get("roofline_ternary_prefill")
        if tp:
            e["roofline_ternary_prefill"] = {"frac": tp["frac"], "avg_us": tp["avg_us"], "traffic": tp["traffic"]}
        return e

    every = [main_res] + others
    line = {
        "metric": "us_per_denoise_step", "value": main_res["us_per_denoise_step"], "unit": "us",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if cfg["dtype"] == "bf16" else "f32", "data": "synthetic",
        "config": {"workload": args.config, "batch": wl[args.config]["B"], "n_layers": cfg["n_layers"],
                   "prefix_tokens_resident": True, "step": "one denoise step over all expert layers",
                   "timed_region": "graph replays in steady state (3 whole chunks + warmup steps run before it)",
                   # every BASELINE workload (both batch sizes), the headline included: us per step, chunk p50 (all steps),
                   # chunk + the once-per-observation prefix K/V build, launches per step, the dominant launch's roofline
                   "workloads": {r["workload"]: compact(r) for r in every}},
        "us_per_action_chunk": main_res["us_per_action_chunk"], "action_chunk_us": main_res["action_chunk_us"],
        "us_per_action_chunk_with_prefix": main_res["us_per_action_chunk_with_prefix"],
        "prefix_kv_build_ms": main_res["prefix_kv_build_ms"],
        # the largest prefix-K/V read (the HBM target's kernel); the launch site with the largest share of the step beside it
        "roofline": main_res["roofline_kv"] or main_res["roofline"],
        "cpu_baseline": main_res.get("cpu_baseline"),
        "device_us_per_step": main_res["device_us_per_step"], "host_us_per_step": main_res["host_us_per_step"],
        "sum_launch_us_per_step": main_res["sum_launch_us_per_step"], "launches_per_step": main_res["launches_per_step"],
        "event_overhead_us_per_launch": main_res["event_overhead_us_per_launch"],
    }
    if main_res["roofline_kv"] and main_res["roofline"] and main_res["roofline"]["kernel"] != main_res["roofline_kv"]["kernel"]:
        line["roofline_dominant"] = {k: main_res["roofline"].get(k) for k in ("kernel", "bound", "achieved", "peak", "unit", "frac", "traffic", "avg_us", "share_of_step")}
    for r in every:  # the ternary prefill GEMM's roofline, whichever workload ran it (the largest batch wins)
        if "roofline_ternary_prefill" in r:
            line["roofline_ternary_prefill"] = dict(r["roofline_ternary_prefill"], workload=r["workload"])
    if args.verbose:
        line["kernels"] = main_res["kernels"]
        line["prefill_kernels"] = main_res["prefill_kernels"]
        line["other_configs"] = others
        if "kernels_isolated" in main_res:
            line["kernels_isolated"] = main_res["kernels_isolated"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
