"""Whole-chunk CPU oracle (TEST INFRASTRUCTURE ONLY): the reference's op sequence
for one observation, composed from the primitives of oracle.cpp.

It keeps what the reference does today, including the per-layer, per-step
ggml_concat(cached_K, k_rope) / ggml_concat(cached_V, v) copies
(src/models/smolvla.cpp:832-833, src/models/pi0.cpp:198-201), so timing it gives
the "restated CPU reference" baseline.

Scope of a layer (the FFN, the VLM backbone between prefix layers and the vision
towers are outside the hot path): pre-norm -> Q/K/V -> RoPE -> concat ->
attention -> Wo + residual.

`emulate_bf16` rounds to bf16 at the points where the GPU path stores bf16
(hidden stream, normalised activations, Q, K, V, attention output); everything
else (scores, softmax, accumulation, RoPE, the Euler state) is fp32/fp64 in both
modes, the reference's precision split (src/act_dtype.h:29-35).
"""
import math

import numpy as np

import oracle as orc


def _rnd(emulate):
    return orc.round_bf16 if emulate else (lambda x: np.asarray(x, np.float32))


def _is_self(cfg, l):
    if cfg["arch"] in ("pi0", "pi05"):
        return True
    if cfg["arch"] == "smolvla":
        return l % cfg["self_attn_every_n"] == 0
    # GR00T DiT: cross on even, self on odd layers (gr00tn1d5.cpp:361-375); N1.6 / N1.7 only
    # when dit_interleave is set (gr00tn1d6.cpp:449, 462)
    return l % 2 == 1 and bool(cfg.get("dit_interleave", 1))


def _split_heads(y, Hq, Hkv, D):
    M = y.shape[0]
    q = y[:, :Hq * D].reshape(M, Hq, D)
    k = y[:, Hq * D:(Hq + Hkv) * D].reshape(M, Hkv, D)
    v = y[:, (Hq + Hkv) * D:].reshape(M, Hkv, D)
    return q, k, v


def flow_expert_chunk(cfg, w, obs, emulate_bf16=False, return_debug=False):
    """SmolVLA / pi0 / pi0.5 / GR00T N1.5 / N1.6 action chunk for one observation.

    obs: img_emb [views*n_img, hidden], n_views, lang (int32 or None), state, noise
    [n_actions, max_action_dim].  Returns [n_actions, max_action_dim] fp32.
    Follows build_compute_graph (src/models/smolvla.cpp:1376-1419), the pi0 main
    graph (src/models/pi0.cpp:559-588) and the GR00T solver loop
    (src/models/gr00tn1d5.cpp:359-381).  pi0.5 is the pi0 schedule with adaRMS norms whose
    (scale, shift, gate) come from the time embedding, gated residuals, no state token
    and no suffix mask (src/models/pi05.cpp:208-283, 610-631).
    """
    arch = cfg["arch"]
    rnd = _rnd(emulate_bf16)
    L, Hq, Hkv, D = cfg["n_layers"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    W, Wv, A, S, steps = cfg["expert_h"], cfg["hidden"], cfg["max_action_dim"], cfg["n_suffix"], cfg["num_steps"]
    kvd = Hkv * D
    eps = cfg["rms_eps"]
    scale = 1.0 / math.sqrt(D)
    views = obs["n_views"]
    n_img_tot = views * cfg["n_img"]
    img = np.asarray(obs["img_emb"], np.float32).reshape(n_img_tot, Wv)
    state = np.zeros(cfg["max_state_dim"], np.float32) if obs.get("state") is None else np.asarray(obs["state"], np.float32)
    gr00t = arch in ("gr00t_n1d5", "gr00t_n1d6")
    alt_vl = arch == "gr00t_n1d6"
    pi05 = arch == "pi05"
    # the DiT head's own MLPs: state + future tokens lead, encode_action / proj_out + decode
    head_io = gr00t and bool(cfg.get("head_io", 0))
    n_lead = 0 if arch in ("smolvla", "pi05") else (1 + cfg["num_future"] if head_io else 1)
    Sa = S - n_lead

    # ---- prefix embeddings, positions, masks
    pad = (0, 0)
    if alt_vl:
        # AlternateVLDiT (gr00tn1d6.cpp:440-467, gr00tn1d7.cpp:559-590): cross layer l attends to
        # the text rows of the backbone features when l % (2 attend_text_every_n) == 0, else to
        # the image rows; without text both are the image rows.  The text rows here are an
        # embedding lookup standing in for the backbone's output at the text positions.
        lang = np.asarray(obs["lang"], np.int32)
        txt = w["prefix.E_lang"][lang] if lang.size else img
        pe = img
        P = n_img_tot
    elif gr00t:
        pe = img
        P = n_img_tot
    else:
        lang = np.asarray(obs["lang"], np.int32)
        n_lang = lang.size
        lscale = np.float32(math.sqrt(Wv))
        if arch == "smolvla":
            Lmax = cfg["n_lang"]
            ids = np.zeros(Lmax, np.int32)
            ids[:n_lang] = lang
            st = orc.linear(state[None, :], w["prefix.Wstate"], w["prefix.bstate"])
            pe = np.concatenate([img * lscale, w["prefix.E_lang"][ids] * lscale, st], 0)
            P = n_img_tot + Lmax + 1
            state_pos = n_img_tot + n_lang
            pad = (n_img_tot + n_lang, n_img_tot + Lmax)
            _, pos_prefill = orc.mask_smolvla_prefill(P, pad[0], pad[1], state_pos)
            pos_self = state_pos + 1 + np.arange(S, dtype=np.int32)
        else:
            pe = np.concatenate([img, w["prefix.E_lang"][lang] * lscale], 0)
            P = n_img_tot + n_lang
            pos_prefill = np.arange(P, dtype=np.int32)
            pos_self = P + np.arange(S, dtype=np.int32)
        pos_cross = np.arange(S, dtype=np.int32)
        base = cfg["rope_freq_base"]
        cp, sp = orc.rope_tables(pos_prefill, D, base)
        cs, ss = orc.rope_tables(pos_self, D, base)
        cc, sc_ = orc.rope_tables(pos_cross, D, base)
    pe = rnd(pe)
    if alt_vl:
        txt = rnd(txt)
    if gr00t and "prefix.vlln_w" in w:
        # vlln, the affine LayerNorm between the backbone and the head (gr00tn1d6.cpp:436,
        # gr00tn1d7.cpp:556): the rows then stand for the backbone's last hidden states
        veps = cfg.get("vlln_eps", 1e-5)
        text_is_image = alt_vl and txt is pe
        pe = rnd(orc.layer_norm(pe, w["prefix.vlln_w"], w["prefix.vlln_b"], veps))
        if alt_vl:
            txt = pe if text_is_image else rnd(orc.layer_norm(txt, w["prefix.vlln_w"], w["prefix.vlln_b"], veps))

    if cfg["suffix_mask"] == 1:
        mask_self = orc.mask_smolvla_full(P, S, pad[0], pad[1])
    elif cfg["suffix_mask"] == 2:
        mask_self = orc.mask_pi0_full(P, S)
    else:
        mask_self = np.zeros((S, P + S), np.float32)
        mask_self[:, pad[0]:pad[1]] = -np.inf
    mask_cross = orc.mask_smolvla_prefix_only(P, S, pad[0], pad[1])

    # ---- prefix K/V per layer, once per observation
    cacheK, cacheV = [None] * L, [None] * L
    for l in range(L):
        self_l = _is_self(cfg, l)
        if gr00t:
            if self_l:
                continue
            src = txt if (alt_vl and l % (2 * cfg["attend_text_every_n"]) == 0) else pe
            kv = orc.linear(src, w["vlm.%d.Wkv" % l], w["vlm.%d.bkv" % l])
            cacheK[l] = rnd(kv[:, :kvd]).reshape(src.shape[0], Hkv, D)
            cacheV[l] = rnd(kv[:, kvd:]).reshape(src.shape[0], Hkv, D)
            continue
        xn = rnd(orc.rms_norm(pe, w["vlm.%d.ln" % l], eps))
        kv = orc.linear(xn, w["vlm.%d.Wkv" % l])
        k = rnd(orc.rope_neox(kv[:, :kvd].reshape(P, Hkv, D), cp, sp))
        v = rnd(kv[:, kvd:]).reshape(P, Hkv, D)
        if arch == "smolvla" and not self_l:
            # expert_cross_kv (smolvla.cpp:853-860): re-project the cached, already rotated K and V
            k = rnd(orc.linear(k.reshape(P, kvd), w["ex.%d.Wk_x" % l])).reshape(P, Hkv, D)
            v = rnd(orc.linear(v.reshape(P, kvd), w["ex.%d.Wv_x" % l])).reshape(P, Hkv, D)
        cacheK[l], cacheV[l] = k, v

    # ---- per-step constants
    dt = (1.0 if gr00t else -1.0) / steps
    dt32 = np.float32(dt)
    if gr00t:
        ada, po_mod = [], []
        n_buckets = cfg.get("num_buckets", 1000)
        for s in range(steps):
            tp = orc.timesteps_proj(int(s / steps * n_buckets))
            t1 = orc.silu(orc.linear(tp[None, :], w["te.l1W"], w["te.l1b"]))
            temb = orc.linear(t1, w["te.l2W"], w["te.l2b"])
            st = orc.silu(temb)
            ada.append([orc.linear(st, w["ex.%d.adaln_w" % l], w["ex.%d.adaln_b" % l])[0] for l in range(L)])
            if head_io:  # DitHead::proj_out's dense: (shift, scale), dit_head.cpp:140-142
                po_mod.append(orc.linear(st, w["aex.po1W"], w["aex.po1b"])[0])
    lead = None
    if head_io:
        # ActionExpert::encode_state (action_expert.cpp:41-44), then the learned future tokens (gr00tn1d5.cpp:371)
        se = np.maximum(orc.linear(state[None, :], w["aex.se_l1W"], w["aex.se_l1b"]), 0)
        lead = orc.linear(se, w["aex.se_l2W"], w["aex.se_l2b"])
        if cfg["num_future"] > 0:  # none in N1.6 / N1.7: hh = [state; actions] (gr00tn1d6.cpp:457)
            lead = np.concatenate([lead, w["aex.future_tokens"]], 0)
    elif n_lead:
        lead = orc.linear(state[None, :], w["act.W_sp"], w["act.b_sp"])

    x = np.asarray(obs["noise"], np.float32).reshape(Sa, A).copy()
    debug = {}
    for s in range(steps):
        bias = None if head_io else w["act.b_in"].copy()
        if pi05:
            # the time only conditions the norms (pi05.cpp:619-622)
            t = np.float32(1.0) + np.float32(s) * dt32
            temb = orc.sinusoidal_time_emb(float(t), W, cfg["min_period"], cfg["max_period"])
            c1 = orc.silu(orc.linear(temb[None, :], w["te.W_tin"], w["te.b_tin"]))
            cond = orc.silu(orc.linear(c1, w["te.W_tout"], w["te.b_tout"]))

            def adarms(x_, name):  # build_adarms, pi05.cpp:208-224
                mod = orc.linear(cond, w[name + "_w"], w[name + "_b"])[0]
                return orc.adarms(x_, mod[:W], mod[W:2 * W], eps), mod[2 * W:]
        elif not gr00t:
            t = np.float32(1.0) + np.float32(s) * dt32
            bias = bias + orc.sinusoidal_time_emb(float(t), W, cfg["min_period"], cfg["max_period"])
        if head_io:
            # ActionExpert::encode_action (action_expert.cpp:46-52) with tau = action_sinusoid(bucket)
            tau = orc.action_sinusoid(int(s / steps * n_buckets), W, Sa)
            a_emb = orc.linear(x, w["aex.ae_W1"], w["aex.ae_b1"])
            m = orc.silu(orc.linear(np.concatenate([a_emb, tau], 1), w["aex.ae_W2"], w["aex.ae_b2"]))
            h = orc.linear(m, w["aex.ae_W3"], w["aex.ae_b3"]) + w["aex.pos_embd"][:Sa]
        elif "act.W_at1" in w and not gr00t:
            # action-time MLP (smolvla.cpp:1397-1403, pi0.cpp:240-244), in the reference's order
            t = np.float32(1.0) + np.float32(s) * dt32
            temb = orc.sinusoidal_time_emb(float(t), W, cfg["min_period"], cfg["max_period"])
            action_emb = orc.linear(x, w["act.W_in"], w["act.b_in"])
            cat = np.concatenate([action_emb, np.broadcast_to(temb, action_emb.shape)], 1)
            mlp1 = orc.linear(cat, w["act.W_at1"], w["act.b_at1"])
            h = orc.linear(orc.silu(mlp1), w["act.W_at2"], w["act.b_at2"])
        else:
            h = orc.linear(x, w["act.W_in"], bias)
        if n_lead:
            h = np.concatenate([lead, h], 0)
        h = rnd(h)
        for l in range(L):
            p = "ex.%d." % l
            self_l = _is_self(cfg, l)
            if pi05:
                hn, gate_attn = adarms(h, p + "ada_in")
                hn = rnd(hn)
            elif gr00t:
                c = ada[s][l]
                hn = rnd(orc.adaln(h, c[:W], c[W:], eps))
            else:
                hn = rnd(orc.rms_norm(h, w[p + "ln"], eps))
            if self_l:
                y = orc.linear(hn, w[p + "Wqkv"], w.get(p + "bqkv"))
                q, k, v = _split_heads(y, Hq, Hkv, D)
                if not gr00t:
                    q, k = orc.rope_neox(q, cs, ss), orc.rope_neox(k, cs, ss)
                q, k, v = rnd(q), rnd(k), rnd(v)
                if cacheK[l] is not None:
                    K_full, V_full = orc.kv_concat(cacheK[l], k), orc.kv_concat(cacheV[l], v)
                    m = mask_self
                else:  # GR00T self-attention over the suffix tokens only
                    K_full, V_full, m = k, v, None
            else:
                q = orc.linear(hn, w[p + "Wq"], w.get(p + "bq")).reshape(S, Hq, D)
                if not gr00t:
                    q = orc.rope_neox(q, cc, sc_)
                q = rnd(q)
                K_full, V_full = cacheK[l], cacheV[l]
                m = mask_cross if (pad[1] > pad[0]) else None
            att = rnd(orc.attention(q, K_full, V_full, m, scale))
            if pi05:
                # gated residuals (pi05.cpp:273-282)
                h = rnd(h + orc.linear(att, w[p + "Wo"]) * gate_attn)
                if cfg.get("ffn_dim", 0) > 0:
                    I = cfg["ffn_dim"]
                    n2, gate_ffn = adarms(h, p + "ada_post")
                    n2 = rnd(n2)
                    Wgu = w[p + "Wgu"]
                    mid = rnd(orc.gelu(orc.linear(n2, Wgu[:I])) * orc.linear(n2, Wgu[I:]))
                    h = rnd(h + orc.linear(mid, w[p + "Wd"]) * gate_ffn)
                continue
            h = rnd(orc.linear(att, w[p + "Wo"], w.get(p + "bo")) + h)
            if cfg.get("ffn_dim", 0) > 0:
                # the FFN half of the layer (smolvla.cpp:845-848, pi0.cpp:227-232, dit_head.cpp:132-133)
                I = cfg["ffn_dim"]
                if gr00t:
                    n3 = rnd(orc.layer_norm(h, None, None, eps))
                    mid = rnd(orc.gelu(orc.linear(n3, w[p + "W1"], w[p + "b1"])))
                    h = rnd(orc.linear(mid, w[p + "W2"], w[p + "b2"]) + h)
                else:
                    n2 = rnd(orc.rms_norm(h, w[p + "ln2"], eps))
                    act = orc.silu if arch == "smolvla" else orc.gelu
                    Wgu = w[p + "Wgu"]
                    mid = rnd(act(orc.linear(n2, Wgu[:I])) * orc.linear(n2, Wgu[I:]))
                    h = rnd(orc.linear(mid, w[p + "Wd"]) + h)
            if return_debug and s == 0 and l == 0:
                debug["q0"], debug["att0"], debug["h0"] = q, att, h
        if pi05:
            hn = rnd(adarms(h, "act.ada_final")[0])
        elif head_io:
            # DitHead::proj_out (dit_head.cpp:139-147) then ActionExpert::decode (action_expert.cpp:54-57)
            sh, sc = po_mod[s][:W], po_mod[s][W:]
            hn = rnd(orc.adaln(h, sc, sh, cfg.get("norm_out_eps", 1e-6)))
            d1 = rnd(orc.linear(hn, w["aex.po2W"], w["aex.po2b"]))
            d2 = rnd(np.maximum(orc.linear(d1, w["aex.ad_l1W"], w["aex.ad_l1b"]), 0))
            v_t = orc.linear(d2[n_lead:], w["aex.ad_l2W"], w["aex.ad_l2b"])
            x = (x + dt32 * v_t).astype(np.float32)
            continue
        elif gr00t:
            hn = rnd(orc.layer_norm(h, None, None, cfg.get("norm_out_eps", 1e-6)))
        else:
            hn = rnd(orc.rms_norm(h, w["act.norm"], eps))
        v_t = orc.linear(hn[n_lead:], w["act.W_out"], w["act.b_out"])
        x = (x + dt32 * v_t).astype(np.float32)
    x[:, cfg["real_action_dim"]:] = 0
    return (x, debug) if return_debug else x


def bitvla_ternary(cfg, w, name, from_fp32):
    """(ternary int8 [N,K], per-row-group scales expanded to ws groups) as the loader derives them."""
    kvd = cfg["n_kv_heads"] * cfg["head_dim"]
    t = w[name + ".t"]
    parts = [cfg["hidden"], kvd, kvd] if name.endswith("Wqkv") else ([t.shape[0] // 2] * 2 if name.endswith("Wgu") else [t.shape[0]])
    group = kvd if name.endswith("Wqkv") else parts[0]
    if from_fp32:
        scales, row, tt = [], 0, np.empty_like(t)
        for n, s in zip(parts, w[name + ".ws"]):
            deq = t[row:row + n].astype(np.float32) * np.float32(s)
            q, am = orc.weight_quant_ternary(deq)
            tt[row:row + n] = q
            scales.append(am)
            row += n
        t = tt
    else:
        scales = list(w[name + ".ws"])
    ws = np.float32([s for n, s in zip(parts, scales) for _ in range(n // group)])
    return t, ws


def bitvla_chunk(cfg, w, obs, from_fp32=False):
    """BitVLA-shape prefix prefill + autoregressive-style append of the action tokens.

    One layer = run_layer's attention half (src/kernels/bitvla/bitvla_lm_cuda.cu:422-486):
    bf16 rmsnorm -> act-quant -> ternary GEMM (int32, bf16 out) -> RoPE(Q,K) ->
    attention -> bf16 sub-norm -> act-quant -> ternary O GEMM -> bf16 add; with cfg["ffn_dim"]
    also its squared-ReLU GLU half (488-520): ffn norm -> act-quant -> fused gate|up GEMM ->
    relu(gate)^2 * up -> ffn sub-norm -> act-quant -> down GEMM -> bf16 add.
    Returns (actions [n_act, A], int32 accumulators of layer 0's QKV GEMM over the prefix).
    """
    L, Hq, Hkv, D, H = cfg["n_layers"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["hidden"]
    kvd, n_act, A = Hkv * D, cfg["n_suffix"], cfg["max_action_dim"]
    eps, scale = cfg["rms_eps"], 1.0 / math.sqrt(D)
    P = cfg["n_img"] + cfg["n_lang"]
    rb = orc.round_bf16
    tern = [(bitvla_ternary(cfg, w, "lm.%d.Wqkv" % l, from_fp32), bitvla_ternary(cfg, w, "lm.%d.Wo" % l, from_fp32))
            for l in range(L)]
    F = cfg.get("ffn_dim", 0)
    tern_ffn = [(bitvla_ternary(cfg, w, "lm.%d.Wgu" % l, from_fp32), bitvla_ternary(cfg, w, "lm.%d.Wd" % l, from_fp32))
                for l in range(L)] if F > 0 else None
    cos_t, sin_t = orc.rope_tables(np.arange(P + n_act, dtype=np.int32), D, cfg["rope_freq_base"])
    cacheK, cacheV = [None] * L, [None] * L
    acc0 = [None]

    def bitlinear(x_bf, t, ws, keep=False):
        q, s = orc.act_quant(x_bf)
        acc = orc.ternary_gemm_i32(q, t)
        if keep and acc0[0] is None:
            acc0[0] = acc
        return orc.from_bf16(orc.ternary_epilogue(acc, s, ws))

    def layers(h, tok0):
        n = h.shape[0]
        for l in range(L):
            (tq, wsq), (to, wso) = tern[l]
            hn = rb(orc.rms_norm(h, w["lm.%d.attn_norm" % l], eps))
            y = bitlinear(hn, tq, wsq, keep=(l == 0))
            q, k, v = _split_heads(y, Hq, Hkv, D)
            q = rb(orc.rope_neox(q, cos_t[tok0:tok0 + n], sin_t[tok0:tok0 + n]))
            k = rb(orc.rope_neox(k, cos_t[tok0:tok0 + n], sin_t[tok0:tok0 + n]))
            if tok0 == 0:
                cacheK[l], cacheV[l] = k, v.copy()
            else:
                cacheK[l], cacheV[l] = orc.kv_concat(cacheK[l][:tok0], k), orc.kv_concat(cacheV[l][:tok0], v)
            att = rb(orc.attention(q, cacheK[l], cacheV[l], None, scale))
            sub = rb(orc.rms_norm(att, w["lm.%d.sub_norm" % l], eps))
            o = bitlinear(sub, to, wso)
            h = rb(h + o)
            if F > 0:
                (tg, wsg), (td, wsd) = tern_ffn[l]
                gu = bitlinear(rb(orc.rms_norm(h, w["lm.%d.ffn_norm" % l], eps)), tg, wsg)
                act = sqrelu_mul(gu, F)
                h = rb(h + bitlinear(rb(orc.rms_norm(act, w["lm.%d.ffn_sub_norm" % l], eps)), td, wsd))
        return h

    emb = np.concatenate([np.asarray(obs["img_emb"], np.float32).reshape(cfg["n_img"], H),
                          w["prefix.E_lang"][np.asarray(obs["lang"], np.int32)]], 0)
    layers(rb(emb), 0)
    hfin = []
    for t in range(n_act):
        h = layers(rb(w["act.emb"][t][None, :]), P + t)
        hfin.append(rb(orc.rms_norm(h, w["act.norm"], eps)))
    hf = np.concatenate(hfin, 0)
    x = orc.linear(hf, w["act.W_out"], w["act.b_out"])
    x[:, cfg["real_action_dim"]:] = 0
    return x, acc0[0]


def sqrelu_mul(gu, ffn):
    """gate_up_fused_sqrelu_mul_bf16 (src/kernels/bitvla/bitvla_lm_cuda.cu:525-548): relu(gate)^2 * up
    on a fused [seq, gate(ffn) | up(ffn)] projection, fp32 products, one rounding to bf16."""
    gu = np.asarray(gu, np.float32)
    g = np.maximum(gu[:, :ffn], np.float32(0))
    return orc.round_bf16((g * g) * gu[:, ffn:2 * ffn])


def bitvla_lm_forward(x, layers, out_norm, n_q, n_kv, D, eps, rope_base):
    """bitvla_lm_cuda_forward (src/kernels/bitvla/bitvla_lm_cuda.cu:668-724): every layer of run_layer
    (395-522) over all seq tokens, no mask, positions 0..seq-1, then the output RMSNorm.

    x [seq, hidden] (bf16 values); layers: dicts with attn_norm, sub_norm, ffn_norm, ffn_sub_norm
    (fp32 vectors of bf16 values) and q, k, v, o, gate_up, down = (ternary int8 [N, K], scales) with one
    scale per tensor, two for gate_up.  Every stored intermediate is rounded to bf16 as the kernels
    store it; scores and softmax are exact (the reference keeps bf16 scores between two GEMMs)."""
    rb = orc.round_bf16
    seq = x.shape[0]
    cos_t, sin_t = orc.rope_tables(np.arange(seq, dtype=np.int32), D, rope_base)
    scale = 1.0 / math.sqrt(D)

    def bitlinear(x_bf, tw):
        t, ws = tw
        q, s = orc.act_quant(x_bf)
        return orc.from_bf16(orc.ternary_epilogue(orc.ternary_gemm_i32(q, t), s, np.asarray(ws, np.float32)))

    h = rb(x)
    for w in layers:
        hn = rb(orc.rms_norm(h, w["attn_norm"], eps))
        q = bitlinear(hn, w["q"]).reshape(seq, n_q, D)
        k = bitlinear(hn, w["k"]).reshape(seq, n_kv, D)
        v = bitlinear(hn, w["v"]).reshape(seq, n_kv, D)
        q, k = rb(orc.rope_neox(q, cos_t, sin_t)), rb(orc.rope_neox(k, cos_t, sin_t))
        att = rb(orc.attention(q, k, v, None, scale)).reshape(seq, n_q * D)
        h = rb(h + bitlinear(rb(orc.rms_norm(att, w["sub_norm"], eps)), w["o"]))
        gu = bitlinear(rb(orc.rms_norm(h, w["ffn_norm"], eps)), w["gate_up"])
        ffn = gu.shape[1] // 2
        act = sqrelu_mul(gu, ffn)
        h = rb(h + bitlinear(rb(orc.rms_norm(act, w["ffn_sub_norm"], eps)), w["down"]))
    return rb(orc.rms_norm(h, out_norm, eps))
