"""A second, independent statement of the action-chunk definitions, in float64 torch.

TEST INFRASTRUCTURE.  oracle/chunk.py composes the oracle's own scalar C++ primitives; this
module is what pins that composition: it was written from the reference's graph builders and
host-side input construction alone, shares no code with the oracle, keeps one function per
architecture (no shared flag-driven loop), works on [token, feature] float64 tensors with
library routines (torch.softmax, F.layer_norm, F.silu, F.gelu, complex multiplication for
the rotation) and builds every mask and position vector from the reference's loops.

Definition of a synthetic chunk (the configurations carry no VLM backbone): every prefix layer
projects the *same* prefix embeddings; without `act.W_at1` the suffix embedding is
`W_in x + b_in + time_emb(t)`; without `ffn_dim` a layer ends after `x + Wo att`.

Reference sites:
  SmolVLA  src/models/smolvla.cpp:778-794 (prefix K/V), 796-834 (self layer), 838-846
           (cross K/V), 848-878 (cross layer), 1361-1419 (graph), 1608-1672 (masks, positions)
  pi0      src/models/pi0.cpp:159-233 (layer), 235-248 (suffix embedding), 559-588 (graph),
           612-661 (positions, mask, time)
  pi0.5    src/models/pi05.cpp:208-283 (adaRMS layer), 602-631 (graph)
  GR00T    src/modules/dit_head.cpp:87-147, src/layers/norm.h:37-46,
           src/models/gr00tn1d5.cpp:359-381, 413-420; src/models/gr00tn1d6.cpp:440-467
  time     src/layers/embed.h:32-44 (timesteps_proj), 61-73 (sinusoidal_time_emb)
"""
import math

import numpy as np
import torch
import torch.nn.functional as F

F64 = torch.float64


def T(a):
    return torch.as_tensor(np.asarray(a), dtype=F64)


def mm(W, x, b=None):
    """ggml_mul_mat(W [K, N], x [K, M]) -> [N, M]: rows of x against rows of W."""
    y = x @ T(W).T
    return y if b is None else y + T(b)


def rms(x, eps, w=None):
    n = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    return n if w is None else n * T(w)


def rope_neox(x, pos, base):
    """x [tokens, heads, D]; pair (i, i + D/2) turns by pos * base^(-2i/D)."""
    D = x.shape[-1]
    half = D // 2
    freq = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * torch.arange(half, dtype=F64) / D)
    ang = torch.as_tensor(np.asarray(pos), dtype=F64)[:, None] * freq[None, :]
    z = torch.complex(x[..., :half], x[..., half:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    return torch.cat([z.real, z.imag], -1)


def attend(q, k, v, mask, scale):
    """q [S, Hq, D], k / v [Tk, Hkv, D], additive mask [S, Tk] or None -> [S, Hq * D].
    Query head h reads kv head h * Hkv / Hq (repeat_kv_bf16_kernel, bitvla_lm_cuda.cu:181-190)."""
    S, Hq, D = q.shape
    rep = Hq // k.shape[1]
    kk, vv = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    sc = torch.einsum("shd,thd->hst", q, kk) * scale
    if mask is not None:
        sc = sc + mask[None]
    p = torch.softmax(sc, -1)
    return torch.einsum("hst,thd->shd", p, vv).reshape(S, Hq * D)


def time_emb(t, dim, min_p, max_p):
    half = dim // 2
    frac = torch.arange(half, dtype=F64) / max(half - 1, 1)
    if half == 1:
        frac = torch.zeros(1, dtype=F64)
    period = min_p * (max_p / min_p) ** frac
    s = 2.0 * math.pi / period * t
    return torch.cat([torch.sin(s), torch.cos(s)])


def timesteps_proj(bucket):
    i = torch.arange(128, dtype=F64)
    emb = float(bucket) * torch.exp(-math.log(10000.0) * i / 127.0)
    return torch.cat([torch.cos(emb), torch.sin(emb)])


def _inf_mask(rows, cols, blocked):
    m = torch.zeros((rows, cols), dtype=F64)
    for i in range(rows):
        for j in range(cols):
            if blocked(i, j):
                m[i, j] = -math.inf
    return m


def _split(y, Hq, Hkv, D):
    M = y.shape[0]
    return (y[:, :Hq * D].reshape(M, Hq, D), y[:, Hq * D:(Hq + Hkv) * D].reshape(M, Hkv, D),
            y[:, (Hq + Hkv) * D:].reshape(M, Hkv, D))


def _glu(cfg, w, p, h1, n2, act):
    I = cfg["ffn_dim"]
    Wgu = w[p + "Wgu"]
    inter = act(mm(Wgu[:I], n2)) * mm(Wgu[I:], n2)
    return mm(w[p + "Wd"], inter)


def _suffix_embedding(cfg, w, x, t):
    """Without the action-time MLP: W_in x + b_in + time_emb(t); with it the reference's
    concat(action_emb, time) -> W_at1 -> silu -> W_at2 (smolvla.cpp:1397-1403)."""
    W = cfg["expert_h"]
    te = time_emb(t, W, cfg["min_period"], cfg["max_period"])
    a = mm(w["act.W_in"], x, w["act.b_in"])
    if "act.W_at1" not in w:
        return a + te
    cat = torch.cat([a, te[None, :].expand(a.shape[0], W)], 1)
    return mm(w["act.W_at2"], F.silu(mm(w["act.W_at1"], cat, w["act.b_at1"])), w["act.b_at2"])


def smolvla(cfg, w, obs):
    L, Hq, Hkv, D = cfg["n_layers"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    Wv, S, steps, eps, base = cfg["hidden"], cfg["n_suffix"], cfg["num_steps"], cfg["rms_eps"], cfg["rope_freq_base"]
    n_img = obs["n_views"] * cfg["n_img"]
    n_lang_max, n_lang = cfg["n_lang"], len(obs["lang"])
    P = n_img + n_lang_max + 1
    Tn = P + S
    pad_start, pad_end = n_img + n_lang, n_img + n_lang_max
    state_pos = n_img + n_lang
    ids = np.zeros(n_lang_max, np.int64)
    ids[:n_lang] = obs["lang"]
    ls = math.sqrt(Wv)
    state = T(obs["state"]) if obs.get("state") is not None else torch.zeros(cfg["max_state_dim"], dtype=F64)
    prefix = torch.cat([T(obs["img_emb"]).reshape(n_img, Wv) * ls, T(w["prefix.E_lang"])[ids] * ls,
                        mm(w["prefix.Wstate"], state[None], w["prefix.bstate"])], 0)
    pos_prefill = [i if i < P - 1 else state_pos for i in range(P)]
    pos_full = [state_pos + 1 + i for i in range(S)]
    pos_rebased = list(range(S))
    causal = cfg["suffix_mask"] == 1  # the reference's block; 0 = the bidirectional variant of the benchmark
    mask_full = _inf_mask(S, Tn, lambda i, j: (pad_start <= j < pad_end) if j < P else (causal and (j - P) > i))
    mask_pfx = _inf_mask(S, P, lambda i, j: pad_start <= j < pad_end)
    scale = 1.0 / math.sqrt(D)
    kvd = Hkv * D
    is_self = [l % cfg["self_attn_every_n"] == 0 for l in range(L)]
    kc, vc = [], []
    for l in range(L):
        xn = rms(prefix, eps, w["vlm.%d.ln" % l])
        kv = mm(w["vlm.%d.Wkv" % l], xn)
        k = rope_neox(kv[:, :kvd].reshape(P, Hkv, D), pos_prefill, base)
        v = kv[:, kvd:].reshape(P, Hkv, D)
        if not is_self[l]:  # expert_cross_kv on the flattened, already rotated cache
            k = mm(w["ex.%d.Wk_x" % l], k.reshape(P, kvd)).reshape(P, Hkv, D)
            v = mm(w["ex.%d.Wv_x" % l], v.reshape(P, kvd)).reshape(P, Hkv, D)
        kc.append(k)
        vc.append(v)
    dt = -1.0 / steps
    x = T(obs["noise"]).reshape(S, cfg["max_action_dim"])
    for step in range(steps):
        h = _suffix_embedding(cfg, w, x, 1.0 + step * dt)
        for l in range(L):
            p = "ex.%d." % l
            xn = rms(h, eps, w[p + "ln"])
            if is_self[l]:
                q, k, v = _split(mm(w[p + "Wqkv"], xn), Hq, Hkv, D)
                q, k = rope_neox(q, pos_full, base), rope_neox(k, pos_full, base)
                att = attend(q, torch.cat([kc[l], k], 0), torch.cat([vc[l], v], 0), mask_full, scale)
            else:
                q = rope_neox(mm(w[p + "Wq"], xn).reshape(S, Hq, D), pos_rebased, base)
                att = attend(q, kc[l], vc[l], mask_pfx, scale)
            h = h + mm(w[p + "Wo"], att)
            if cfg.get("ffn_dim", 0) > 0:
                h = h + _glu(cfg, w, p, h, rms(h, eps, w[p + "ln2"]), F.silu)
        v_t = mm(w["act.W_out"], rms(h, eps, w["act.norm"]), w["act.b_out"])
        x = x + dt * v_t
    return _finish(cfg, x)


def pi0(cfg, w, obs):
    L, Hq, Hkv, D = cfg["n_layers"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    Wv, S, steps, eps, base = cfg["hidden"], cfg["n_suffix"], cfg["num_steps"], cfg["rms_eps"], cfg["rope_freq_base"]
    n_img = obs["n_views"] * cfg["n_img"]
    n_lang = len(obs["lang"])
    P, chunk = n_img + n_lang, S - 1
    prefix = torch.cat([T(obs["img_emb"]).reshape(n_img, Wv), T(w["prefix.E_lang"])[np.asarray(obs["lang"], np.int64)] * math.sqrt(Wv)], 0)
    pos_p, pos_s = list(range(P)), [P + i for i in range(S)]
    # row 0 is the state token: of the suffix it sees only itself (pi0.cpp:638-653)
    mask = _inf_mask(S, P + S, lambda i, j: j >= P and i == 0 and (j - P) != 0)
    scale = 1.0 / math.sqrt(D)
    kvd = Hkv * D
    kc, vc = [], []
    for l in range(L):
        kv = mm(w["vlm.%d.Wkv" % l], rms(prefix, eps, w["vlm.%d.ln" % l]))
        kc.append(rope_neox(kv[:, :kvd].reshape(P, Hkv, D), pos_p, base))
        vc.append(kv[:, kvd:].reshape(P, Hkv, D))
    state = T(obs["state"]) if obs.get("state") is not None else torch.zeros(cfg["max_state_dim"], dtype=F64)
    state_emb = mm(w["act.W_sp"], state[None], w["act.b_sp"])
    dt = -1.0 / steps
    x = T(obs["noise"]).reshape(chunk, cfg["max_action_dim"])
    for step in range(steps):
        h = torch.cat([state_emb, _suffix_embedding(cfg, w, x, 1.0 + step * dt)], 0)
        for l in range(L):
            p = "ex.%d." % l
            q, k, v = _split(mm(w[p + "Wqkv"], rms(h, eps, w[p + "ln"])), Hq, Hkv, D)
            q, k = rope_neox(q, pos_s, base), rope_neox(k, pos_s, base)
            h = h + mm(w[p + "Wo"], attend(q, torch.cat([kc[l], k], 0), torch.cat([vc[l], v], 0), mask, scale))
            if cfg.get("ffn_dim", 0) > 0:
                h = h + _glu(cfg, w, p, h, rms(h, eps, w[p + "ln2"]), lambda z: F.gelu(z, approximate="tanh"))
        hf = rms(h, eps, w["act.norm"])[1:]  # the action rows
        x = x + dt * mm(w["act.W_out"], hf, w["act.b_out"])
    return _finish(cfg, x)


def pi05(cfg, w, obs):
    L, Hq, Hkv, D = cfg["n_layers"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    Wv, W, S, steps, eps, base = cfg["hidden"], cfg["expert_h"], cfg["n_suffix"], cfg["num_steps"], cfg["rms_eps"], cfg["rope_freq_base"]
    n_img = obs["n_views"] * cfg["n_img"]
    P = n_img + len(obs["lang"])
    prefix = torch.cat([T(obs["img_emb"]).reshape(n_img, Wv), T(w["prefix.E_lang"])[np.asarray(obs["lang"], np.int64)] * math.sqrt(Wv)], 0)
    pos_p, pos_s = list(range(P)), [P + i for i in range(S)]
    scale = 1.0 / math.sqrt(D)
    kvd = Hkv * D
    kc, vc = [], []
    for l in range(L):
        kv = mm(w["vlm.%d.Wkv" % l], rms(prefix, eps, w["vlm.%d.ln" % l]))
        kc.append(rope_neox(kv[:, :kvd].reshape(P, Hkv, D), pos_p, base))
        vc.append(kv[:, kvd:].reshape(P, Hkv, D))

    def adarms(x_, name, cond):
        mod = mm(w[name + "_w"], cond, w[name + "_b"])[0]
        n = rms(x_, eps)
        return n + n * mod[:W] + mod[W:2 * W], mod[2 * W:]

    dt = -1.0 / steps
    x = T(obs["noise"]).reshape(S, cfg["max_action_dim"])
    for step in range(steps):
        te = time_emb(1.0 + step * dt, W, cfg["min_period"], cfg["max_period"])[None]
        cond = F.silu(mm(w["te.W_tout"], F.silu(mm(w["te.W_tin"], te, w["te.b_tin"])), w["te.b_tout"]))
        h = mm(w["act.W_in"], x, w["act.b_in"])
        for l in range(L):
            p = "ex.%d." % l
            xn, g_attn = adarms(h, p + "ada_in", cond)
            q, k, v = _split(mm(w[p + "Wqkv"], xn), Hq, Hkv, D)
            q, k = rope_neox(q, pos_s, base), rope_neox(k, pos_s, base)
            h = h + mm(w[p + "Wo"], attend(q, torch.cat([kc[l], k], 0), torch.cat([vc[l], v], 0), None, scale)) * g_attn
            if cfg.get("ffn_dim", 0) > 0:
                n2, g_ffn = adarms(h, p + "ada_post", cond)
                h = h + _glu(cfg, w, p, h, n2, lambda z: F.gelu(z, approximate="tanh")) * g_ffn
        hf, _ = adarms(h, "act.ada_final", cond)
        x = x + dt * mm(w["act.W_out"], hf, w["act.b_out"])
    return _finish(cfg, x)


def gr00t(cfg, w, obs):
    """N1.5 (cross onto all backbone rows on even layers, self on odd) and N1.6 / N1.7
    (cross layers alternate text / image rows; with dit_interleave 0 every layer is a cross layer)."""
    L, H, D = cfg["n_layers"], cfg["n_q_heads"], cfg["head_dim"]
    Wv, W, S, steps, eps = cfg["hidden"], cfg["expert_h"], cfg["n_suffix"], cfg["num_steps"], cfg["rms_eps"]
    alt = cfg["arch"] == "gr00t_n1d6"
    interleave = bool(cfg.get("dit_interleave", 1))
    img = T(obs["img_emb"]).reshape(obs["n_views"] * cfg["n_img"], Wv)
    txt = img
    if alt and obs.get("lang") is not None and len(obs["lang"]):
        txt = T(w["prefix.E_lang"])[np.asarray(obs["lang"], np.int64)]
    if "prefix.vlln_w" in w:  # vlln on the backbone rows (gr00tn1d6.cpp:436)
        vl = lambda x: F.layer_norm(x, (Wv,), T(w["prefix.vlln_w"]), T(w["prefix.vlln_b"]), cfg.get("vlln_eps", 1e-5))
        img, txt = vl(img), vl(txt)
    scale = 1.0 / math.sqrt(D)
    kvd = H * D
    cross = [not (interleave and l % 2 == 1) for l in range(L)]
    Kc, Vc = [None] * L, [None] * L
    for l in range(L):
        if not cross[l]:
            continue
        src = txt if (alt and l % (2 * cfg["attend_text_every_n"]) == 0) else img
        kv = mm(w["vlm.%d.Wkv" % l], src, w["vlm.%d.bkv" % l])
        Kc[l], Vc[l] = kv[:, :kvd].reshape(-1, H, D), kv[:, kvd:].reshape(-1, H, D)
    state = T(obs["state"]) if obs.get("state") is not None else torch.zeros(cfg["max_state_dim"], dtype=F64)
    head_io = bool(cfg.get("head_io", 0))
    if head_io:  # encode_state, then the learned future tokens: 1 + num_future leading rows
        lead = mm(w["aex.se_l2W"], F.relu(mm(w["aex.se_l1W"], state[None], w["aex.se_l1b"])), w["aex.se_l2b"])
        if cfg["num_future"] > 0:  # N1.6 / N1.7 have no future tokens (gr00tn1d6.cpp:457)
            lead = torch.cat([lead, T(w["aex.future_tokens"])], 0)
    else:
        lead = mm(w["act.W_sp"], state[None], w["act.b_sp"])
    n_lead = lead.shape[0]
    AH = S - n_lead
    dt = 1.0 / steps
    x = T(obs["noise"]).reshape(AH, cfg["max_action_dim"])
    for s in range(steps):
        bucket = int(s / steps * cfg.get("num_buckets", 1000))
        temb = mm(w["te.l2W"], F.silu(mm(w["te.l1W"], timesteps_proj(bucket)[None], w["te.l1b"])), w["te.l2b"])
        if head_io:
            # encode_action: W3 silu(W2 [W1 x + b1 ; tau] + b2) + b3 + pos, tau = sin | cos of bucket * 10000^(-i / half)
            half = W // 2
            ang = float(bucket) * torch.exp(-torch.arange(half, dtype=F64) * (math.log(10000.0) / half))
            tau = torch.cat([torch.sin(ang), torch.cos(ang)])[None].expand(AH, W)
            a = mm(w["aex.ae_W1"], x, w["aex.ae_b1"])
            act_rows = mm(w["aex.ae_W3"], F.silu(mm(w["aex.ae_W2"], torch.cat([a, tau], 1), w["aex.ae_b2"])), w["aex.ae_b3"])
            h = torch.cat([lead, act_rows + T(w["aex.pos_embd"])[:AH]], 0)
        else:
            h = torch.cat([lead, mm(w["act.W_in"], x, w["act.b_in"])], 0)
        for l in range(L):
            p = "ex.%d." % l
            cond = mm(w[p + "adaln_w"], F.silu(temb), w[p + "adaln_b"])[0]
            xn = F.layer_norm(h, (W,), eps=eps)
            n = xn + xn * cond[:W] + cond[W:]
            if cross[l]:
                q = mm(w[p + "Wq"], n, w[p + "bq"]).reshape(S, H, D)
                att = attend(q, Kc[l], Vc[l], None, scale)
            else:
                q, k, v = _split(mm(w[p + "Wqkv"], n, w[p + "bqkv"]), H, H, D)
                att = attend(q, k, v, None, scale)
            h = h + mm(w[p + "Wo"], att, w[p + "bo"])
            if cfg.get("ffn_dim", 0) > 0:
                n3 = F.layer_norm(h, (W,), eps=eps)
                h = h + mm(w[p + "W2"], F.gelu(mm(w[p + "W1"], n3, w[p + "b1"]), approximate="tanh"), w[p + "b2"])
        hn = F.layer_norm(h, (W,), eps=cfg.get("norm_out_eps", 1e-6))
        if head_io:
            # proj_out: the dense on silu(temb) yields (shift, scale); then decode's relu MLP; the
            # velocity is the last AH rows
            po = mm(w["aex.po1W"], F.silu(temb), w["aex.po1b"])[0]
            hm = hn + hn * po[W:] + po[:W]
            pred = mm(w["aex.ad_l2W"], F.relu(mm(w["aex.ad_l1W"], mm(w["aex.po2W"], hm, w["aex.po2b"]), w["aex.ad_l1b"])), w["aex.ad_l2b"])
            x = x + dt * pred[-AH:]
        else:
            x = x + dt * mm(w["act.W_out"], hn[1:], w["act.b_out"])
    return _finish(cfg, x)


def _finish(cfg, x):
    out = x.numpy().copy()
    out[:, cfg["real_action_dim"]:] = 0
    return out


def chunk(cfg, w, obs):
    return {"smolvla": smolvla, "pi0": pi0, "pi05": pi05, "gr00t_n1d5": gr00t, "gr00t_n1d6": gr00t}[cfg["arch"]](cfg, w, obs)
