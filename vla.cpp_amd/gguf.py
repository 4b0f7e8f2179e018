"""GGUF files: a writer, a ctypes mirror of the library's reader, and export of the
synthetic checkpoints under the reference's tensor names.

The reader (``Reader``) binds ``include/vla_gguf.h``; its method names are those of the
reference's ``struct gguf_reader`` (src/gguf_reader.h:33-216).  The writer follows the
published container format (versions 2 and 3) and exists so that tests and users without
the reference's converters (scripts/convert_*_to_gguf.py need the ``gguf`` package) can
produce files ``vla_model_load`` accepts.
"""
import ctypes
import struct

import numpy as np

# metadata value types / tensor types by their on-disk numbers
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
T_F32, T_F16, T_I8, T_BF16 = 0, 1, 24, 30
_SCALAR_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
               F64: "<d"}


def _s(text):
    b = text.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _value(vtype, value):
    if vtype == STRING:
        return _s(value)
    if vtype == ARRAY:
        etype, items = value
        out = struct.pack("<IQ", etype, len(items))
        for it in items:
            out += _value(etype, it)
        return out
    return struct.pack(_SCALAR_FMT[vtype], value)


def bf16_bits(x):
    """fp32 -> bf16 bits, round to nearest even (values must not be NaN)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def write_gguf(path, kv, tensors, alignment=32, version=3):
    """kv: {key: (value type, value)}; tensors: {name: (type number, ndarray)} in the order
    given.  An array's numpy shape is written reversed (ne[0] = last numpy axis).  BF16
    tensors are passed as uint16 bit patterns, F16 as float16, I8 as int8 / uint8 bytes."""
    kv = dict(kv)
    if alignment != 32:
        kv["general.alignment"] = (U32, alignment)
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(kv))
    for k, (vt, v) in kv.items():
        head += _s(k) + struct.pack("<I", vt) + _value(vt, v)
    infos, blobs, off = b"", [], 0
    for name, (tt, arr) in tensors.items():
        arr = np.ascontiguousarray(arr)
        want = {T_F32: np.float32, T_F16: np.float16, T_BF16: np.uint16}.get(tt)
        if want is not None and arr.dtype != want:
            raise ValueError("%s: dtype %s does not match tensor type %d" % (name, arr.dtype, tt))
        if tt == T_I8 and arr.dtype.itemsize != 1:
            raise ValueError("%s: I8 tensors take one-byte elements" % name)
        dims = list(reversed(arr.shape)) or [1]
        infos += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", tt, off)
        blobs.append((off, arr.tobytes()))
        off = (off + arr.nbytes + alignment - 1) // alignment * alignment
    head += infos
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        pos = 0
        for o, b in blobs:
            f.write(b"\0" * (o - pos))
            f.write(b)
            pos = o + len(b)


class Reader:
    """ctypes mirror of the library's GGUF reader (src/gguf_reader.h:33-216)."""

    def __init__(self, lib, path):
        self._L = lib
        vp, cp, i32, i64 = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int32, ctypes.c_int64
        sig = {
            "vla_gguf_open": (vp, [cp]), "vla_gguf_close": (None, [vp]), "vla_gguf_version": (i32, [vp]),
            "vla_gguf_data_offset": (i64, [vp]), "vla_gguf_has_key": (i32, [vp, cp]), "vla_gguf_key_type": (i32, [vp, cp]),
            "vla_gguf_u32": (ctypes.c_uint32, [vp, cp]), "vla_gguf_f32": (ctypes.c_float, [vp, cp]),
            "vla_gguf_f64": (ctypes.c_double, [vp, cp]), "vla_gguf_str": (i64, [vp, cp, vp, i64]),
            "vla_gguf_array_len": (i64, [vp, cp, vp]), "vla_gguf_n_tensors": (i64, [vp]),
            "vla_gguf_tensor_name": (cp, [vp, i64]), "vla_gguf_tensor_info": (i32, [vp, cp, vp, vp, vp, vp, vp]),
            "vla_gguf_read_raw": (i32, [vp, cp, vp, i64]), "vla_gguf_read_f32": (i32, [vp, cp, vp, i64]),
            "vla_gguf_read_convert": (i32, [vp, cp, i32, i32, vp, i64]),
            "vla_gguf_fetch_rows_f32": (i32, [vp, cp, vp, i64, vp, i64]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        self._h = lib.vla_gguf_open(path.encode())
        if not self._h:
            raise RuntimeError("vla_gguf_open failed for %s" % path)

    def close(self):
        if self._h:
            self._L.vla_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    version = property(lambda self: self._L.vla_gguf_version(self._h))
    data_offset = property(lambda self: self._L.vla_gguf_data_offset(self._h))

    def has(self, k):
        return bool(self._L.vla_gguf_has_key(self._h, k.encode()))

    def key_type(self, k):
        return self._L.vla_gguf_key_type(self._h, k.encode())

    def u32(self, k):
        return self._L.vla_gguf_u32(self._h, k.encode())

    def f32(self, k):
        return self._L.vla_gguf_f32(self._h, k.encode())

    def f64(self, k):
        return self._L.vla_gguf_f64(self._h, k.encode())

    def str(self, k):
        n = self._L.vla_gguf_str(self._h, k.encode(), None, 0)
        if n < 0:
            return ""
        buf = ctypes.create_string_buffer(n + 1)
        self._L.vla_gguf_str(self._h, k.encode(), buf, n + 1)
        return buf.raw[:n].decode("utf-8")

    def array_len(self, k):
        et = ctypes.c_int32(-1)
        n = self._L.vla_gguf_array_len(self._h, k.encode(), ctypes.byref(et))
        return n, et.value

    def tensor_names(self):
        return [self._L.vla_gguf_tensor_name(self._h, i).decode() for i in range(self._L.vla_gguf_n_tensors(self._h))]

    def meta(self, name):
        """None, or dict(type, n_dims, ne, offset, nbytes)."""
        t, nd, off, nb = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64(), ctypes.c_int64()
        ne = (ctypes.c_int64 * 4)()
        rc = self._L.vla_gguf_tensor_info(self._h, name.encode(), ctypes.byref(t), ctypes.byref(nd), ne, ctypes.byref(off),
                                          ctypes.byref(nb))
        if rc != 0:
            return None
        return dict(type=t.value, n_dims=nd.value, ne=list(ne), offset=off.value, nbytes=nb.value)

    def read_raw(self, name, nbytes):
        buf = np.empty(nbytes, np.uint8)
        rc = self._L.vla_gguf_read_raw(self._h, name.encode(), buf.ctypes.data, nbytes)
        return buf if rc == 0 else None

    def read_f32(self, name):
        m = self.meta(name)
        if m is None:
            return None
        out = np.empty(int(np.prod(m["ne"])), np.float32)
        rc = self._L.vla_gguf_read_f32(self._h, name.encode(), out.ctypes.data, out.size)
        return out.reshape(list(reversed(m["ne"][:m["n_dims"]]))) if rc == 0 else None

    def read_convert(self, name, target, gemma_norm=False):
        m = self.meta(name)
        if m is None:
            return None
        n = int(np.prod(m["ne"]))
        nbytes = {T_F32: 4 * n, T_BF16: 2 * n}.get(target, m["nbytes"])
        out = np.empty(nbytes, np.uint8)
        rc = self._L.vla_gguf_read_convert(self._h, name.encode(), target, int(gemma_norm), out.ctypes.data, nbytes)
        return out if rc == 0 else None

    def fetch_rows_f32(self, name, rows, cols):
        ids = np.ascontiguousarray(rows, np.int32)
        out = np.empty((ids.size, cols), np.float32)
        rc = self._L.vla_gguf_fetch_rows_f32(self._h, name.encode(), ids.ctypes.data, ids.size, out.ctypes.data, cols)
        return out if rc == 0 else None


def _wt(cfg, a):
    """A weight matrix in the file's type: BF16 bits for bf16 models, else F32."""
    if cfg["dtype"] == "bf16":
        return (T_BF16, bf16_bits(a))
    return (T_F32, np.ascontiguousarray(a, np.float32))


def write_synthetic_gguf(path, cfg, w, ladder_pack=None):
    """The synthetic weights of checkpoint.synth_weights under the reference's GGUF names
    and metadata keys: SmolVLA (src/models/smolvla.cpp:570-634, 648-755, 1099-1236), pi0
    (src/models/pi0.cpp:252-297, 427-437), pi0.5 (src/models/pi05.cpp:292-328, 459-485) --
    these need cfg["ffn_dim"] and, except pi0.5, cfg["time_mlp"] -- and the BitVLA language model
    (src/models/bitvla.cpp:349-373, 640-700; ladder_pack(int8 [N, K]) -> bytes writes the
    int2-packed form with ".scale" sidecars, else float tensors the loader quantises)."""
    f32 = lambda a: (T_F32, np.ascontiguousarray(a, np.float32))
    L, Hq, Hkv, D = cfg["n_layers"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd = Hq * D, Hkv * D
    kv, t = {}, {}
    if cfg["arch"] in ("smolvla", "pi0", "pi05"):
        arch = cfg["arch"]
        smol, pi05 = arch == "smolvla", arch == "pi05"
        I, W = cfg["ffn_dim"], cfg["expert_h"]
        u = lambda k, v: kv.__setitem__(arch + "." + k, (U32, int(v)))
        # Gemma norm weights are stored minus one (the loader adds it back); exact for the
        # synthetic weights, which lie in [0.5, 2)
        nrm = (lambda a: f32(a)) if smol else (lambda a: f32(np.asarray(a, np.float32) - np.float32(1)))
        kv[arch + ".architecture"] = (STRING, arch)
        chunk = cfg["n_suffix"] - (1 if arch == "pi0" else 0)
        for k, v in (("hidden", cfg["hidden"]), ("intermediate", 4 * cfg["hidden"]), ("n_q_heads", Hq), ("n_kv_heads", Hkv),
                     ("head_dim", D), ("n_layers", L), ("expert_h", W), ("expert_inter", I), ("chunk_size", chunk),
                     ("num_steps", cfg["num_steps"]), ("max_state_dim", cfg["max_state_dim"]),
                     ("max_action_dim", cfg["max_action_dim"]), ("real_state_dim", cfg["real_state_dim"]),
                     ("real_action_dim", cfg["real_action_dim"]), ("tokenizer_max_length", cfg["n_lang"]),
                     ("n_img_tokens", cfg["n_img"])):
            u(k, v)
        if smol:
            u("vocab_size", cfg["vocab"])
            u("self_attn_every_n_layers", cfg["self_attn_every_n"])
        kv[arch + ".min_period"] = (F64, float(cfg["min_period"]))
        kv[arch + ".max_period"] = (F64, float(cfg["max_period"]))
        t["token_embd.weight"] = f32(w["prefix.E_lang"])
        if smol:
            t["state_proj.weight"], t["state_proj.bias"] = f32(w["prefix.Wstate"]), f32(w["prefix.bstate"])
        elif not pi05:
            t["state_proj.weight"], t["state_proj.bias"] = f32(w["act.W_sp"]), f32(w["act.b_sp"])
        t["action_in_proj.weight"], t["action_in_proj.bias"] = f32(w["act.W_in"]), f32(w["act.b_in"])
        t["action_out_proj.weight"], t["action_out_proj.bias"] = f32(w["act.W_out"]), f32(w["act.b_out"])
        if pi05:
            t["time_mlp_in.weight"], t["time_mlp_in.bias"] = f32(w["te.W_tin"]), f32(w["te.b_tin"])
            t["time_mlp_out.weight"], t["time_mlp_out.bias"] = f32(w["te.W_tout"]), f32(w["te.b_tout"])
            t["aex.output_norm.weight"], t["aex.output_norm.bias"] = f32(w["act.ada_final_w"]), f32(w["act.ada_final_b"])
        else:
            t["action_time_mlp_in.weight"], t["action_time_mlp_in.bias"] = f32(w["act.W_at1"]), f32(w["act.b_at1"])
            t["action_time_mlp_out.weight"], t["action_time_mlp_out.bias"] = f32(w["act.W_at2"]), f32(w["act.b_at2"])
            t["aex.output_norm.weight"] = nrm(w["act.norm"])
        every = cfg["self_attn_every_n"] if smol else 1
        for l in range(L):
            a, v, e, p = "aex.blk.%d." % l, "vlm.blk.%d." % l, "ex.%d." % l, "vlm.%d." % l
            if pi05:
                t[a + "attn_norm.weight"], t[a + "attn_norm.bias"] = f32(w[e + "ada_in_w"]), f32(w[e + "ada_in_b"])
                t[a + "ffn_norm.weight"], t[a + "ffn_norm.bias"] = f32(w[e + "ada_post_w"]), f32(w[e + "ada_post_b"])
            else:
                t[a + "attn_norm.weight"], t[a + "ffn_norm.weight"] = nrm(w[e + "ln"]), nrm(w[e + "ln2"])
            if l % every == 0:
                Wqkv = w[e + "Wqkv"]
                t[a + "attn_q.weight"], t[a + "attn_k.weight"] = _wt(cfg, Wqkv[:qd]), _wt(cfg, Wqkv[qd:qd + kvd])
                t[a + "attn_v.weight"] = _wt(cfg, Wqkv[qd + kvd:])
            else:
                t[a + "attn_q.weight"], t[a + "attn_k.weight"] = _wt(cfg, w[e + "Wq"]), _wt(cfg, w[e + "Wk_x"])
                t[a + "attn_v.weight"] = _wt(cfg, w[e + "Wv_x"])
            t[a + "attn_o.weight"] = _wt(cfg, w[e + "Wo"])
            t[a + "ffn_gate.weight"], t[a + "ffn_up.weight"] = _wt(cfg, w[e + "Wgu"][:I]), _wt(cfg, w[e + "Wgu"][I:])
            t[a + "ffn_down.weight"] = _wt(cfg, w[e + "Wd"])
            t[v + "attn_norm.weight"] = nrm(w[p + "ln"])
            t[v + "attn_k.weight"], t[v + "attn_v.weight"] = _wt(cfg, w[p + "Wkv"][:kvd]), _wt(cfg, w[p + "Wkv"][kvd:])
            # tensors of the file that are not on the path; the importer must skip them
            t[v + "attn_q.weight"] = _wt(cfg, np.zeros((8, cfg["hidden"]), np.float32))
    elif cfg["arch"] == "bitvla":
        H = cfg["hidden"]
        kv["bitvla.architecture"] = (STRING, "bitvla")
        for k, v in (("lm.hidden", H), ("lm.layers", L), ("lm.q_heads", Hq), ("lm.kv_heads", Hkv), ("lm.head_dim", D),
                     ("lm.vocab_size", cfg["vocab"]), ("vit.n_patches", cfg["n_img"]), ("lm.max_text", cfg["n_lang"]),
                     ("action.action_dim", cfg["real_action_dim"]), ("quant.int2_packed", 1 if ladder_pack else 0)):
            kv["bitvla." + k] = (U32, int(v))
        kv["bitvla.lm.rms_eps"] = (F32, float(cfg["rms_eps"]))
        kv["bitvla.lm.rope_theta"] = (F32, float(cfg["rope_freq_base"]))
        t["token_embd.weight"] = f32(w["prefix.E_lang"])
        t["lm.output_norm.weight"] = f32(w["act.norm"])
        t["act.emb"], t["act.W_out"], t["act.b_out"] = f32(w["act.emb"]), f32(w["act.W_out"]), f32(w["act.b_out"])
        for l in range(L):
            b, o = "lm.blk.%d." % l, "lm.%d." % l
            t[b + "attn_norm.weight"], t[b + "attn_sub_norm.weight"] = f32(w[o + "attn_norm"]), f32(w[o + "sub_norm"])
            tq, ws = w[o + "Wqkv.t"], w[o + "Wqkv.ws"]
            parts = (("attn_q", tq[:qd], ws[0]), ("attn_k", tq[qd:qd + kvd], ws[1]), ("attn_v", tq[qd + kvd:], ws[2]),
                     ("attn_o", w[o + "Wo.t"], w[o + "Wo.ws"][0]))
            for name, tern, scale in parts:
                if ladder_pack:
                    t[b + name + ".weight"] = (T_I8, np.ascontiguousarray(ladder_pack(tern), np.uint8))
                    t[b + name + ".scale"] = f32(np.float32([scale]))
                else:
                    # floats whose absmean quantisation gives back (tern, scale): see checkpoint._dequant_sources
                    t[b + name + ".weight"] = f32(tern.astype(np.float32) * np.float32(scale))
    elif cfg["arch"] in ("gr00t_n1d5", "gr00t_n1d6") and cfg.get("head_io", 0):
        # GR00T action head (src/models/gr00tn1d5.cpp:92-147; src/modules/dit_head.cpp:29-85;
        # src/modules/action_expert.cpp:20-39): the head's MLPs are cat_linear stacks, one
        # [in][out] matrix per embodiment (ggml ne = [out, in, n]); the synthetic weights go into
        # row `embodiment`, the other rows hold noise that must not be read.  N1.6 / N1.7
        # (cfg["variant"] "n1_6" / "n1_7"; src/models/gr00tn1d6.cpp:96-189, 294-298,
        # src/models/gr00tn1d7.cpp:119-215): their key prefix, no future tokens,
        # attend_text_every_n_blocks, embodiment_id_mapping written with a space after the colon
        # as json.dumps does, token_embd.weight for the text rows and aex.vlln.
        W, Wv, I, A = cfg["expert_h"], cfg["hidden"], cfg["ffn_dim"], cfg["max_action_dim"]
        alt = cfg["arch"] == "gr00t_n1d6"
        variant = cfg.get("variant", "n1_6") if alt else "n1_5"
        pfx = "gr00t_%s." % variant
        n_emb, emb = cfg.get("max_embodiments", 32), cfg.get("embodiment", {"n1_5": 24, "n1_6": 20, "n1_7": 2}[variant])
        rr = np.random.default_rng(99)
        kv[pfx + "architecture"] = (STRING, "gr00t_" + variant)
        for k, v in (("backbone_embedding_dim", Wv), ("input_embedding_dim", W), ("dit_hidden", W), ("dit_heads", Hq),
                     ("dit_head_dim", D), ("dit_layers", L), ("dit_interleave", cfg.get("dit_interleave", 1)),
                     ("action_horizon", cfg["n_suffix"] - 1 - cfg["num_future"]),
                     ("action_dim", A), ("max_state_dim", cfg["max_state_dim"]), ("num_inference_timesteps", cfg["num_steps"]),
                     ("num_timestep_buckets", cfg.get("num_buckets", 1000)), ("max_num_embodiments", n_emb),
                     ("n_img_tokens", cfg["n_img"])):
            kv[pfx + k] = (U32, int(v))
        kv[pfx + "ln_eps"] = (F32, float(cfg["rms_eps"]))
        kv[pfx + "norm_out_eps"] = (F32, float(cfg["norm_out_eps"]))
        if alt:
            kv[pfx + "attend_text_every_n_blocks"] = (U32, int(cfg["attend_text_every_n"]))
            kv[pfx + "max_seq_len"] = (U32, int(cfg["n_lang"]))
            kv[pfx + "vlln_eps"] = (F32, float(cfg.get("vlln_eps", 1e-5)))
            tag = cfg.get("default_tag", "gr1" if variant == "n1_6" else "libero_sim")
            kv[pfx + "embodiment_id_mapping"] = (STRING, '{"new_embodiment": 31, "%s": %d, "other_robot": 3}' % (tag, emb))
            if cfg.get("vocab", 0) > 0:
                t["token_embd.weight"] = f32(w["prefix.E_lang"])
            # N1.7's vlln sits in front of the VL self-attention stack, inside the backbone: present in the file, not on the path
            t["aex.vlln.weight"] = f32(w["prefix.vlln_w"] if "prefix.vlln_w" in w else np.ones(Wv))
            t["aex.vlln.bias"] = f32(w["prefix.vlln_b"] if "prefix.vlln_b" in w else np.zeros(Wv))
        else:
            kv[pfx + "num_target_vision_tokens"] = (U32, int(cfg["num_future"]))
            kv[pfx + "embodiment_tag_mapping"] = (STRING, '{"new_embodiment":31,"gr1":%d}' % emb)

        def cat(wm, b):  # [out][in] weight, [out] bias -> per-embodiment stacks
            wm, b = np.asarray(wm, np.float32), np.asarray(b, np.float32)
            W3 = rr.standard_normal((n_emb, wm.shape[1], wm.shape[0])).astype(np.float32)
            B2 = rr.standard_normal((n_emb, wm.shape[0])).astype(np.float32)
            W3[emb], B2[emb] = wm.T, b
            return f32(W3), f32(B2)

        # (the synthetic time-embedding weights are not bf16 values: kept F32 so the file equals the VLAW container)
        t["aex.dit.time_emb.l1.weight"], t["aex.dit.time_emb.l1.bias"] = f32(w["te.l1W"]), f32(w["te.l1b"])
        t["aex.dit.time_emb.l2.weight"], t["aex.dit.time_emb.l2.bias"] = f32(w["te.l2W"]), f32(w["te.l2b"])
        t["aex.dit.proj_out1.weight"], t["aex.dit.proj_out1.bias"] = f32(w["aex.po1W"]), f32(w["aex.po1b"])
        t["aex.dit.proj_out2.weight"], t["aex.dit.proj_out2.bias"] = _wt(cfg, w["aex.po2W"]), f32(w["aex.po2b"])
        for g_name, wn, bn in (("state_enc.l1", "se_l1W", "se_l1b"), ("state_enc.l2", "se_l2W", "se_l2b"), ("act_enc.W1", "ae_W1", "ae_b1"),
                               ("act_enc.W2", "ae_W2", "ae_b2"), ("act_enc.W3", "ae_W3", "ae_b3"), ("act_dec.l1", "ad_l1W", "ad_l1b"),
                               ("act_dec.l2", "ad_l2W", "ad_l2b")):
            t["aex.%s.W" % g_name], t["aex.%s.b" % g_name] = cat(w["aex." + wn], w["aex." + bn])
        t["aex.pos_embd"] = f32(w["aex.pos_embd"])
        if cfg["num_future"] > 0:
            t["aex.future_tokens"] = f32(w["aex.future_tokens"])
        interleave = bool(cfg.get("dit_interleave", 1))
        for l in range(L):
            a, e, p = "aex.dit.%d." % l, "ex.%d." % l, "vlm.%d." % l
            t[a + "adaln.weight"], t[a + "adaln.bias"] = _wt(cfg, w[e + "adaln_w"]), f32(w[e + "adaln_b"])
            if interleave and l % 2 == 1:
                Wqkv, bqkv = w[e + "Wqkv"], w[e + "bqkv"]
                parts = ((Wqkv[:W], bqkv[:W]), (Wqkv[W:2 * W], bqkv[W:2 * W]), (Wqkv[2 * W:], bqkv[2 * W:]))
            else:
                Wkv, bkv = w[p + "Wkv"], w[p + "bkv"]
                parts = ((w[e + "Wq"], w[e + "bq"]), (Wkv[:W], bkv[:W]), (Wkv[W:], bkv[W:]))
            for nm, (wm, bm) in zip(("attn_q", "attn_k", "attn_v"), parts):
                t[a + nm + ".weight"], t[a + nm + ".bias"] = _wt(cfg, wm), f32(bm)
            t[a + "attn_o.weight"], t[a + "attn_o.bias"] = _wt(cfg, w[e + "Wo"]), f32(w[e + "bo"])
            t[a + "ff0.weight"], t[a + "ff0.bias"] = _wt(cfg, w[e + "W1"]), f32(w[e + "b1"])
            t[a + "ff2.weight"], t[a + "ff2.bias"] = _wt(cfg, w[e + "W2"]), f32(w[e + "b2"])
    else:
        raise ValueError("no GGUF layout for arch %r" % cfg["arch"])
    write_gguf(path, kv, t)


def import_trace(lib, path):
    """Names of the GGUF tensors the library's checkpoint import reads from `path`, in order
    (vla_gguf_import_trace); raises when the file cannot be imported."""
    lib.vla_gguf_import_trace.restype = ctypes.c_int64
    lib.vla_gguf_import_trace.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int64]
    buf = ctypes.create_string_buffer(1 << 20)
    n = lib.vla_gguf_import_trace(path.encode(), buf, len(buf))
    if n < 0:
        raise RuntimeError("vla_gguf_import_trace returned %d" % n)
    return buf.value.decode().split("\n")[:-1]
