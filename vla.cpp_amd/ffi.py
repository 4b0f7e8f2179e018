"""ctypes mirror of include/vla.h (ABI v1 structs and entry points) plus the batch /
phase-split extensions.  Field order and types follow the header exactly (the
reference's bindings do the same against its header,
bindings/python/vla_cpp/_ffi.py:124-163); tests/test_abi_cpu.py checks them
against the header text."""
import ctypes

import numpy as np

from . import lib

ABI_VERSION = 1
VLA_OK, VLA_ERR_ARG, VLA_ERR_PREDICT, VLA_ERR_EXCEPTION = 0, -1, -2, -3

_i32, _i64, _f32, _f64 = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_double


class Config(ctypes.Structure):
    _fields_ = [
        ("n_img", _i64), ("n_lang", _i64), ("n_state", _i64), ("n_prefix", _i64), ("n_suffix", _i64), ("n_full", _i64),
        ("hidden", _i64), ("expert_h", _i64), ("intermediate", _i64), ("expert_inter", _i64),
        ("n_q_heads", _i64), ("n_kv_heads", _i64), ("head_dim", _i64), ("q_full_dim", _i64), ("kv_full_dim", _i64),
        ("n_layers", _i64), ("self_attn_every_n", _i32),
        ("max_state_dim", _i64), ("max_action_dim", _i64), ("real_state_dim", _i64), ("real_action_dim", _i64),
        ("norm_eps", _f32), ("min_period", _f64), ("max_period", _f64), ("num_steps", _i32),
        ("rms_eps", _f32), ("rope_n_dims", _i32), ("rope_mode", _i32), ("rope_freq_base", _f32),
        ("denormalized", _i32),
    ]


class Image(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("w", _i32), ("h", _i32), ("format", _i32)]


class Inputs(ctypes.Structure):
    _fields_ = [
        ("images", ctypes.POINTER(Image)), ("n_images", _i32),
        ("precomputed_img_emb", ctypes.POINTER(_f32)), ("n_img_views", _i32),
        ("lang_tokens", ctypes.POINTER(_i32)), ("n_lang", _i32),
        ("state", ctypes.POINTER(_f32)), ("noise", ctypes.POINTER(_f32)),
        ("attention_mask", ctypes.POINTER(_i32)), ("attention_mask_n", _i32),
        ("timing_detail", _i32),
    ]


class Stats(ctypes.Structure):
    _fields_ = [("ms_total", _f32), ("ms_vision", _f32), ("ms_inference", _f32), ("ms_prefill", _f32),
                ("ms_denoise", _f32)]


_bound = False


def _bind():
    global _bound
    L = lib()
    if _bound:
        return L
    L.vla_abi_version.restype = _i32
    L.vla_model_load.restype = ctypes.c_void_p
    L.vla_model_load.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p]
    L.vla_model_free.argtypes = [ctypes.c_void_p]
    L.vla_model_free.restype = None
    L.vla_model_config.argtypes = [ctypes.c_void_p, ctypes.POINTER(Config)]
    L.vla_predict.argtypes = [ctypes.c_void_p, ctypes.POINTER(Inputs), ctypes.POINTER(ctypes.POINTER(_f32)),
                              ctypes.POINTER(_i64)]
    L.vla_free_actions.argtypes = [ctypes.POINTER(_f32)]
    L.vla_free_actions.restype = None
    L.vla_last_stats.argtypes = [ctypes.c_void_p, ctypes.POINTER(Stats)]
    L.vla_prefill_batch.argtypes = [ctypes.c_void_p, ctypes.POINTER(Inputs), _i32]
    L.vla_denoise_async.argtypes = [ctypes.c_void_p, _i32, ctypes.c_void_p]
    L.vla_denoise_steps_async.argtypes = [ctypes.c_void_p, _i32, ctypes.c_void_p]
    L.vla_fetch_actions.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.POINTER(_f32)), ctypes.POINTER(_i64)]
    L.vla_predict_batch.argtypes = [ctypes.c_void_p, ctypes.POINTER(Inputs), _i32,
                                    ctypes.POINTER(ctypes.POINTER(_f32)), ctypes.POINTER(_i64)]
    L.vla_profile_begin.argtypes = [ctypes.c_void_p]
    L.vla_profile_end.argtypes = [ctypes.c_void_p, ctypes.c_char_p, _i64]
    L.vla_profile_end.restype = _i64
    _bound = True
    return L


def _fp(a):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(_f32))


def make_inputs(obs_list):
    """obs_list: dicts with img_emb [views*n_img, hidden] f32, n_views, lang (int32 array or None),
    state (f32 or None), noise (f32 or None).  Returns (ctypes array, keepalive list)."""
    arr = (Inputs * len(obs_list))()
    keep = []
    for i, o in enumerate(obs_list):
        img = np.ascontiguousarray(o["img_emb"], np.float32)
        lang = None if o.get("lang") is None else np.ascontiguousarray(o["lang"], np.int32)
        state = None if o.get("state") is None else np.ascontiguousarray(o["state"], np.float32)
        noise = None if o.get("noise") is None else np.ascontiguousarray(o["noise"], np.float32)
        keep += [img, lang, state, noise]
        arr[i].precomputed_img_emb = _fp(img)
        arr[i].n_img_views = int(o["n_views"])
        arr[i].lang_tokens = None if lang is None else lang.ctypes.data_as(ctypes.POINTER(_i32))
        arr[i].n_lang = 0 if lang is None else lang.size
        arr[i].state = _fp(state)
        arr[i].noise = _fp(noise)
        arr[i].timing_detail = int(o.get("timing_detail", 0))
    return arr, keep


class Model:
    """Handle over vla_model_load / vla_predict and the batch extensions."""

    def __init__(self, ckpt_path):
        self._L = _bind()
        self._h = self._L.vla_model_load(None, ckpt_path.encode(), None)
        if not self._h:
            raise RuntimeError("vla_model_load failed for %s" % ckpt_path)

    def close(self):
        if self._h:
            self._L.vla_model_free(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def config(self):
        c = Config()
        assert self._L.vla_model_config(self._h, ctypes.byref(c)) == VLA_OK
        return c

    def stats(self):
        s = Stats()
        assert self._L.vla_last_stats(self._h, ctypes.byref(s)) == VLA_OK
        return s

    def _take(self, p, n):
        out = np.ctypeslib.as_array(p, shape=(n.value,)).copy()
        self._L.vla_free_actions(p)
        return out

    def predict(self, obs):
        arr, keep = make_inputs([obs])
        p, n = ctypes.POINTER(_f32)(), _i64()
        rc = self._L.vla_predict(self._h, arr, ctypes.byref(p), ctypes.byref(n))
        if rc != VLA_OK:
            raise RuntimeError("vla_predict returned %d" % rc)
        return self._take(p, n)

    def prefill_batch(self, obs_list):
        arr, keep = make_inputs(obs_list)
        rc = self._L.vla_prefill_batch(self._h, arr, len(obs_list))
        if rc != VLA_OK:
            raise RuntimeError("vla_prefill_batch returned %d" % rc)

    def denoise_async(self, chunks=1, stream=None):
        rc = self._L.vla_denoise_async(self._h, chunks, stream)
        if rc != VLA_OK:
            raise RuntimeError("vla_denoise_async returned %d" % rc)

    def denoise_steps_async(self, n_steps, stream=None):
        rc = self._L.vla_denoise_steps_async(self._h, n_steps, stream)
        if rc != VLA_OK:
            raise RuntimeError("vla_denoise_steps_async returned %d" % rc)

    def fetch(self):
        p, n = ctypes.POINTER(_f32)(), _i64()
        rc = self._L.vla_fetch_actions(self._h, ctypes.byref(p), ctypes.byref(n))
        if rc != VLA_OK:
            raise RuntimeError("vla_fetch_actions returned %d" % rc)
        return self._take(p, n)

    def profile_begin(self):
        assert self._L.vla_profile_begin(self._h) == VLA_OK

    def profile_end(self):
        """{"phase.label": {"us": ..., "launches": ...}} for the launches since profile_begin()."""
        import json
        buf = ctypes.create_string_buffer(1 << 12)
        n = self._L.vla_profile_end(self._h, buf, len(buf))
        if n < -16:  # too small: the profile is kept, the size needed is -16 - n
            buf = ctypes.create_string_buffer(-16 - n)
            n = self._L.vla_profile_end(self._h, buf, len(buf))
        if n < 0:
            raise RuntimeError("vla_profile_end returned %d" % n)
        return json.loads(buf.value.decode())

    def predict_batch(self, obs_list):
        self.prefill_batch(obs_list)
        self.denoise_async(1, None)
        return self.fetch()
