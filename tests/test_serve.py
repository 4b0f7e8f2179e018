"""Serving boundary (include/vla_serve.h): the proto3 codec against the protobuf runtime
built from the message definitions of the reference's src/serving/vla.proto (declared here
field by field, so the check does not depend on this library's own encoder), the server's
request checks, and several queued requests answered by batched engine calls."""
import ctypes
import os

import numpy as np
import pytest
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

from util import declared_symbols, pkg

from vla_cpp_amd import checkpoint as ckpt  # noqa: E402

F = descriptor_pb2.FieldDescriptorProto


def _messages():
    """vla.Image, vla.PredictRequest, vla.PredictResponse with the field numbers and types
    of src/serving/vla.proto."""
    fd = descriptor_pb2.FileDescriptorProto(name="vla_test.proto", package="vlatest", syntax="proto3")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, num, ftype, rep, tname in fields:
            f = m.field.add(name=fname, number=num, type=ftype, label=F.LABEL_REPEATED if rep else F.LABEL_OPTIONAL)
            if tname:
                f.type_name = tname
        return m

    img = msg("Image", [("encoding", 1, F.TYPE_ENUM, False, ".vlatest.Image.Encoding"), ("height", 2, F.TYPE_UINT32, False, None),
                        ("width", 3, F.TYPE_UINT32, False, None), ("data", 4, F.TYPE_BYTES, False, None)])
    en = img.enum_type.add(name="Encoding")
    for i, n in enumerate(("JPEG", "RGB_U8", "F32_RGB_01")):
        en.value.add(name=n, number=i)
    msg("PredictRequest", [("images", 1, F.TYPE_MESSAGE, True, ".vlatest.Image"), ("lang_tokens", 2, F.TYPE_INT32, True, None),
                           ("state", 3, F.TYPE_FLOAT, True, None), ("noise", 4, F.TYPE_FLOAT, True, None),
                           ("request_id", 5, F.TYPE_UINT64, False, None), ("precomputed_img_emb", 6, F.TYPE_FLOAT, True, None),
                           ("precomputed_img_emb_n_views", 7, F.TYPE_UINT32, False, None),
                           ("attention_mask", 8, F.TYPE_UINT32, True, None)])
    msg("PredictResponse", [("request_id", 1, F.TYPE_UINT64, False, None), ("action_chunk", 2, F.TYPE_FLOAT, True, None),
                            ("chunk_size", 3, F.TYPE_UINT32, False, None), ("action_dim", 4, F.TYPE_UINT32, False, None),
                            ("latency_ms_total", 5, F.TYPE_FLOAT, False, None), ("latency_ms_inference", 6, F.TYPE_FLOAT, False, None),
                            ("error", 7, F.TYPE_STRING, False, None), ("latency_ms_prefill", 8, F.TYPE_FLOAT, False, None),
                            ("latency_ms_denoise", 9, F.TYPE_FLOAT, False, None), ("latency_ms_vision", 10, F.TYPE_FLOAT, False, None)])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = lambda n: message_factory.GetMessageClass(pool.FindMessageTypeByName("vlatest." + n))
    return get("PredictRequest"), get("PredictResponse")


PredictRequest, PredictResponse = _messages()


class WireResponse(ctypes.Structure):
    _fields_ = [("request_id", ctypes.c_uint64), ("chunk_size", ctypes.c_uint32), ("action_dim", ctypes.c_uint32),
                ("latency_ms_total", ctypes.c_float), ("latency_ms_inference", ctypes.c_float), ("latency_ms_prefill", ctypes.c_float),
                ("latency_ms_denoise", ctypes.c_float), ("latency_ms_vision", ctypes.c_float), ("n_actions", ctypes.c_int64),
                ("error_len", ctypes.c_int64)]


def _lib():
    L = pkg.lib()
    L.vla_wire_encode_request.restype = ctypes.c_void_p
    L.vla_wire_encode_request.argtypes = [ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p,
                                          ctypes.c_int32, ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint32, ctypes.c_void_p]
    L.vla_wire_decode_response.restype = ctypes.c_int32
    L.vla_wire_decode_response.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                           ctypes.c_int64]
    L.vla_serve_free.restype = None
    L.vla_serve_free.argtypes = [ctypes.c_void_p]
    L.vla_serve_requests.restype = ctypes.c_int32
    L.vla_serve_requests.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    L.vla_model_n_actions.restype = ctypes.c_int64
    L.vla_model_n_actions.argtypes = [ctypes.c_void_p]
    return L


def encode_request(L, rid, lang, state, noise, emb, n_views):
    n = ctypes.c_int64()
    arr = lambda a, t: None if a is None else np.ascontiguousarray(a, t)
    lang, state, noise, emb = arr(lang, np.int32), arr(state, np.float32), arr(noise, np.float32), arr(emb, np.float32)
    p = lambda a: None if a is None else a.ctypes.data
    sz = lambda a: 0 if a is None else a.size
    f = L.vla_wire_encode_request(rid, p(lang), sz(lang), p(state), sz(state), p(noise), sz(noise), p(emb), sz(emb), n_views, ctypes.byref(n))
    assert f
    out = ctypes.string_at(f, n.value)
    L.vla_serve_free(f)
    return out


def decode_response(L, frame):
    r = WireResponse()
    if L.vla_wire_decode_response(frame, len(frame), ctypes.byref(r), None, 0, None, 0) != 0:
        return None
    act = np.empty(r.n_actions, np.float32)
    err = ctypes.create_string_buffer(r.error_len + 1)
    assert L.vla_wire_decode_response(frame, len(frame), ctypes.byref(r), act.ctypes.data, act.size, err, r.error_len + 1) == 0
    return r, act, err.raw[:r.error_len].decode()


def test_header_symbols_are_exported():
    names = declared_symbols("vla_serve.h")
    assert set(names) == {"vla_serve_requests", "vla_serve_free", "vla_wire_encode_request", "vla_wire_decode_response",
                          "vla_model_n_actions"}
    for n in names:
        assert hasattr(pkg.lib(), n)


def test_request_encoder_gives_the_protobuf_runtime_bytes():
    L = _lib()
    r = np.random.default_rng(1)
    lang = np.int32([5, 0, 300, 2 ** 31 - 1, 17])
    state, noise, emb = (r.standard_normal(n).astype(np.float32) for n in (32, 50 * 32, 2 * 64 * 96))
    state[3] = -0.0
    for rid, nz, views in ((0, None, 2), (2 ** 63 + 12345, noise, 2), (7, noise, 0)):
        mine = encode_request(L, rid, lang, state, nz, emb, views)
        q = PredictRequest(lang_tokens=lang.tolist(), state=state.tolist(), noise=[] if nz is None else nz.tolist(), request_id=rid,
                           precomputed_img_emb=emb.tolist(), precomputed_img_emb_n_views=views)
        assert mine == q.SerializeToString(deterministic=True)
        back = PredictRequest.FromString(mine)
        assert list(back.lang_tokens) == lang.tolist() and back.request_id == rid
        assert np.array_equal(np.float32(back.state).view(np.uint32), state.view(np.uint32))


def test_response_decoder_reads_protobuf_runtime_frames():
    L = _lib()
    act = np.random.default_rng(2).standard_normal(50 * 32).astype(np.float32)
    resp = PredictResponse(request_id=99, action_chunk=act.tolist(), chunk_size=50, action_dim=32, latency_ms_total=12.5,
                           latency_ms_inference=11.25, latency_ms_prefill=3.5, latency_ms_denoise=7.75)
    r, got, err = decode_response(L, resp.SerializeToString())
    assert (r.request_id, r.chunk_size, r.action_dim, r.n_actions, err) == (99, 50, 32, act.size, "")
    assert np.array_equal(got, act) and (r.latency_ms_total, r.latency_ms_prefill, r.latency_ms_vision) == (12.5, 3.5, 0.0)
    r, got, err = decode_response(L, PredictResponse(request_id=3, error="state length 31 != expected 32").SerializeToString())
    assert r.request_id == 3 and got.size == 0 and err == "state length 31 != expected 32"
    r, got, err = decode_response(L, b"")  # every field at its default
    assert (r.request_id, r.n_actions, err) == (0, 0, "")
    # malformed frames: truncated varint / length past the end / wrong wire type for a known field
    frame = resp.SerializeToString()
    assert decode_response(L, frame[:-3]) is None and decode_response(L, b"\x12\xff\xff\x03abc") is None
    assert decode_response(L, b"\x0d\x00\x00\x00\x00") is None  # request_id as fixed32
    # unknown fields are skipped; unpacked repeated floats are accepted
    unpacked = b"\x15" + np.float32(1.5).tobytes() + b"\x15" + np.float32(-2.0).tobytes() + b"\xa0\x06\x07" + b"\x08\x05"
    r, got, err = decode_response(L, unpacked)
    assert got.tolist() == [1.5, -2.0] and r.request_id == 5


# ------------------------------------------------------------------ batched serving on the GPU
@pytest.mark.gpu
def test_queued_requests_are_answered_in_batches_with_the_servers_checks(tmp_path):
    from test_gpu_chunk import make_obs
    from vla_cpp_amd import ffi
    L = _lib()
    cfg = ckpt.smolvla_config(n_layers=4, dtype="bf16", suffix_mask=1)
    w = ckpt.synth_weights(cfg, seed=0x5EED + 31)
    path = os.path.join(str(tmp_path), "serve.vlaw")
    ckpt.write_synthetic(path, cfg, w)
    m = ffi.Model(path)
    assert L.vla_model_n_actions(m._h) == 50
    r = np.random.default_rng(340)
    # five good requests in two shapes (2 views / 48 tokens x3, 1 view / 20 tokens x2) and the bad ones between them
    obs = [make_obs(cfg, r, n_views=2) for _ in range(3)] + [make_obs(cfg, r, n_views=1, n_lang=20) for _ in range(2)]
    want = [m.predict_batch([o]).reshape(50, 32) for o in obs]

    def frame(o, rid, **over):
        d = dict(lang=o["lang"], state=o["state"], noise=o["noise"], emb=o["img_emb"], n_views=o["n_views"])
        d.update(over)
        return PredictRequest(lang_tokens=np.asarray(d["lang"]).tolist(), state=np.asarray(d["state"]).ravel().tolist(),
                              noise=[] if d["noise"] is None else np.asarray(d["noise"]).ravel().tolist(), request_id=rid,
                              precomputed_img_emb=np.asarray(d["emb"]).ravel().tolist(),
                              precomputed_img_emb_n_views=d["n_views"]).SerializeToString()

    nan_state = obs[0]["state"].copy()
    nan_state[4] = np.nan
    frames = [
        frame(obs[0], 100), frame(obs[3], 101),
        frame(obs[0], 102, state=obs[0]["state"][:31]),            # wrong state length
        frame(obs[1], 103),
        b"\x12\xff\xff\xff\x0f",                                  # not a message
        frame(obs[4], 105), frame(obs[2], 106),
        frame(obs[0], 107, lang=[3, -2, 5]),                       # negative token
        frame(obs[0], 108, n_views=3),                             # embedding size does not match the views
        frame(obs[0], 109, state=nan_state),
        frame(obs[0], 110, noise=obs[0]["noise"].ravel()[:100]),
        PredictRequest(request_id=111, lang_tokens=[1], state=obs[0]["state"].tolist()).SerializeToString(),  # no image input at all
        frame(obs[0], 112, lang=np.zeros(49, np.int32)),           # longer than tokenizer_max_length
        # passes the wire checks, is rejected by the engine (token outside the vocabulary): it shares
        # the (2 views, 48 tokens) batch with frames 0, 3 and 6, which must still be served
        frame(obs[0], 113, lang=np.full(48, cfg["vocab"] + 7, np.int32)),
    ]
    n = len(frames)
    bufs = [ctypes.create_string_buffer(f, len(f)) for f in frames]
    req = (ctypes.c_void_p * n)(*[ctypes.cast(b, ctypes.c_void_p) for b in bufs])
    lens = (ctypes.c_int64 * n)(*[len(f) for f in frames])
    resp = (ctypes.c_void_p * n)()
    rlen = (ctypes.c_int64 * n)()
    assert L.vla_serve_requests(m._h, n, req, lens, resp, rlen) == 0
    out = []
    for i in range(n):
        raw = ctypes.string_at(resp[i], rlen[i])
        out.append(PredictResponse.FromString(raw))      # the protobuf runtime reads every reply
        L.vla_serve_free(resp[i])
    good = {0: 0, 1: 3, 3: 1, 5: 4, 6: 2}                 # frame index -> observation
    for i, o in good.items():
        p = out[i]
        assert p.error == "" and p.request_id == 100 + i and (p.chunk_size, p.action_dim) == (50, 32)
        got = np.float32(p.action_chunk).reshape(50, 32)
        # batched with other requests: bf16 results do not depend on the batch (same kernels per row)
        assert np.array_equal(got, want[o])
        assert p.latency_ms_total > 0 and abs(p.latency_ms_prefill + p.latency_ms_denoise - p.latency_ms_total) < 1e-3
    errs = {2: "state length 31 != expected 32", 4: "request parse failed", 7: "lang_tokens[1] = -2 is negative",
            8: "precomputed_img_emb size %d != %d (n_views=3 * n_img_per_view=64 * hidden=960)" % (2 * 64 * 960, 3 * 64 * 960),
            9: "state[4] = nan is not finite (NaN/Inf)", 10: "noise length 100 != 0 or 1600 (chunk_size * action_dim)",
            11: "PredictRequest must contain images or precomputed_img_emb", 12: "lang_tokens length 49 out of range [1, 48]",
            13: "predict failed"}
    for i, text in errs.items():
        assert out[i].error == text and len(out[i].action_chunk) == 0, (i, out[i].error)
        assert out[i].request_id == (0 if i == 4 else 100 + i)
    # no requests, NULL handle
    assert L.vla_serve_requests(m._h, 0, None, None, None, None) == 0
    assert L.vla_serve_requests(None, 1, req, lens, resp, rlen) == -1
    m.close()
