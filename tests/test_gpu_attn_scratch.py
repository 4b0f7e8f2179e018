"""Scratch-memory ownership of the attention entry points.

A call whose keys are sliced across workgroups needs device memory beyond its inputs and
outputs.  vla_attn_prefix_suffix keeps blocks per stream, vla_attn_prefix_suffix_ws takes the
caller's block (what a model handle uses).  Both run the same kernels, so the results are
bit-identical, and two model handles in one process never touch each other's scratch: the
reference's contract is one call at a time per handle (include/vla.h:18-19), not per process.
"""
import os

import numpy as np
import pytest
import torch

import oracle as orc
from util import pkg

pytestmark = pytest.mark.gpu

from vla_cpp_amd import checkpoint as ckpt  # noqa: E402
from vla_cpp_amd import ffi  # noqa: E402

BF16 = pkg.VLA_DT_BF16

# (name, B, S, Hq, Hkv, D, T, dtype, mask): shapes that take each sliced dispatch
SLICED = [
    ("decode-arrive", 8, 1, 20, 5, 128, 519, pkg.VLA_DT_BF16_P2, pkg.VLA_MASK_NONE),
    ("decode-merge-kernel", 2, 5, 6, 2, 64, 2100, BF16, pkg.VLA_MASK_NONE),
    ("pi0-wide-fp16-partials", 1, 51, 8, 1, 256, 867, BF16, pkg.VLA_MASK_PI0_STATE),
    ("fp32-lds-split", 2, 5, 6, 2, 64, 600, pkg.VLA_DT_F32, pkg.VLA_MASK_CAUSAL_SUFFIX),
]


def bf(a, dt=BF16):
    if dt == pkg.VLA_DT_F32:
        return torch.from_numpy(np.ascontiguousarray(a, np.float32)).cuda().contiguous()
    return torch.from_numpy(orc.to_bf16(a).view(np.int16)).cuda().contiguous()


def setup_case(case, seed=0):
    name, B, S, Hq, Hkv, D, T, dt, mk = case
    r = np.random.default_rng(4000 + seed + T)
    t_max = (T + 63) // 64 * 64
    Q = r.standard_normal((B, S, Hq, D)).astype(np.float32)
    K = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    V = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    st = pkg.VLA_DT_F32 if dt == pkg.VLA_DT_F32 else BF16  # storage type
    tt = torch.float32 if dt == pkg.VLA_DT_F32 else torch.int16
    kc = torch.zeros((B, Hkv, t_max, D), dtype=tt, device="cuda")
    vc = torch.zeros((B, Hkv, D, t_max), dtype=tt, device="cuda")
    pkg.call("vla_kv_append", kc, vc, bf(K, st), bf(V, st), st, B, Hkv, D, t_max, 0, T)
    return bf(Q, st), kc, vc, t_max


def run(entry, case, q, kc, vc, t_max, extra=()):
    name, B, S, Hq, Hkv, D, T, dt, mk = case
    out = torch.zeros((B, S, Hq * D), dtype=torch.float32 if dt == pkg.VLA_DT_F32 else torch.int16, device="cuda")
    P = T - S if mk != pkg.VLA_MASK_NONE else T
    fn = getattr(pkg.lib(), entry)
    rc = fn(pkg.ptr(q), pkg.ptr(kc), pkg.ptr(vc), pkg.ptr(out), dt, B, S, Hq, Hkv, D, t_max, T, 1.0 / np.sqrt(D), mk, P, 0, 0,
            None, *extra, pkg.stream())
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


@pytest.mark.parametrize("case", SLICED, ids=[c[0] for c in SLICED])
def test_caller_owned_workspace_gives_the_library_owned_bits(case):
    name, B, S, Hq, Hkv, D, T, dt, mk = case
    need = pkg.lib().vla_attn_workspace_bytes(dt, B, S, Hq, Hkv, D, T)
    assert need > 0, "the case is meant to need scratch memory"
    q, kc, vc, t_max = setup_case(case)
    rc, want = run("vla_attn_prefix_suffix", case, q, kc, vc, t_max)
    assert rc == pkg.VLA_K_OK and np.any(want)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    for _ in range(3):  # the part that must stay zero is left at zero by every launch
        rc, got = run("vla_attn_prefix_suffix_ws", case, q, kc, vc, t_max, (ws.data_ptr(), need))
        assert rc == pkg.VLA_K_OK and np.array_equal(got, want)
    # too small, or missing: refused before anything is launched
    rc, got = run("vla_attn_prefix_suffix_ws", case, q, kc, vc, t_max, (ws.data_ptr(), need - 256))
    assert rc == pkg.VLA_K_ERR_WORKSPACE and not np.any(got)
    rc, got = run("vla_attn_prefix_suffix_ws", case, q, kc, vc, t_max, (None, 0))
    assert rc == pkg.VLA_K_ERR_WORKSPACE and not np.any(got)


def test_workspace_reset_restores_counters_left_behind_by_a_launch_that_did_not_finish():
    """The slices of the decode shape count themselves in and the last one merges; the counters are
    left at zero by a launch that ran to its end.  Counters as a launch cut short would leave them
    (written here by the host, no kernel is interrupted) are put back by vla_attn_workspace_reset,
    and the next launch gives the usual bits."""
    case = SLICED[0]
    name, B, S, Hq, Hkv, D, T, dt, mk = case
    need = pkg.lib().vla_attn_workspace_bytes(dt, B, S, Hq, Hkv, D, T)
    q, kc, vc, t_max = setup_case(case)
    rc, want = run("vla_attn_prefix_suffix", case, q, kc, vc, t_max)
    assert rc == pkg.VLA_K_OK
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    rc, got = run("vla_attn_prefix_suffix_ws", case, q, kc, vc, t_max, (ws.data_ptr(), need))
    assert rc == pkg.VLA_K_OK and np.array_equal(got, want)
    ws.view(torch.int32)[:4096] = 3  # units that had counted three slices in when their launch ended
    torch.cuda.synchronize()
    lib = pkg.lib()
    assert lib.vla_attn_workspace_reset(ws.data_ptr(), need, pkg.stream()) == pkg.VLA_K_OK
    torch.cuda.synchronize()
    assert int(ws.view(torch.int32)[:16384].abs().sum()) == 0
    rc, got = run("vla_attn_prefix_suffix_ws", case, q, kc, vc, t_max, (ws.data_ptr(), need))
    assert rc == pkg.VLA_K_OK and np.array_equal(got, want)
    # nothing to do for a shape without a workspace; a block too small to hold the counters is refused
    assert lib.vla_attn_workspace_reset(None, 0, pkg.stream()) == pkg.VLA_K_OK
    assert lib.vla_attn_workspace_reset(ws.data_ptr(), 1024, pkg.stream()) == pkg.VLA_K_ERR_WORKSPACE
    assert lib.vla_attn_workspace_reset(ws.data_ptr() + 4, need - 4, pkg.stream()) == pkg.VLA_K_ERR_WORKSPACE


def test_shapes_without_key_slices_need_no_workspace():
    # batch 32 SmolVLA: enough workgroups without slicing; NULL workspace is accepted
    case = ("smolvla-b32", 32, 50, 15, 5, 64, 291, BF16, pkg.VLA_MASK_NONE)
    assert pkg.lib().vla_attn_workspace_bytes(BF16, 32, 50, 15, 5, 64, 291) == 0
    q, kc, vc, t_max = setup_case(case)
    rc, want = run("vla_attn_prefix_suffix", case, q, kc, vc, t_max)
    rc2, got = run("vla_attn_prefix_suffix_ws", case, q, kc, vc, t_max, (None, 0))
    assert rc == rc2 == pkg.VLA_K_OK and np.array_equal(got, want)


def test_library_blocks_are_per_stream_and_survive_growth():
    # a small sliced shape, then a larger one on the same stream (the block grows; the old one
    # stays allocated), then the small one again, and the small one on a second stream
    small, big = SLICED[3], SLICED[2]
    qs, ks, vs, ts = setup_case(small)
    qb, kb, vb, tb = setup_case(big)
    _, want_s = run("vla_attn_prefix_suffix", small, qs, ks, vs, ts)
    _, want_b = run("vla_attn_prefix_suffix", big, qb, kb, vb, tb)
    _, again = run("vla_attn_prefix_suffix", small, qs, ks, vs, ts)
    assert np.array_equal(again, want_s)
    s2 = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(s2):
        _, other = run("vla_attn_prefix_suffix", small, qs, ks, vs, ts)
        _, other_b = run("vla_attn_prefix_suffix", big, qb, kb, vb, tb)
    assert np.array_equal(other, want_s) and np.array_equal(other_b, want_b)


def _load(tmp_path, cfg, w, name):
    path = os.path.join(str(tmp_path), name + ".vlaw")
    ckpt.write_synthetic(path, cfg, w)
    return ffi.Model(path)


def _obs(cfg, r, n_views):
    A = cfg["max_action_dim"]
    n_act = cfg["n_suffix"] - 1
    o = dict(img_emb=r.standard_normal((n_views * cfg["n_img"], cfg["hidden"])).astype(np.float32), n_views=n_views,
             noise=r.standard_normal((n_act, A)).astype(np.float32), lang=r.integers(0, cfg["vocab"], cfg["n_lang"]).astype(np.int32),
             state=r.standard_normal(cfg["max_state_dim"]).astype(np.float32))
    return o


def test_two_handles_with_different_scratch_needs_do_not_disturb_each_other(tmp_path):
    # pi0 at batch 1 (seven key slices) and a second handle at batch 4 whose partial rows need
    # a larger block: each handle replays its captured chunk; alternating them three times
    # gives, every time, the bits each gives alone.
    cfg = ckpt.pi0_config(n_layers=3)
    w = ckpt.synth_weights(cfg, seed=77)
    r = np.random.default_rng(78)
    obs1 = [_obs(cfg, r, 3)]
    obs4 = [_obs(cfg, r, 3) for _ in range(4)]
    a = _load(tmp_path, cfg, w, "a")
    alone_a = [a.predict_batch(obs1) for _ in range(3)]  # eager, capture, replay
    assert np.array_equal(alone_a[0], alone_a[1]) and np.array_equal(alone_a[0], alone_a[2])
    a.close()
    b = _load(tmp_path, cfg, w, "b")
    alone_b = [b.predict_batch(obs4) for _ in range(3)]
    assert np.array_equal(alone_b[0], alone_b[2])
    b.close()
    a, b = _load(tmp_path, cfg, w, "a"), _load(tmp_path, cfg, w, "b")
    for _ in range(3):
        assert np.array_equal(a.predict_batch(obs1), alone_a[0])
        assert np.array_equal(b.predict_batch(obs4), alone_b[0])
    # freeing one handle leaves the other's graph intact
    b.close()
    assert np.array_equal(a.predict_batch(obs1), alone_a[0])
    a.close()
