"""vla_attn_prefix_suffix_noalloc: the attention entry point for callers that cannot allocate.

Its scratch memory is a fixed device array inside the library; it runs the kernels of
vla_attn_prefix_suffix, so its output is held to that entry point's, bit for bit, on shapes
that take each sliced dispatch -- two calls in a row, the second with a smaller input, since
every call on a GPU shares the one array and finds the last call's contents in it.
"""
import numpy as np
import pytest
import torch

from util import pkg
from test_gpu_attn_scratch import SLICED, run, setup_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("first,second", [(SLICED[0], ("decode-arrive-small", 3, 1, 20, 5, 128, 400, pkg.VLA_DT_BF16_P2, pkg.VLA_MASK_NONE)),
                                          (SLICED[2], SLICED[3]), (SLICED[1], SLICED[0])],
                         ids=["arrive-merge", "lds-split", "merge-kernel-then-arrive"])
def test_no_alloc_entry_point_matches_the_allocating_one(first, second):
    assert pkg.lib().vla_kernels_init() == pkg.VLA_K_OK
    for case in (first, second, first):
        name, B, S, Hq, Hkv, D, T, dt, mk = case
        assert 0 < pkg.lib().vla_attn_workspace_bytes(dt, B, S, Hq, Hkv, D, T) <= (64 << 10) + (16 << 20)
        q, kc, vc, t_max = setup_case(case, seed=11)
        rc, want = run("vla_attn_prefix_suffix", case, q, kc, vc, t_max)
        assert rc == pkg.VLA_K_OK and np.any(want)
        free_before = torch.cuda.mem_get_info()[0]
        rc, got = run("vla_attn_prefix_suffix_noalloc", case, q, kc, vc, t_max)
        assert rc == pkg.VLA_K_OK and np.array_equal(got, want), name
        rc, got = run("vla_attn_prefix_suffix_noalloc", case, q, kc, vc, t_max)
        assert rc == pkg.VLA_K_OK and np.array_equal(got, want), name
        # free device memory did not shrink (the output tensor of run() comes from torch's cache after the first call)
        assert torch.cuda.mem_get_info()[0] >= free_before


@pytest.mark.parametrize("case", [SLICED[0], SLICED[2], SLICED[1]], ids=["arrive-merge", "lds-split", "merge-kernel"])
def test_no_alloc_entry_point_runs_under_global_stream_capture(case):
    # The structural check: the call is recorded into a HIP graph in global capture mode, on a stream
    # that has never seen the shape.  hipMalloc, hipFree and synchronous hipMemset are refused in that
    # mode and would fail the capture; the graph is then replayed several times, with eager work of
    # the same entry point (on other inputs) and synchronisations between the replays, and every
    # replay gives the allocating entry point's bits (no memset node, no stale counter).
    assert pkg.lib().vla_kernels_init() == pkg.VLA_K_OK
    name, B, S, Hq, Hkv, D, T, dt, mk = case
    q, kc, vc, t_max = setup_case(case, seed=23)
    q2, kc2, vc2, _ = setup_case(case, seed=24)
    rc, want = run("vla_attn_prefix_suffix", case, q, kc, vc, t_max)
    assert rc == pkg.VLA_K_OK and np.any(want)
    out = torch.zeros((B, S, Hq * D), dtype=torch.float32 if dt == pkg.VLA_DT_F32 else torch.int16, device="cuda")
    P = T - S if mk != pkg.VLA_MASK_NONE else T
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side, capture_error_mode="global"):
        rc = pkg.lib().vla_attn_prefix_suffix_noalloc(pkg.ptr(q), pkg.ptr(kc), pkg.ptr(vc), pkg.ptr(out), dt, B, S, Hq, Hkv, D, t_max, T,
                                                      1.0 / np.sqrt(D), mk, P, 0, 0, None, pkg.stream())
    assert rc == pkg.VLA_K_OK
    for i in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want), (name, i)
        rc, _ = run("vla_attn_prefix_suffix_noalloc", case, q2, kc2, vc2, t_max)  # eager use of the same array in between
        assert rc == pkg.VLA_K_OK


def test_no_alloc_entry_point_refuses_what_does_not_fit():
    # pi0 at batch 16: four key slices of 512 padded rows per observation, 33 MB of partials
    case = ("pi0-b16", 16, 51, 8, 1, 256, 867, pkg.VLA_DT_BF16, pkg.VLA_MASK_PI0_STATE)
    assert pkg.lib().vla_attn_workspace_bytes(pkg.VLA_DT_BF16, 16, 51, 8, 1, 256, 867) > (64 << 10) + (16 << 20)
    q, kc, vc, t_max = setup_case(case)
    rc, got = run("vla_attn_prefix_suffix_noalloc", case, q, kc, vc, t_max)
    assert rc == pkg.VLA_K_ERR_WORKSPACE and not np.any(got)
    # shapes that need no scratch at all are accepted whatever their size
    case = ("smolvla-b32", 32, 50, 15, 5, 64, 291, pkg.VLA_DT_BF16, pkg.VLA_MASK_NONE)
    q, kc, vc, t_max = setup_case(case)
    rc, want = run("vla_attn_prefix_suffix", case, q, kc, vc, t_max)
    rc2, got = run("vla_attn_prefix_suffix_noalloc", case, q, kc, vc, t_max)
    assert rc == rc2 == pkg.VLA_K_OK and np.array_equal(got, want)
