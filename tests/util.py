"""Helpers shared by the GPU parity tests: package loader, tensor movers, error norms."""
import os
import re
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

pkg = entry.load_package()


def dev(a):
    """numpy -> contiguous cuda tensor (uint16 arrays are carried as int16 bit patterns)."""
    import torch
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().contiguous()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda().contiguous()
    return torch.from_numpy(a).cuda().contiguous()


def host(t, dtype=None):
    a = t.detach().cpu().numpy()
    if dtype is not None:
        a = a.view(dtype)
    return a


def rel_err(got, want):
    """max |got - want| / max |want|: the relative measure used for the fp tolerances."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(?:VLA_KAPI|VLA_API|VLA_GGUF_API|VLA_SERVE_API)\s+[\w\s\*]+?\b(\w+)\s*\(", text)))
