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


def one_ulp_noise(x, r, frac=0.01):
    """x (fp32 values that are bf16-representable) with `frac` of its elements moved to a
    neighbouring bf16 value: the probe that measures how far a quantised network moves under
    the smallest possible input difference.  Stays finite; zero moves to the smallest positive."""
    import oracle as orc
    b = orc.to_bf16(x).astype(np.int32).ravel()
    idx = r.choice(b.size, max(1, int(frac * b.size)), replace=False)
    mag = np.clip((b[idx] & 0x7fff) + r.choice(np.int32([-1, 1]), idx.size), 0, 0x7f7f)
    b[idx] = (b[idx] & 0x8000) | mag
    return orc.from_bf16(b.astype(np.uint16).reshape(np.shape(x)))
