"""CPU-side checks of the C-ABI library: it loads, exports every declared
symbol, and its host-only helpers (no GPU needed) agree with the oracle."""
import ctypes
import os

import numpy as np
import pytest

import oracle as orc
from util import ROOT, declared_symbols, pkg


def test_library_exports_every_declared_kernel_symbol():
    lib = pkg.lib()
    names = declared_symbols("vla_kernels.h")
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), "libvla.so does not export %s" % n
    assert set(names) == set(pkg.KERNEL_API), "ctypes table and header disagree"
    assert lib.vla_kernels_arch() == b"gfx950"


def test_rope_tables_host_equals_oracle_tables():
    lib = pkg.lib()
    pos = np.int32([0, 1, 49, 241, 290, 866])
    for D, base in ((64, 10000.0), (256, 10000.0), (128, 500000.0)):
        c = np.empty((pos.size, D // 2), np.float32)
        s = np.empty_like(c)
        assert lib.vla_rope_tables_host(pos.ctypes.data, pos.size, D, base, c.ctypes.data, s.ctypes.data) == 0
        oc, os_ = orc.rope_tables(pos, D, base)
        assert np.array_equal(c, oc) and np.array_equal(s, os_)
    assert lib.vla_rope_tables_host(pos.ctypes.data, pos.size, 63, 1e4, c.ctypes.data, s.ctypes.data) == pkg.VLA_K_ERR_ARG


def test_ternary_quant_and_packers_against_oracle():
    lib = pkg.lib()
    r = np.random.default_rng(21)
    N, K = 64, 256
    W = (r.standard_normal((N, K)) * 0.02).astype(np.float32)
    t = np.empty((N, K), np.int8)
    am = ctypes.c_float()
    assert lib.vla_ternary_quant_host(W.ctypes.data, W.size, t.ctypes.data, ctypes.addressof(am)) == 0
    ot, oam = orc.weight_quant_ternary(W)
    assert np.array_equal(t, ot) and np.float32(am.value) == oam
    # packing: word (n, w) decodes (reference decode) to the 16 values k = 16w..16w+15
    nwords = lib.vla_ternary_packed_words(N, K)
    assert nwords == N * K // 16 and lib.vla_ternary_packed_words(48, K) == 64 * K // 16
    packed = np.empty(nwords, np.uint32)
    assert lib.vla_ternary_pack_host(t.ctypes.data, N, K, packed.ctypes.data) == 0
    word = lambda buf, n, w: buf[pkg.tern_word_index(n, w, K)]
    for n, w in ((0, 0), (5, 3), (63, 15), (33, 1), (31, 14)):
        assert np.array_equal(orc.decode_i2s_to_i8s(word(packed, n, w)), t[n, 16 * w:16 * w + 16])
    # the 64 words of one (32-column block, 32-k group) are contiguous, [k half][column]
    assert pkg.tern_word_index(32, 2, K) == (1 * (K // 32) + 1) * 64
    assert pkg.tern_word_index(32 + 7, 3, K) == (1 * (K // 32) + 1) * 64 + 32 + 7
    # ladder -> gfx950 repack is a word permutation that inverts the reference's swizzle
    ladder = orc.pack_ladder_int2(t)
    rep = np.empty_like(packed)
    assert lib.vla_ternary_repack_ladder_host(ladder.ctypes.data, N, K, rep.ctypes.data) == 0
    assert np.array_equal(rep, packed)
    # raw ladder bytes (code 0 -> -2 allowed) survive the repack too
    raw = r.integers(0, 256, N * K // 4).astype(np.uint8)
    assert lib.vla_ternary_repack_ladder_host(raw.ctypes.data, N, K, rep.ctypes.data) == 0
    U = orc.unpack_ladder_int2(raw, N, K)
    dec = np.stack([[orc.decode_i2s_to_i8s(word(rep, n, w)) for w in range(K // 16)] for n in range(N)]).reshape(N, K)
    assert np.array_equal(dec, U)
    # columns past N (rounded up to 32) are packed as weight 0
    t48 = t[:48]
    p48 = np.empty(lib.vla_ternary_packed_words(48, K), np.uint32)
    assert lib.vla_ternary_pack_host(t48.ctypes.data, 48, K, p48.ctypes.data) == 0
    assert list(orc.decode_i2s_to_i8s(word(p48, 50, 3))) == [0] * 16
    assert lib.vla_ternary_repack_ladder_host(raw.ctypes.data, 24, K, rep.ctypes.data) == pkg.VLA_K_ERR_SHAPE


def test_pair_rope_rows_host_is_the_row_permutation_the_decode_epilogue_assumes():
    # Packing the permuted ternary matrix equals permuting the packed words: inside Q and K heads
    # 32-row block b holds rows 16b..16b+15 then D/2+16b..D/2+16b+15; V rows stay.
    lib = pkg.lib()
    Hq, Hkv, D, K = 3, 1, 64, 128
    N = (Hq + 2 * Hkv) * D
    r = np.random.default_rng(5)
    t = r.integers(-1, 2, (N, K)).astype(np.int8)
    src = np.arange(N)
    for n in range((Hq + Hkv) * D):
        rr, nl = n % D, n % 32
        src[n] = n - rr + (16 * (rr // 32) + nl if nl < 16 else D // 2 + 16 * (rr // 32) + nl - 16)
    assert sorted(src) == list(range(N))
    packed, want, got = (np.empty(N * K // 16, np.uint32) for _ in range(3))
    assert lib.vla_ternary_pack_host(t.ctypes.data, N, K, packed.ctypes.data) == 0
    tp = np.ascontiguousarray(t[src])
    assert lib.vla_ternary_pack_host(tp.ctypes.data, N, K, want.ctypes.data) == 0
    assert lib.vla_ternary_pair_rope_rows_host(packed.ctypes.data, Hq, Hkv, D, K, got.ctypes.data) == 0
    assert np.array_equal(got, want)
    assert lib.vla_ternary_pair_rope_rows_host(packed.ctypes.data, Hq, Hkv, 48, K, got.ctypes.data) == pkg.VLA_K_ERR_SHAPE
    assert lib.vla_ternary_pair_rope_rows_host(packed.ctypes.data, Hq, Hkv, D, K, packed.ctypes.data) == pkg.VLA_K_ERR_ARG


def test_fold_adaln_weight_host_operands():
    """Operand set of the projection launch that takes a DiT block's modulated LayerNorm
    inside it: rounded W (1 + scale), column sums of the rounded values, bias + W shift.
    With them rstd (x W'^T - mean colsum) + bias' equals adaln(x) W^T + b up to the bf16
    rounding of W' (checked in float64 on unrounded-compatible values)."""
    lib = pkg.lib()
    r = np.random.default_rng(5)
    N, K = 24, 48
    W = orc.round_bf16((0.2 * r.standard_normal((N, K))).astype(np.float32))
    b = r.standard_normal(N).astype(np.float32)
    # scales that keep W (1 + scale) exactly representable in bf16: powers of two minus one
    sc = r.choice(np.array([0.0, 1.0, -0.5, 3.0], np.float32), K)
    sh = r.standard_normal(K).astype(np.float32)
    Wf, cs, bs = np.empty((N, K), np.uint16), np.empty(N, np.float32), np.empty(N, np.float32)
    assert lib.vla_fold_adaln_weight_host(orc.to_bf16(W).ctypes.data, b.ctypes.data, sc.ctypes.data, sh.ctypes.data, N, K,
                                          Wf.ctypes.data, cs.ctypes.data, bs.ctypes.data) == pkg.VLA_K_OK
    Wf32 = orc.from_bf16(Wf)
    assert np.array_equal(Wf32, W * (1.0 + sc))
    assert np.allclose(cs, Wf32.astype(np.float64).sum(1), rtol=1e-6, atol=1e-6)
    assert np.allclose(bs, b + W.astype(np.float64) @ sh.astype(np.float64), rtol=1e-6, atol=1e-6)
    x = r.standard_normal((7, K)) * 3 + 1.5
    mean, var = x.mean(1, keepdims=True), x.var(1, keepdims=True)
    rstd = 1.0 / np.sqrt(var + 1e-5)
    got = rstd * (x @ Wf32.astype(np.float64).T - mean * cs[None, :]) + bs[None, :]
    want = (((x - mean) * rstd) * (1.0 + sc) + sh) @ W.astype(np.float64).T + b
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # general scales: round to nearest even of the fp32 product, no bias
    sc2 = (0.3 * r.standard_normal(K)).astype(np.float32)
    assert lib.vla_fold_adaln_weight_host(orc.to_bf16(W).ctypes.data, None, sc2.ctypes.data, sh.ctypes.data, N, K,
                                          Wf.ctypes.data, cs.ctypes.data, bs.ctypes.data) == pkg.VLA_K_OK
    assert np.array_equal(Wf, orc.to_bf16(W * (np.float32(1.0) + sc2)))
    assert np.allclose(bs, W.astype(np.float64) @ sh.astype(np.float64), rtol=1e-6, atol=1e-6)
    assert lib.vla_fold_adaln_weight_host(None, None, sc.ctypes.data, sh.ctypes.data, N, K, Wf.ctypes.data, cs.ctypes.data,
                                          bs.ctypes.data) == pkg.VLA_K_ERR_ARG


def test_fold_norm_weight_host_rounds_products_to_nearest_even():
    lib = pkg.lib()
    r = np.random.default_rng(7)
    N, K = 37, 48
    W = orc.round_bf16(r.standard_normal((N, K)).astype(np.float32))
    g = orc.round_bf16((1 + 0.5 * r.standard_normal(K)).astype(np.float32))
    out = np.empty((N, K), np.uint16)
    assert lib.vla_fold_norm_weight_host(orc.to_bf16(W).ctypes.data, orc.to_bf16(g).ctypes.data, pkg.VLA_DT_BF16, N, K,
                                         out.ctypes.data) == pkg.VLA_K_OK
    assert np.array_equal(out, orc.to_bf16(W * g[None, :]))  # products of bf16 values are exact in fp32: one rounding
    out32 = np.empty((N, K), np.float32)
    assert lib.vla_fold_norm_weight_host(W.ctypes.data, g.ctypes.data, pkg.VLA_DT_F32, N, K, out32.ctypes.data) == pkg.VLA_K_OK
    assert np.array_equal(out32, W * g[None, :])
    assert lib.vla_fold_norm_weight_host(None, g.ctypes.data, pkg.VLA_DT_F32, N, K, out32.ctypes.data) == pkg.VLA_K_ERR_ARG


def test_null_and_shape_errors_are_reported_not_fatal():
    lib = pkg.lib()
    assert lib.vla_kv_append(None, None, None, None, 0, 1, 0, 64, 64, 0, 1, None) == pkg.VLA_K_ERR_ARG
    assert lib.vla_rope_neox(None, None, None, 0, 1, 1, 1, 64, None) == pkg.VLA_K_ERR_ARG
    assert lib.vla_linear(None, None, None, None, None, 0, 0, 1, 1, 4, None) == pkg.VLA_K_ERR_ARG
    assert lib.vla_attn_prefix_suffix(None, None, None, None, 0, 1, 1, 1, 1, 64, 64, 1, 1.0, 0, 0, 0, 0, None, None) == pkg.VLA_K_ERR_ARG
    assert lib.vla_ternary_gemm(None, None, None, None, None, None, None, 1, 1, 16, 128, None) == pkg.VLA_K_ERR_ARG


# ---------------------------------------------------------------- struct layout of include/vla.h
def _header_fields(text, name):
    """(field, C type) pairs of `typedef struct { ... } name;`, one per declarator."""
    import re
    m = re.search(r"typedef struct \{([^{}]*)\}\s*" + name + r"\s*;", text, re.S)
    assert m, name + " not found in vla.h"
    body = re.sub(r"/\*.*?\*/", "", m.group(1), flags=re.S)
    out = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        first, *rest = [d.strip() for d in decl.split(",")]
        parts = first.replace("*", " * ").split()
        ctype = " ".join(p for p in parts[:-1] if p != "const")
        out.append((parts[-1], ctype))
        out += [(r.lstrip("* "), ctype) for r in rest]
    return out


def test_ctypes_structs_follow_the_header_field_for_field(tmp_path):
    """The check the reference runs on its own bindings (tests/py/test_bindings.py:29-64): field
    order and types of the ctypes mirrors against the header text -- and, since a C compiler is
    at hand, sizes and offsets against what gcc lays out."""
    import ctypes
    import subprocess
    from vla_cpp_amd import ffi
    text = open(os.path.join(ROOT, "include", "vla.h")).read()
    c_types = {"int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64, "float": ctypes.c_float, "double": ctypes.c_double}
    pairs = (("vla_config", ffi.Config), ("vla_image", ffi.Image), ("vla_inputs", ffi.Inputs), ("vla_stats", ffi.Stats))
    prog = ["#include <stdio.h>", "#include <stddef.h>", '#include "vla.h"', "int main(void) {"]
    for c_name, py in pairs:
        hdr = _header_fields(text, c_name)
        assert [n for n, _ in hdr] == [n for n, _ in py._fields_], c_name
        for (hn, ht), (pn, pt) in zip(hdr, py._fields_):
            if ht.endswith("*"):
                assert issubclass(pt, (ctypes._Pointer, ctypes.c_void_p)) or pt is ctypes.c_void_p, (c_name, hn)
            else:
                assert pt is c_types[ht], (c_name, hn, ht, pt)
            prog.append('  printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (c_name, hn, c_name, hn))
        prog.append('  printf("%s %%zu\\n", sizeof(%s));' % (c_name, c_name))
    prog += ["  return 0;", "}"]
    src, exe = os.path.join(str(tmp_path), "layout.c"), os.path.join(str(tmp_path), "layout")
    open(src, "w").write("\n".join(prog))
    subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), src, "-o", exe], check=True)  # the header is C-clean
    want = dict(l.split() for l in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.splitlines())
    for c_name, py in pairs:
        assert ctypes.sizeof(py) == int(want[c_name]), c_name
        for n, _ in py._fields_:
            assert getattr(py, n).offset == int(want["%s.%s" % (c_name, n)]), (c_name, n)
    assert ffi.ABI_VERSION == int(__import__("re").search(r"#define VLA_ABI_VERSION\s+(\d+)", text).group(1))
