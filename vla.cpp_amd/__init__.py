"""MI355X-native action-expert attention path: loader for ``libvla.so``.

The product is the C-ABI shared library built from ``csrc/`` (HIP kernels) and
``host/`` (C++ host layer); this module only locates it, declares the ctypes
signatures of ``include/vla_kernels.h`` / ``include/vla.h`` and offers thin
helpers that pass torch device pointers through.  There is no fallback: if the
library is missing, loading raises.

The directory name is not a Python identifier, so import it through
``load_package()`` in ``__graft_entry__`` (module name ``vla_cpp_amd``).
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libvla.so")

VLA_DT_F32, VLA_DT_BF16, VLA_DT_BF16_P2 = 0, 1, 2
VLA_ACT_NONE, VLA_ACT_SILU, VLA_ACT_GELU, VLA_ACT_RELU = 0, 1, 2, 3
VLA_MASK_NONE, VLA_MASK_CAUSAL_SUFFIX, VLA_MASK_PI0_STATE = 0, 1, 2
VLA_K_OK, VLA_K_ERR_ARG, VLA_K_ERR_SHAPE, VLA_K_ERR_LAUNCH, VLA_K_ERR_WORKSPACE = 0, -1, -2, -3, -4

_lib = None

_vp, _i, _f, _d, _i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_double, ctypes.c_int64

# name -> argtypes (restype int unless listed in _RESTYPES)
KERNEL_API = {
    "vla_kv_append": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "vla_kv_gather": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "vla_rope_tables_host": [_vp, _i, _i, _d, _vp, _vp],
    "vla_rope_neox": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "vla_rms_norm": [_vp, _vp, _vp, _i, _i, _i, _f, _vp],
    "vla_adaln": [_vp, _vp, _vp, _vp, _i, _i, _i, _f, _vp],
    "vla_linear": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "vla_adarms": [_vp, _vp, _vp, _vp, _i, _i, _i, _f, _vp],
    "vla_linear_gated": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "vla_linear_act": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "vla_glu_linear": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp],
    "vla_attn_qkv_rope": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp],
    "vla_rmsnorm_attn_qkv_rope": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp],
    "vla_fold_norm_weight_host": [_vp, _vp, _i, _i, _i, _vp],
    "vla_layernorm_attn_qkv_rope": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _f,
                                    _vp],
    "vla_layernorm_qkv_self_attention": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _f, _vp, _vp],
    "vla_layernorm_qkv_self_attention_stats": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _f, _f, _vp, _vp],
    "vla_layernorm_attn_qkv_rope_stats": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _f,
                                          _vp],
    "vla_linear_row_stats": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "vla_fold_adaln_weight_host": [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp],
    "vla_qkv_split_rope_append": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    "vla_attn_prefix_suffix": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i, _vp, _vp],
    "vla_attn_prefix_suffix_noalloc": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i, _vp, _vp],
    "vla_attn_prefix_suffix_ws": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i, _vp, _vp,
                                  ctypes.c_size_t, _vp],
    "vla_attn_workspace_bytes": [_i, _i, _i, _i, _i, _i, _i],
    "vla_attn_workspace_reset": [_vp, ctypes.c_size_t, _vp],
    "vla_embed_suffix": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "vla_embed_suffix_act": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "vla_finish_suffix_rows": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "vla_set_lead_rows": [_vp, _vp, _i, _i, _i, _i, _i, _vp],
    "vla_euler_step": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp],
    "vla_rmsnorm_euler_step": [_vp, _vp, _vp, _f, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp],
    "vla_adanorm_euler_step": [_vp, _vp, _vp, _vp, _i, _f, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp],
    "vla_act_quant_bf16": [_vp, _vp, _vp, _vp, _i, _i, _vp],
    "vla_ternary_quant_host": [_vp, _i64, _vp, _vp],
    "vla_ternary_packed_words": [_i, _i],
    "vla_ternary_pack_host": [_vp, _i, _i, _vp],
    "vla_ternary_repack_ladder_host": [_vp, _i, _i, _vp],
    "vla_ternary_gemm": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "vla_ternary_gemm_add": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "vla_rmsnorm_act_quant_bf16": [_vp, _vp, _vp, _vp, _vp, _f, _i, _i, _vp],
    "vla_sqrelu_rmsnorm_act_quant_bf16": [_vp, _vp, _vp, _vp, _vp, _f, _i, _i, _vp],
    "vla_rmsnorm_ternary_gemv": [_vp, _vp, _f, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "vla_sqrelu_rmsnorm_ternary_gemv": [_vp, _vp, _f, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "vla_rmsnorm_ternary_gemv_rope_append": [_vp, _vp, _f, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i,
                                             _vp],
    "vla_ternary_pair_rope_rows_host": [_vp, _i, _i, _i, _i, _vp],
    "bitvla_rmsnorm_bf16": [_vp, _vp, _vp, _f, _i, _i, _vp],
    "bitvla_rope_neox_bf16": [_vp, _vp, _vp, _i, _i, _i, _vp],
    "bitvla_softmax_scaled_bf16": [_vp, _f, _i, _i, _vp],
    "bitvla_add_bf16": [_vp, _vp, _vp, _i, _vp],
    "gate_up_fused_sqrelu_mul_bf16": [_vp, _vp, _i, _i, _vp],
    "bitvla_lm_hip_init": [_i, _i, _i, _i, _i, _i, _f, _f, _i],
    "bitvla_lm_hip_free": [_vp],
    "bitvla_lm_hip_set_layer": [_vp, _i, _vp],
    "bitvla_lm_hip_set_output_norm": [_vp, _vp],
    "bitvla_lm_hip_forward": [_vp, _vp, _vp, _i, _vp],
    "bitvla_repeat_kv_bf16": [_vp, _vp, _i, _i, _i, _i, _vp],
    "bitvla_transpose_sNhd_to_NshHd_bf16": [_vp, _vp, _i, _i, _i, _vp],
    "bitvla_transpose_NshHd_to_sNhd_bf16": [_vp, _vp, _i, _i, _i, _vp],
    "bitvla_gather_rows_bf16": [_vp, _vp, _vp, _i, _i, _vp],
    "bitvla_act_quant": [_vp, _vp, _vp, _i, _i, _vp],
    "bitlinear_int8xint2_m": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "bitlinear_int8xint2": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "vla_kernels_arch": [],
    "vla_kernels_init": [],
    "vla_kernels_reload_env": [],
    "vla_kernels_tuning_generation": [],
}
_RESTYPES = {"vla_kernels_arch": ctypes.c_char_p, "vla_attn_workspace_bytes": ctypes.c_size_t,
             "vla_kernels_reload_env": None, "vla_ternary_packed_words": ctypes.c_long,
             "bitvla_lm_hip_init": ctypes.c_void_p, "bitvla_lm_hip_free": None, "bitvla_lm_hip_set_layer": None,
             "bitvla_lm_hip_set_output_norm": None}


def tern_word_index(n, w, K):
    """Index of packed word (column n, 16-k group w) in the gfx950 ternary layout."""
    return (((n >> 5) * (K // 32) + (w >> 1)) * 2 + (w & 1)) * 32 + (n & 31)


def lib():
    """The loaded C-ABI library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libvla.so is missing (%s): build it with __graft_entry__.build(); there is no CPU fallback" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in KERNEL_API.items():
            fn = getattr(_lib, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, ctypes.c_int)
    return _lib


def ptr(t):
    """Device (or host) address of a torch tensor / numpy array, or None."""
    if t is None:
        return None
    if hasattr(t, "data_ptr"):
        assert t.is_contiguous(), "kernels take contiguous buffers"
        return t.data_ptr()
    return t.ctypes.data


def stream():
    """The current torch HIP stream as a hipStream_t value."""
    import torch
    return torch.cuda.current_stream().cuda_stream


def check(rc, what=""):
    if rc != VLA_K_OK:
        raise RuntimeError("%s failed with vla_kstatus %d" % (what or "kernel call", rc))


def call(name, *args):
    """Call a kernel entry point, translating tensors to pointers and appending the current stream."""
    fn = getattr(lib(), name)
    conv = [ptr(a) if (a is None or hasattr(a, "data_ptr") or hasattr(a, "ctypes")) else a for a in args]
    rc = fn(*conv, stream())
    check(rc, name)
    return rc
