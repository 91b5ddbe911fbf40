"""ctypes binding of libkx.so (include/kx.h).

Mirrors what a caller of the reference's executor boundary would bind
(reference: blok/runtime.py:70-83 spawns the executor; here the same operators
are reachable in-process).  Device memory is owned through kx_dev_malloc /
kx_dev_free so that no other GPU runtime is needed.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


class KxError(RuntimeError):
    """A libkx call returned a non-zero status (reference: die(), src/kimi_exec.cu:495-498)."""


def lib_path():
    return os.path.join(_HERE, "libkx.so")


class KxConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "n_layers", "first_dense", "hidden", "heads", "qk_nope", "qk_rope", "v_head", "q_rank",
        "kv_rank", "experts", "topk", "moe_inter", "shared_inter", "dense_inter", "vocab",
        "max_batch", "max_context")] + [("eos_id", C.c_uint32)] + [(n, C.c_float) for n in (
            "rms_eps", "rope_theta", "routed_scale", "yarn_factor", "yarn_beta_fast",
            "yarn_beta_slow", "yarn_orig_ctx", "yarn_mscale_all_dim", "init_sigma", "expert_scale_sigma")] + [
                ("seed", C.c_uint64)]


class KxMoeWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "d_router_gate", "d_router_bias", "d_gate_packed", "d_gate_scale", "d_up_packed",
        "d_up_scale", "d_down_packed", "d_down_scale", "d_shared_gate", "d_shared_up",
        "d_shared_down")]


_P, _I, _U64, _F, _SZ = C.c_void_p, C.c_int32, C.c_uint64, C.c_float, C.c_size_t
_PP = C.POINTER(C.c_void_p)
_SIGS = {
    "kx_config_default": [C.POINTER(KxConfig)],
    "kx_device_info": [C.c_char_p, _SZ, C.POINTER(C.c_int32), C.POINTER(C.c_uint64)],
    "kx_dev_malloc": [_PP, _SZ],
    "kx_dev_free": [_P],
    "kx_dev_memset": [_P, C.c_int, _SZ, _P],
    "kx_dev_mem_info": [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "kx_h2d": [_P, _P, _SZ],
    "kx_d2h": [_P, _P, _SZ],
    "kx_sync": [_P],
    "kx_event_create": [_PP],
    "kx_event_destroy": [_P],
    "kx_event_record": [_P, _P],
    "kx_event_elapsed_ms": [_P, _P, C.POINTER(C.c_float)],
    "kx_fill_normal_bf16": [_P, _U64, _U64, _U64, _F, C.c_int, _P],
    "kx_fill_normal_f32": [_P, _U64, _U64, _U64, _F, _P],
    "kx_fill_words_u32": [_P, _U64, _U64, _U64, _P],
    "kx_fill_tokens_u32": [_P, _U64, _U64, _U64, C.c_uint32, _P],
    "kx_dev_copy": [_P, _P, _U64, _P],
    "kx_i4_unpack": [_P, _P, _I, _I, _P],
    "kx_i4_dequant": [_P, _P, _P, _I, _I, _P],
    "kx_i4_gemv": [_P, _P, _P, _P, _I, _I, _I, _P],
    "kx_rmsnorm": [_P, _P, _P, _I, _I, _F, _P],
    "kx_gemv_bf16": [_P, _P, _P, _I, _I, _I, C.c_int, _P],
    "kx_lm_head_argmax": [_P, _P, _P, _P, _I, _I, _I, _P, _P],
    "kx_static_scratch_init": [],
    "kx_lm_head_argmax_static": [_P, _P, _P, _P, _I, _I, _I, _P],
    "kx_router_topk": [_P, _P, _P, _P, _I, _I, _I, _F, _P],
    "kx_bucket": [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P],
    "kx_moe_workspace_create": [C.POINTER(KxConfig), _I, _PP],
    "kx_moe_workspace_destroy": [_P],
    "kx_moe_workspace_views": [_P, _PP, _PP, _PP, _PP, _PP, _PP, _PP, _PP],
    "kx_moe_decode_layer": [C.POINTER(KxConfig), C.POINTER(KxMoeWeights), _P, _P, _P, _I, C.c_uint32, _P],
    "kx_fill_affine_bf16": [_P, _U64, _U64, _U64, _F, _F, _P],
    "kx_rope_table": [C.POINTER(KxConfig), _I, _I, _P],
    "kx_softmax_scale": [C.POINTER(KxConfig), C.POINTER(C.c_float), C.POINTER(C.c_float)],
    "kx_q_absorb": [C.POINTER(KxConfig), _P, _P, _P, _P, _I, _P],
    "kx_mla_workspace_bytes": [C.POINTER(KxConfig), _I, _I, C.POINTER(_SZ)],
    "kx_mla_decode": [C.POINTER(KxConfig), _P, _SZ, _P, _P, _P, _I, _I, _I, _P],
    "kx_model_bytes": [C.POINTER(KxConfig), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "kx_model_create": [C.POINTER(KxConfig), _PP],
    "kx_model_destroy": [_P],
    "kx_prefill": [_P, _P, _I, _I],
    "kx_decode_step": [_P, _P],
    "kx_greedy_sample": [_P, _P],
    "kx_generate": [_P, _P, _I, _I, _I, C.c_int, _P, _P],
    "kx_model_hidden": [_P, _P],
    "kx_model_logits": [_P, _P],
    "kx_model_latent": [_P, _I, _I, _I, _I, _P],
    "kx_model_timing": [_P, C.POINTER(C.c_float)],
    "kx_model_steps_decoded": [_P, C.POINTER(C.c_int32)],
    "kx_model_set_fusion": [_P, C.c_uint32],
    "kx_model_debug_fail_waits": [_P],
    "kx_model_set_attention_kernel": [_P, _I],
    "kx_model_set_routing_record": [_P, C.c_int],
    "kx_model_set_exact": [_P, C.c_uint32],
    "kx_model_rewind": [_P, _I],
    "kx_model_routing": [_P, _I, _P, _P],
    "kx_model_routing_history": [_P, _I, _I, _I, _P],
    "kx_model_set_prefill_chunk": [_P, _I],
    "kx_model_stream": [_P, _PP],
    "kx_moe_prefill_layer": [C.POINTER(KxConfig), C.POINTER(KxMoeWeights), _P, _P, _P, _I, C.c_uint32, _P],
    "kx_moe_decode_layer_timed": [C.POINTER(KxConfig), C.POINTER(KxMoeWeights), _P, _P, _P, _I,
                                  C.c_uint32, _P, C.POINTER(C.c_float)],
    "kx_moe_routed_only": [C.POINTER(KxConfig), C.POINTER(KxMoeWeights), _P, _P, _I, _I, _P],
    "kx_index_check": [C.POINTER(KxConfig), C.c_char_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "kx_index_infer_config": [C.c_char_p, C.POINTER(KxConfig)],
    "kx_model_load": [C.POINTER(KxConfig), C.c_char_p, _PP],
    "kx_model_load_info": [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_double)],
    "kx_tokenizer_open": [C.c_char_p, _PP],
    "kx_tokenizer_close": [_P],
    "kx_tokenizer_info": [_P, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)],
    "kx_pretokenize": [C.c_char_p, _SZ, _P, _SZ, C.POINTER(_SZ)],
    "kx_tokenizer_encode": [_P, C.c_char_p, _SZ, C.c_int, _P, _SZ, C.POINTER(_SZ)],
    "kx_tokenizer_decode": [_P, _P, _SZ, _P, _SZ, C.POINTER(_SZ)],
    "kx_encode_prompt": [_P, C.c_char_p, _SZ, _P, _SZ, C.POINTER(_SZ)],
}

_lib = None


def load_library(path):
    """A library file with the signatures of include/kx.h bound.  Raises KxError when it is missing: there is no fallback."""
    if not os.path.exists(path):
        raise KxError(f"{path} is not built; run `make -C blok_amd/csrc` "
                      "(or __graft_entry__.build())")
    lib = C.CDLL(path)
    lib.kx_last_error.restype = C.c_char_p
    lib.kx_last_error.argtypes = []
    for name, args in _SIGS.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = C.c_int
    return lib


def kx():
    """The loaded library (blok_amd/libkx.so)."""
    global _lib
    if _lib is None:
        _lib = load_library(lib_path())
    return _lib


def check(rc):
    if rc != 0:
        raise KxError(kx().kx_last_error().decode("utf-8", "replace"))


def default_config():
    cfg = KxConfig()
    check(kx().kx_config_default(C.byref(cfg)))
    return cfg


class DevBuf:
    """A device allocation owned through the C ABI."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(kx().kx_dev_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        check(kx().kx_h2d(buf.ptr, arr.ctypes.data, arr.nbytes))
        return buf

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        check(kx().kx_h2d(self.ptr, arr.ctypes.data, arr.nbytes))

    def to_numpy(self, dtype, shape, offset_bytes=0):
        out = np.empty(shape, dtype=dtype)
        assert offset_bytes + out.nbytes <= self.nbytes
        check(kx().kx_d2h(out.ctypes.data, self.ptr + offset_bytes, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            kx().kx_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
