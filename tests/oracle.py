"""ctypes binding of the CPU oracle (oracle/kx_oracle.cpp) for the tests.

The oracle is test infrastructure: it is loaded here, by __graft_entry__.smoke()
and by the cpu_baseline leg of bench.py, and nowhere else.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "build", "libkx_oracle.so")

_P, _I, _U64, _F = C.c_void_p, C.c_int, C.c_uint64, C.c_float


class OxMoeWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "router_gate", "router_bias", "gate_packed", "gate_scale", "up_packed", "up_scale",
        "down_packed", "down_scale", "shared_gate", "shared_up", "shared_down")]


_SIGS = {
    "ox_expf": ([_F, _I], _F),
    "ox_bf16": ([_F], C.c_uint16),
    "ox_fill_normal_bf16": ([_P, _U64, _U64, _U64, _F, _I], None),
    "ox_fill_normal_f32": ([_P, _U64, _U64, _U64, _F], None),
    "ox_fill_words_u32": ([_P, _U64, _U64, _U64], None),
    "ox_i4_unpack": ([_P, _P, _I, _I], None),
    "ox_i4_dequant": ([_P, _P, _P, _I, _I], None),
    "ox_i4_gemv": ([_P, _P, _P, _P, _I, _I, _I, _I], None),
    "ox_rmsnorm": ([_P, _P, _P, _I, _I, _F, _I], None),
    "ox_gemv_bf16": ([_P, _P, _P, _I, _I, _I, _I, _I], None),
    "ox_router_topk": ([_P, _P, _P, _P, _I, _I, _I, _F, _I], None),
    "ox_bucket": ([_P, _I, _I, _I, _P, _P, _P, _P], _I),
    "ox_moe_layer": ([C.POINTER(OxMoeWeights), _P, _P, _I, _I, _I, _I, _I, _I, _F, C.c_uint32, _I,
                      _P, _P, _P, _P, _P], None),
    "ox_fill_affine_bf16": ([_P, _U64, _U64, _U64, _F, _F], None),
    "ox_fill_tokens_u32": ([_P, _U64, _U64, _U64, C.c_uint32], None),
    "ox_yarn_inv_freq": ([_P, _I], _F),
    "ox_rope_table": ([_P, _I, _I, _P], None),
    "ox_rope_apply": ([_P, _P, _P, _I], None),
    "ox_softmax_scale": ([_P, C.POINTER(C.c_float), C.POINTER(C.c_float)], None),
    "ox_mla_span_tiles": ([_I], _I),
    "ox_mla_decode": ([_P, _P, C.c_size_t, _P, _P, _I, _I, _I], None),
    "ox_model_create": ([_P, _I], _P),
    "ox_model_create_ex": ([_P, _I, C.c_uint32], _P),
    "ox_model_experts_produced": ([_P], _U64),
    "ox_model_keep_experts": ([_P, _I], None),
    "ox_model_destroy": ([_P], None),
    "ox_model_set_tensor": ([_P, _I, _I, _I, _P, _U64], _I),
    "ox_model_step": ([_P, _P, _I, _I, _I, _P], _I),
    "ox_generate": ([_P, _P, _I, _I, _I, _I, _P, _P], _I),
    "ox_model_logits": ([_P], C.POINTER(C.c_float)),
    "ox_model_hidden": ([_P], C.POINTER(C.c_uint16)),
    "ox_model_latent": ([_P, _I], C.POINTER(C.c_uint16)),
    "ox_moe_layer_routed": ([C.POINTER(OxMoeWeights), _P, _P, _I, _I, _I, _I, _I, _I, C.c_uint32, _I, _P, _P], None),
    "ox_num_threads": ([], _I),
    "ox_set_threads": ([_I], None),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", ORACLE_DIR], check=True, capture_output=True)
        lib = C.CDLL(LIB)
        for name, (args, res) in _SIGS.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = res
        _lib = lib
    return _lib


def ptr(a):
    return a.ctypes.data if a is not None else None


# ---- numpy helpers shared by the tests -------------------------------------------
def bf16_to_f32(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(f):
    """integer round-to-nearest-even, no float library involved"""
    u = np.asarray(f, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = u + 0x7FFF + ((u >> 16) & 1)
    return (r >> 16).astype(np.uint16)


def normal_bf16(n, seed, tid, sigma, absval=0):
    out = np.empty(n, dtype=np.uint16)
    load().ox_fill_normal_bf16(ptr(out), n, seed, tid, sigma, absval)
    return out


def normal_f32(n, seed, tid, sigma):
    out = np.empty(n, dtype=np.float32)
    load().ox_fill_normal_f32(ptr(out), n, seed, tid, sigma)
    return out


def words_u32(n, seed, tid):
    out = np.empty(n, dtype=np.uint32)
    load().ox_fill_words_u32(ptr(out), n, seed, tid)
    return out


def max_rel(a, b):
    """max |a-b| over max |b|: the normalised maximum error used for the 1e-2 bar"""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30))


def elem_err(a, b):
    """Element-wise criterion beside max_rel: max over elements of |a-b| / (|b| + rms(b)).  An element is held to
    its own magnitude once that is above the tensor's RMS, and to the RMS below it (an fp32-accumulated dot product
    that cancels to near zero has no relative accuracy of its own)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    rms = max(float(np.sqrt(np.mean(b * b))), 1e-30)
    return float(np.max(np.abs(a - b) / (np.abs(b) + rms)))


def tokens_u32(n, seed, tid, vocab):
    out = np.empty(n, dtype=np.uint32)
    load().ox_fill_tokens_u32(ptr(out), n, seed, tid, vocab)
    return out


def small_config(n_layers=3, first_dense=1, batch=1, context=96):
    """A stack with every feature of the Kimi-K2 one at sizes the scalar oracle finishes in seconds.
    kv_rank 512 / qk_rope 64 / qk_nope 128 / v_head 128 are the real ones (the attention kernel is built for them)."""
    from blok_amd.lib import KxConfig
    c = KxConfig()
    c.n_layers, c.first_dense = n_layers, first_dense
    c.hidden, c.heads, c.qk_nope, c.qk_rope, c.v_head = 1024, 8, 128, 64, 128
    c.q_rank, c.kv_rank, c.experts, c.topk = 512, 512, 16, 4
    c.moe_inter, c.shared_inter, c.dense_inter, c.vocab = 1024, 512, 1536, 2048
    c.max_batch, c.max_context, c.eos_id = batch, context, 2047
    c.rms_eps, c.rope_theta, c.routed_scale = 1e-5, 50000.0, 2.827
    c.yarn_factor, c.yarn_beta_fast, c.yarn_beta_slow, c.yarn_orig_ctx, c.yarn_mscale_all_dim = 32.0, 32.0, 1.0, 4096.0, 1.0
    c.init_sigma, c.expert_scale_sigma, c.seed = 0.02, 0.02, 1234
    return c


class OxModel:
    def __init__(self, cfg, mode, experts_on_demand=False):
        """experts_on_demand: the routed experts are generated when a token first selects them (same values: the
        generator is a function of seed, tensor and index), so a stack with hundreds of GB of experts fits."""
        self.cfg, self.lib = cfg, load()
        self.h = self.lib.ox_model_create_ex(C.byref(cfg), mode, 1 if experts_on_demand else 0)

    def generate(self, prompt, n_tokens, ignore_eos=True):
        B, P = prompt.shape
        out = np.zeros((B, n_tokens), dtype=np.uint32)
        counts = np.zeros(B, dtype=np.int32)
        rc = self.lib.ox_generate(self.h, ptr(np.ascontiguousarray(prompt)), B, P, n_tokens, int(ignore_eos), ptr(out), ptr(counts))
        return rc, out, counts

    def step(self, ids, pos, sample):
        """one decode step of every sequence at position pos; returns the sampled ids (or None)"""
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        out = np.zeros(len(ids), dtype=np.uint32)
        if self.lib.ox_model_step(self.h, ptr(ids), len(ids), pos, int(sample), ptr(out)) != 0:
            raise ValueError("ox_model_step: bad argument")
        return out if sample else None

    def set_tensor(self, layer, tid, expert, arr):
        arr = np.ascontiguousarray(arr)
        if self.lib.ox_model_set_tensor(self.h, layer, tid, expert, ptr(arr), arr.nbytes) != 0:
            raise ValueError(f"ox_model_set_tensor({layer}, {tid}, {expert}, {arr.nbytes} bytes) does not fit the model")

    def logits(self, B):
        p = self.lib.ox_model_logits(self.h)
        return np.ctypeslib.as_array(p, shape=(self.cfg.max_batch, self.cfg.vocab))[:B].copy()

    def hidden(self, B):
        p = self.lib.ox_model_hidden(self.h)
        return np.ctypeslib.as_array(p, shape=(self.cfg.max_batch, self.cfg.hidden))[:B].copy()

    def latent(self, layer):
        p = self.lib.ox_model_latent(self.h, layer)
        kva = self.cfg.kv_rank + self.cfg.qk_rope
        return np.ctypeslib.as_array(p, shape=(self.cfg.max_batch, self.cfg.max_context, kva)).copy()

    def close(self):
        if self.h:
            self.lib.ox_model_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()
