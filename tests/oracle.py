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
