"""Pins the oracle's INT4 functions (oracle/kx_oracle.cpp) without a GPU.

Reference semantics: src/kimi_exec.cu:300-323.  The reference's own tests hold no
vector for this arithmetic, so the checks are closed forms, an exhaustive dequant
sweep against integer-arithmetic rounding, and float64 dot products.
"""
import numpy as np
import pytest

import oracle as O
from oracle import ptr


def rne_bf16_remainder(f32):
    """bf16 RNE written with an explicit remainder test (not the +0x7fff trick)."""
    u = np.asarray(f32, dtype=np.float32).view(np.uint32).astype(np.uint64)
    upper, lower = u >> 16, u & 0xFFFF
    up = (lower > 0x8000) | ((lower == 0x8000) & ((upper & 1) == 1))
    return (upper + up).astype(np.uint16)


def unpack_np(packed):
    """closed form of :311 -- lane j of a word is bits 4j..4j+3, minus 8"""
    p = packed.astype(np.uint32)
    lanes = np.stack([((p >> np.uint32(4 * j)) & np.uint32(0xF)).astype(np.int8) - 8 for j in range(8)], axis=-1)
    return lanes.reshape(*packed.shape[:-1], packed.shape[-1] * 8)


def test_unpack_all_nibble_lane_combinations(ox):
    for lane in range(8):
        for nib in range(16):
            w = np.array([[np.uint32(nib << (4 * lane))]], dtype=np.uint32)
            q = np.empty((1, 8), dtype=np.int8)
            ox.ox_i4_unpack(ptr(w), ptr(q), 1, 8)
            expect = np.full(8, -8, dtype=np.int8)
            expect[lane] = nib - 8
            assert (q[0] == expect).all()


def test_unpack_random_and_repack(ox):
    w = O.words_u32(64 * 128, 1, 7).reshape(64, 128)
    q = np.empty((64, 1024), dtype=np.int8)
    ox.ox_i4_unpack(ptr(w), ptr(q), 64, 1024)
    assert (q == unpack_np(w)).all()
    assert q.min() == -8 and q.max() == 7
    n = (q.astype(np.int64) + 8).reshape(64, 128, 8)
    repacked = sum(n[..., j].astype(np.uint64) << (4 * j) for j in range(8)).astype(np.uint32)
    assert (repacked == w).all()


def test_dequant_exhaustive_16_nibbles_x_65536_scales(ox):
    # every bf16 bit pattern as a scale (finite ones), every nibble value
    scales = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    finite = ((scales >> 7) & 0xFF) != 0xFF
    scales = scales[finite]
    rows = scales.size                    # one row per scale, one group per row
    # a group of 32 columns: nibble value = column index mod 16
    word = np.uint32(sum(((8 * p + j) % 16) << (4 * j) for p in range(1) for j in range(8)))
    words = np.empty((rows, 4), dtype=np.uint32)
    for p in range(4):
        words[:, p] = sum(((8 * p + j) % 16) << (4 * j) for j in range(8))
    w = np.empty((rows, 32), dtype=np.uint16)
    ox.ox_i4_dequant(ptr(words), ptr(scales), ptr(w), rows, 32)
    q = (np.arange(32) % 16 - 8).astype(np.float64)
    prod = O.bf16_to_f32(scales).astype(np.float64)[:, None] * q[None, :]      # exact in float64
    with np.errstate(over="ignore"):
        prod32 = prod.astype(np.float32)                                        # exact (11-bit significand) or inf
    assert (prod32.astype(np.float64) == prod).all() or np.isinf(prod32).any()
    expect = rne_bf16_remainder(prod32)
    assert (w == expect).all()
    assert word == words[0, 0]


def _case(rows, cols, tokens, seed):
    packed = O.words_u32(rows * cols // 8, seed, 1).reshape(rows, cols // 8)
    scale = O.normal_bf16(rows * cols // 32, seed, 2, 0.02, 1).reshape(rows, cols // 32)
    x = O.normal_bf16(tokens * cols, seed, 3, 1.0).reshape(tokens, cols)
    return packed, scale, x


def _dot64(ox, packed, scale, x):
    rows, cols = packed.shape[0], packed.shape[1] * 8
    w = np.empty((rows, cols), dtype=np.uint16)
    ox.ox_i4_dequant(ptr(packed), ptr(scale), ptr(w), rows, cols)
    return O.bf16_to_f32(x).astype(np.float64) @ O.bf16_to_f32(w).astype(np.float64).T


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("rows,cols,tokens", [(48, 2048, 2), (40, 7168, 1), (7, 1024, 3)])
def test_gemv_against_float64_dot(ox, mode, rows, cols, tokens):
    packed, scale, x = _case(rows, cols, tokens, 11)
    y = np.empty((tokens, rows), dtype=np.uint16)
    ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y), rows, cols, tokens, mode)
    ref = _dot64(ox, packed, scale, x)
    err = O.max_rel(O.bf16_to_f32(y), ref)
    # one bf16 rounding of the output is 2^-9 relative; the bar of the path is 1e-2
    assert err < 1e-2, err
    assert err < 6e-3, err


@pytest.mark.parametrize("mode", [0, 1])
def test_gemv_unit_vector_reads_back_one_weight(ox, mode):
    rows, cols = 16, 1024
    packed = O.words_u32(rows * cols // 8, 5, 1).reshape(rows, cols // 8)
    scale = np.full((rows, cols // 32), 0x3F80, dtype=np.uint16)   # 1.0
    q = unpack_np(packed)
    for k in (0, 1, 4, 5, 7, 31, 32, 333, 1023):
        x = np.zeros((1, cols), dtype=np.uint16)
        x[0, k] = 0x3F80
        y = np.empty((1, rows), dtype=np.uint16)
        ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y), rows, cols, 1, mode)
        assert (O.bf16_to_f32(y[0]) == q[:, k].astype(np.float32)).all(), k


@pytest.mark.parametrize("mode", [0, 1])
def test_gemv_ones_gives_row_sums(ox, mode):
    rows, cols = 16, 2048
    packed = O.words_u32(rows * cols // 8, 6, 1).reshape(rows, cols // 8)
    scale = np.full((rows, cols // 32), 0x3F80, dtype=np.uint16)
    x = np.full((1, cols), 0x3F80, dtype=np.uint16)
    y = np.empty((1, rows), dtype=np.uint16)
    ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y), rows, cols, 1, mode)
    sums = unpack_np(packed).astype(np.int64).sum(axis=1).astype(np.float32)   # exact in f32
    assert (y[0] == rne_bf16_remainder(sums)).all()


def test_gemv_modes_agree_config1_shape(ox):
    # BASELINE config 1: K=7168 -> N=2048, batch 1
    packed, scale, x = _case(2048, 7168, 1, 0)
    y0 = np.empty((1, 2048), dtype=np.uint16)
    y1 = np.empty((1, 2048), dtype=np.uint16)
    ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y0), 2048, 7168, 1, 0)
    ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y1), 2048, 7168, 1, 1)
    err = O.max_rel(O.bf16_to_f32(y1), O.bf16_to_f32(y0))
    assert err < 1e-2, err
    # most outputs round to the same bf16 value
    assert np.mean(y0 == y1) > 0.5
