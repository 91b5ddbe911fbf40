"""GPU parity of the INT4 operators, through the C ABI, against the oracle.

Bars: unpack, dequant and the synthetic fills are bit-exact; the fused GEMV is
bit-exact against the oracle's kx schedule (mode 1) and within max-rel 1e-2 of
the reference schedule (mode 0).
"""
import numpy as np
import pytest

import oracle as O
from kxt import check, dev, say
from oracle import ptr

pytestmark = pytest.mark.gpu
from blok_amd.lib import DevBuf  # noqa: E402


def test_fill_kernels_match_oracle(kxlib, ox):
    n = 100003
    for tid, sigma, absval in ((3, 1.0, 0), (4, 0.02, 1)):
        b = DevBuf(n * 2)
        check(kxlib.kx_fill_normal_bf16(b.ptr, n, 42, tid, sigma, absval, None))
        check(kxlib.kx_sync(None))
        assert (b.to_numpy(np.uint16, (n,)) == O.normal_bf16(n, 42, tid, sigma, absval)).all()
    b = DevBuf(n * 4)
    check(kxlib.kx_fill_normal_f32(b.ptr, n, 42, 5, 0.01, None))
    check(kxlib.kx_sync(None))
    assert (b.to_numpy(np.uint32, (n,)) == O.normal_f32(n, 42, 5, 0.01).view(np.uint32)).all()
    check(kxlib.kx_fill_words_u32(b.ptr, n, 42, 6, None))
    check(kxlib.kx_sync(None))
    assert (b.to_numpy(np.uint32, (n,)) == O.words_u32(n, 42, 6)).all()
    check(kxlib.kx_fill_tokens_u32(b.ptr, n, 42, 4, 163840, None))
    check(kxlib.kx_sync(None))
    assert (b.to_numpy(np.uint32, (n,)) == O.tokens_u32(n, 42, 4, 163840)).all()
    assert kxlib.kx_fill_tokens_u32(b.ptr, n, 42, 4, 0, None) != 0


def test_unpack_and_dequant_bit_exact(kxlib, ox):
    rows, cols = 96, 2048
    packed = O.words_u32(rows * cols // 8, 1, 1).reshape(rows, cols // 8)
    # scales: every finite bf16 pattern appears
    scale = (np.arange(rows * cols // 32, dtype=np.uint32) * 11 % 65536).astype(np.uint16)
    scale[((scale >> 7) & 0xFF) == 0xFF] = 0x3C00
    scale = scale.reshape(rows, cols // 32)
    dp, ds = dev(packed), dev(scale)
    dq, dw = DevBuf(rows * cols), DevBuf(rows * cols * 2)
    check(kxlib.kx_i4_unpack(dp.ptr, dq.ptr, rows, cols, None))
    check(kxlib.kx_i4_dequant(dp.ptr, ds.ptr, dw.ptr, rows, cols, None))
    check(kxlib.kx_sync(None))
    q = np.empty((rows, cols), dtype=np.int8)
    w = np.empty((rows, cols), dtype=np.uint16)
    ox.ox_i4_unpack(ptr(packed), ptr(q), rows, cols)
    ox.ox_i4_dequant(ptr(packed), ptr(scale), ptr(w), rows, cols)
    assert (dq.to_numpy(np.int8, (rows, cols)) == q).all()
    assert (dw.to_numpy(np.uint16, (rows, cols)) == w).all()


def test_dequant_exhaustive_scales(kxlib, ox):
    scales = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    scales = scales[((scales >> 7) & 0xFF) != 0xFF]
    rows = scales.size
    words = np.empty((rows, 4), dtype=np.uint32)
    for p in range(4):
        words[:, p] = sum(((8 * p + j) % 16) << (4 * j) for j in range(8))
    dp, ds, dw = dev(words), dev(scales), DevBuf(rows * 32 * 2)
    check(kxlib.kx_i4_dequant(dp.ptr, ds.ptr, dw.ptr, rows, 32, None))
    check(kxlib.kx_sync(None))
    w = np.empty((rows, 32), dtype=np.uint16)
    ox.ox_i4_dequant(ptr(words), ptr(scales), ptr(w), rows, 32)
    assert (dw.to_numpy(np.uint16, (rows, 32)) == w).all()


@pytest.mark.parametrize("rows,cols,tokens", [
    (2048, 7168, 1),     # BASELINE config 1
    (7168, 2048, 1),     # down_proj shape
    (100, 1024, 3),      # ragged rows, one slice
    (70, 3072, 5),       # three slices, odd token count
    (256, 7168, 8),
    (33, 16384, 2),      # widest supported
])
def test_gemv_parity(kxlib, ox, rows, cols, tokens):
    say(f"i4_gemv rows={rows} cols={cols} tokens={tokens}")
    packed = O.words_u32(rows * cols // 8, 2, 1).reshape(rows, cols // 8)
    scale = O.normal_bf16(rows * cols // 32, 2, 2, 0.02, 1).reshape(rows, cols // 32)
    x = O.normal_bf16(tokens * cols, 2, 3, 1.0).reshape(tokens, cols)
    dp, ds, dx, dy = dev(packed), dev(scale), dev(x), DevBuf(tokens * rows * 2)
    check(kxlib.kx_i4_gemv(dp.ptr, ds.ptr, dx.ptr, dy.ptr, rows, cols, tokens, None))
    check(kxlib.kx_sync(None))
    y = dy.to_numpy(np.uint16, (tokens, rows))
    y1 = np.empty_like(y)
    y0 = np.empty_like(y)
    ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y1), rows, cols, tokens, 1)
    ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y0), rows, cols, tokens, 0)
    assert (y == y1).all(), f"{np.count_nonzero(y != y1)} of {y.size} outputs differ from the kx schedule"
    err = O.max_rel(O.bf16_to_f32(y), O.bf16_to_f32(y0))
    assert err < 1e-2, err


def test_gemv_rejects_bad_shapes(kxlib):
    b = DevBuf(1024)
    assert kxlib.kx_i4_gemv(b.ptr, b.ptr, b.ptr, b.ptr, 8, 1000, 1, None) != 0
    assert b"1024" in kxlib.kx_last_error()
    assert kxlib.kx_i4_gemv(None, b.ptr, b.ptr, b.ptr, 8, 1024, 1, None) != 0
    assert kxlib.kx_i4_gemv(b.ptr, b.ptr, b.ptr, b.ptr, 8, 1024, 0, None) != 0
