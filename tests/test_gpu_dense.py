"""GPU parity of RMSNorm and the bf16 GEMV against the oracle (bit-exact vs mode 1,
max-rel 1e-2 vs the reference schedule, mode 0)."""
import numpy as np
import pytest

import oracle as O
from kxt import check, dev, say
from oracle import ptr

pytestmark = pytest.mark.gpu
from blok_amd.lib import DevBuf  # noqa: E402


@pytest.mark.parametrize("n,tokens", [(7168, 3), (1536, 2), (512, 5), (8, 1), (1000, 1)])
def test_rmsnorm_parity(kxlib, ox, n, tokens):
    say(f"rmsnorm n={n} tokens={tokens}")
    x = O.normal_bf16(tokens * n, 3, 1, 1.5).reshape(tokens, n)
    w = O.normal_bf16(n, 3, 2, 1.0)
    dx, dw, dy = dev(x), dev(w), DevBuf(tokens * n * 2)
    check(kxlib.kx_rmsnorm(dx.ptr, dw.ptr, dy.ptr, tokens, n, 1e-5, None))
    check(kxlib.kx_sync(None))
    y = dy.to_numpy(np.uint16, (tokens, n))
    y1, y0 = np.empty_like(y), np.empty_like(y)
    ox.ox_rmsnorm(ptr(x), ptr(w), ptr(y1), tokens, n, 1e-5, 1)
    ox.ox_rmsnorm(ptr(x), ptr(w), ptr(y0), tokens, n, 1e-5, 0)
    assert (y == y1).all()
    assert O.max_rel(O.bf16_to_f32(y), O.bf16_to_f32(y0)) < 1e-2


@pytest.mark.parametrize("rows,cols,tokens,f32", [
    (384, 7168, 1, 1),      # router gate, fp32 logits
    (384, 7168, 8, 1),
    (2112, 7168, 1, 0),     # q_a + kv_a
    (2112, 7168, 2, 0),     # the same for two and four tokens: one workgroup per CU, chunks planned for one round
    (2112, 7168, 4, 0),
    (7168, 8192, 3, 0),     # o_proj, three tokens on the four-token kernel
    (1000, 1536, 3, 0),     # q_b-like, ragged rows
    (128, 512, 2, 0),       # W_UV-like, one slice
    (64, 8192, 1, 0),       # o_proj width
    (40, 18432, 2, 0),      # dense down width (three slices per wave)
    (96, 2048, 5, 0),
    (384, 7168, 32, 1),     # 8 tokens and more against a small matrix: token blocks side by side in the grid
    (384, 7168, 16, 1),
    (8192, 512, 32, 0),     # 32 chunks of 256 rows per token block
    (1000, 1536, 13, 0),    # the same, ragged rows and a ragged last token block
    (2048, 512, 9, 0),
    (384, 1024, 70, 1),     # more than 32 tokens: still one launch
])
def test_gemv_bf16_parity(kxlib, ox, rows, cols, tokens, f32):
    say(f"gemv_bf16 rows={rows} cols={cols} tokens={tokens} f32={f32}")
    w = O.normal_bf16(rows * cols, 4, 1, 0.02).reshape(rows, cols)
    x = O.normal_bf16(tokens * cols, 4, 2, 1.0).reshape(tokens, cols)
    esz = 4 if f32 else 2
    dw, dx, dy = dev(w), dev(x), DevBuf(tokens * rows * esz)
    check(kxlib.kx_gemv_bf16(dw.ptr, dx.ptr, dy.ptr, rows, cols, tokens, f32, None))
    check(kxlib.kx_sync(None))
    dt = np.uint32 if f32 else np.uint16
    y = dy.to_numpy(dt, (tokens, rows))
    y1, y0 = np.empty_like(y), np.empty_like(y)
    ox.ox_gemv_bf16(ptr(w), ptr(x), ptr(y1), rows, cols, tokens, f32, 1)
    ox.ox_gemv_bf16(ptr(w), ptr(x), ptr(y0), rows, cols, tokens, f32, 0)
    assert (y == y1).all(), f"{np.count_nonzero(y != y1)} of {y.size} differ"
    to_f = (lambda a: a.view(np.float32)) if f32 else O.bf16_to_f32
    assert O.max_rel(to_f(y), to_f(y0)) < 1e-2


@pytest.mark.parametrize("vocab,hidden,tokens", [(5000, 1024, 1), (5000, 1024, 3), (777, 512, 9)])
def test_lm_head_argmax_parity(kxlib, ox, vocab, hidden, tokens):
    # logits = bf(W n) to the bit against the oracle's GEMV; the id is the lowest index of the largest rounded logit:
    # the winning row of token 0 is copied to a later row, so that token has an exact tie
    say(f"lm_head_argmax vocab={vocab} hidden={hidden} tokens={tokens}")
    w = O.normal_bf16(vocab * hidden, 6, 1, 0.02).reshape(vocab, hidden)
    x = O.normal_bf16(tokens * hidden, 6, 2, 1.0).reshape(tokens, hidden)
    y1 = np.empty((tokens, vocab), dtype=np.uint16)
    ox.ox_gemv_bf16(ptr(w), ptr(x), ptr(y1), vocab, hidden, tokens, 0, 1)
    first = int(np.argmax(O.bf16_to_f32(y1)[0]))
    later = vocab - 1 if first != vocab - 1 else vocab - 2
    w[max(first, later)] = w[min(first, later)]
    ox.ox_gemv_bf16(ptr(w), ptr(x), ptr(y1), vocab, hidden, tokens, 0, 1)
    exp = O.bf16_to_f32(y1)
    dw, dx = dev(w), dev(x)
    dl, di, ds = DevBuf(tokens * vocab * 4), DevBuf(tokens * 4), DevBuf(tokens * 512)
    check(kxlib.kx_lm_head_argmax(dw.ptr, dx.ptr, dl.ptr, di.ptr, vocab, hidden, tokens, ds.ptr, None))
    check(kxlib.kx_sync(None))
    got = dl.to_numpy(np.float32, (tokens, vocab))
    ids = di.to_numpy(np.uint32, (tokens,))
    assert (got.view(np.uint32) == exp.view(np.uint32)).all()
    assert (ids == np.argmax(exp, axis=1)).all()
    assert ids[0] == min(first, later)


def test_shape_errors(kxlib):
    b = DevBuf(4096)
    assert kxlib.kx_gemv_bf16(b.ptr, b.ptr, b.ptr, 4, 500, 1, 0, None) != 0
    assert b"512" in kxlib.kx_last_error()
    assert kxlib.kx_rmsnorm(b.ptr, b.ptr, b.ptr, 1, 7, 1e-5, None) != 0
    assert kxlib.kx_rmsnorm(None, b.ptr, b.ptr, 1, 8, 1e-5, None) != 0
