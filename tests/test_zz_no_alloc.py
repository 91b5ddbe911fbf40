"""kx_lm_head_argmax_static -- the entry point that allocates nothing -- against kx_lm_head_argmax.

The two share their kernels; what differs is where the argmax partials live (a device array inside the library
instead of the caller's buffer).  Logits and ids must agree to the bit, on two calls in a row of which the
second is smaller (fewer rows, a shorter vocabulary): the array then still holds the first call's partials.
The second test checks the property the entry point is named for: device memory free before a call = free after it.
"""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from blok_amd.lib import DevBuf, check
from kxt import dev, say


def _run_both(kxlib, vocab, hidden, tokens, seed):
    w = O.normal_bf16(vocab * hidden, seed, 1, 0.02).reshape(vocab, hidden)
    x = O.normal_bf16(tokens * hidden, seed, 2, 1.0).reshape(tokens, hidden)
    dw, dx = dev(w), dev(x)
    res = []
    for static in (False, True):
        dl, di = DevBuf(tokens * vocab * 4), DevBuf(tokens * 4)
        check(kxlib.kx_dev_memset(dl.ptr, 0xFF, tokens * vocab * 4, None))
        check(kxlib.kx_dev_memset(di.ptr, 0xFF, tokens * 4, None))
        if static:
            check(kxlib.kx_lm_head_argmax_static(dw.ptr, dx.ptr, dl.ptr, di.ptr, vocab, hidden, tokens, None))
        else:
            ds = DevBuf(tokens * 512)
            check(kxlib.kx_lm_head_argmax(dw.ptr, dx.ptr, dl.ptr, di.ptr, vocab, hidden, tokens, ds.ptr, None))
        check(kxlib.kx_sync(None))
        res.append((dl.to_numpy(np.uint32, (tokens, vocab)), di.to_numpy(np.uint32, (tokens,))))
    return res


@pytest.mark.gpu
def test_static_entry_point_matches_the_allocating_one(kxlib):
    check(kxlib.kx_static_scratch_init())
    for vocab, hidden, tokens, seed in ((6000, 1024, 7, 21), (1500, 512, 2, 22)):
        say(f"lm_head_argmax_static vocab={vocab} hidden={hidden} tokens={tokens}")
        (l0, i0), (l1, i1) = _run_both(kxlib, vocab, hidden, tokens, seed)
        assert (l0 == l1).all(), f"{np.count_nonzero(l0 != l1)} logits differ"
        assert (i0 == i1).all(), (i0, i1)
        assert (i0 < vocab).all()


@pytest.mark.gpu
def test_static_entry_point_takes_no_device_memory(kxlib):
    check(kxlib.kx_static_scratch_init())
    vocab, hidden, tokens = 3000, 512, 5
    w = O.normal_bf16(vocab * hidden, 23, 1, 0.02).reshape(vocab, hidden)
    x = O.normal_bf16(tokens * hidden, 23, 2, 1.0).reshape(tokens, hidden)
    dw, dx, dl, di = dev(w), dev(x), DevBuf(tokens * vocab * 4), DevBuf(tokens * 4)

    def free_now():
        free, total = C.c_size_t(), C.c_size_t()
        check(kxlib.kx_dev_mem_info(C.byref(free), C.byref(total)))
        return free.value

    check(kxlib.kx_lm_head_argmax_static(dw.ptr, dx.ptr, dl.ptr, di.ptr, vocab, hidden, tokens, None))   # code objects, streams: loaded
    check(kxlib.kx_sync(None))
    before = free_now()
    for _ in range(3):
        check(kxlib.kx_lm_head_argmax_static(dw.ptr, dx.ptr, dl.ptr, di.ptr, vocab, hidden, tokens, None))
        assert free_now() == before, "a call of the entry point that allocates nothing changed the free device memory"
    check(kxlib.kx_sync(None))
    assert free_now() == before


@pytest.mark.gpu
def test_static_entry_point_rejects_more_rows_than_it_holds(kxlib):
    b = DevBuf(4096)
    assert kxlib.kx_lm_head_argmax_static(b.ptr, b.ptr, b.ptr, b.ptr, 512, 512, 257, None) != 0
    assert b"256" in kxlib.kx_last_error()
