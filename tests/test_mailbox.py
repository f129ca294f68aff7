"""The word a ReLU classification kernel posts to the host (call number | crossing count | inactive
count) and the rule by which the host tells a fresh word from a stale one.

The host-side helpers are plain C functions of the library (no device call), so the packing and the
wrap of the 16-bit call number are checked on the CPU; the GPU test drives a context across the wrap."""
import ctypes as C
import os

import numpy as np
import pytest

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nnv_amd", "libnnvhip.so")
EMPTY = (1 << 64) - 1

needs_lib = pytest.mark.skipif(not os.path.exists(LIB), reason="library not built (python -m nnv_amd.build)")


def _pack(lib, m, inactive, call):
    w = C.c_uint64()
    assert lib.nnvhip_debug_mailbox_pack(m, inactive, call, C.byref(w)) == 0
    return w.value


def _unpack(lib, w):
    posted, m, inactive, call = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
    assert lib.nnvhip_debug_mailbox_unpack(C.c_uint64(w), C.byref(posted), C.byref(m), C.byref(inactive), C.byref(call)) == 0
    return posted.value, m.value, inactive.value, call.value


@needs_lib
def test_word_layout_and_round_trip():
    from nnv_amd import _lib
    lib = _lib.load()
    # layout: call number in bits 48..63, crossing count in bits 24..47, inactive count in bits 0..23
    assert _pack(lib, 1, 0, 0) == 1 << 24 and _pack(lib, 0, 1, 0) == 1 and _pack(lib, 0, 0, 1) == 1 << 48
    rs = np.random.RandomState(0)
    for _ in range(2000):
        N = int(rs.randint(1, 1 << 24))
        m = int(rs.randint(0, N + 1))
        inactive = int(rs.randint(0, N - m + 1))
        call = int(rs.randint(0, 1 << 31))
        w = _pack(lib, m, inactive, call)
        assert _unpack(lib, w) == (1, m, inactive, call & 0xffff)


@needs_lib
def test_no_posted_word_equals_the_empty_pattern_and_stale_words_are_not_fresh():
    from nnv_amd import _lib
    lib = _lib.load()
    assert _unpack(lib, EMPTY)[0] == 0
    top = (1 << 24) - 1            # largest dimension the mailbox path serves is 2^24 - 1
    # the counts of one set add up to at most its dimension: the extreme words of every call number
    for call in (0, 1, 0x7fff, 0xfffe, 0xffff, 0x10000, 0x1ffff, 65536 * 7):
        for m, inactive in ((0, 0), (top, 0), (0, top), (top // 2, top - top // 2), (1, top - 1)):
            assert m + inactive <= top
            w = _pack(lib, m, inactive, call)
            assert w != EMPTY and _unpack(lib, w)[0] == 1
    # a word last written 65536 calls ago carries the same 16-bit call number as the current call: the
    # number alone cannot tell them apart (which is why the host clears the word before the launch) ...
    stale = _pack(lib, 5, 7, 123)
    assert _unpack(lib, stale)[3] == _unpack(lib, _pack(lib, 0, 0, 123 + 65536))[3]
    # ... and the zero-filled word of a context that never posted looks like call 0 with no crossing
    # neuron: it, too, is only ruled out by the empty pattern
    assert _unpack(lib, 0) == (1, 0, 0, 0)
    assert _unpack(lib, _pack(lib, 0, 0, 65536)) == (1, 0, 0, 0)


@pytest.mark.gpu
def test_relu_calls_across_the_wrap_of_the_call_number():
    """Single-set calls up to and past call 65536 of a context, then an array call whose higher words were
    last written many calls earlier: every count must be the set's own."""
    import nnv_amd
    from nnv_amd import _lib
    from oracle import nnv_oracle as o
    ctx = nnv_amd.default_context()
    lib = ctx.lib
    rs = np.random.RandomState(11)
    N, n = 48, 6
    stars, expect = [], []
    for k in range(12):
        V = rs.randn(N, n + 1)
        V[:, 0] += 1.2 * k - 6.0          # different centres: different counts from set to set
        S = nnv_amd.Star(V, np.zeros((1, n)), np.zeros(1))
        lb, ub = o.estimate_ranges(o.OStar(V, np.zeros((1, n)), np.zeros(1), -np.ones(n), np.ones(n)))
        stars.append(S)
        expect.append((int(np.sum(ub <= 0)), int(np.sum((lb < 0) & (ub > 0)))))
    assert len(set(expect)) > 8

    def relu(sets):
        arr = (C.c_void_p * len(sets))(*[s._h.h for s in sets])
        out = (C.c_void_p * len(sets))()
        _lib.check(lib.nnvhip_relu_relax(ctx.handle, _lib.ORDER_AREA, 1.0, len(sets), arr, out))
        got = []
        for h in out:
            ni, nc = C.c_int64(), C.c_int64()
            _lib.check(lib.nnvhip_star_relu_counts(h, C.byref(ni), C.byref(nc)))
            got.append((ni.value, nc.value))
            _lib.check(lib.nnvhip_star_release(h))
        return got

    # an array call first: words 1..11 are written now and not again until the second array call
    assert relu(stars) == expect
    _lib.check(lib.nnvhip_debug_set_relu_call_number(ctx.handle, 65536 - 40))
    for t in range(80):                      # crosses call number 0xffff -> 0x0000
        k = t % len(stars)
        assert relu([stars[k]]) == [expect[k]], "single-set call %d" % t
    # exactly 65536 calls after the first array call its words carry this call's 16-bit number again
    _lib.check(lib.nnvhip_debug_set_relu_call_number(ctx.handle, 65536))
    rev = stars[::-1]
    assert relu(rev) == expect[::-1]
    # the long way: more than 65536 real calls on one context
    _lib.check(lib.nnvhip_debug_set_relu_call_number(ctx.handle, 0))
    one = (C.c_void_p * 1)()
    for t in range(66000):
        k = t % len(stars)
        arr = (C.c_void_p * 1)(stars[k]._h.h)
        _lib.check(lib.nnvhip_relu_relax(ctx.handle, _lib.ORDER_INDEX, 1.0, 1, arr, one))
        ni, nc = C.c_int64(), C.c_int64()
        _lib.check(lib.nnvhip_star_relu_counts(one[0], C.byref(ni), C.byref(nc)))
        assert (ni.value, nc.value) == expect[k], "call %d" % t
        _lib.check(lib.nnvhip_star_release(one[0]))
    assert relu(stars) == expect
