"""GPU test of nerva_hip_argmax_static, the entry point that allocates nothing.

It must return what nerva_hip_argmax returns (bit-exact: an index) on two calls in a row, the
second over a smaller input, with no allocation counted by the library while it runs, and it
must refuse counts above its stated maximum without launching.
"""
import ctypes as C

import numpy as np
import pytest

import nerva_amd as N
import oracle as O
from nerva_amd import abi

pytestmark = pytest.mark.gpu


def test_argmax_static_matches_argmax_on_two_calls_second_smaller():
    rc, res = N.Device.smoke()   # the library's init call: resolves the scratch address, creates the stream
    assert rc == 0 and res.status == 0
    rng = np.random.default_rng(11)
    big = rng.normal(0, 3, 151936).astype(np.float32)
    big[[5, 140000]] = big.max() + 1.0          # a tie: the lower index wins
    big[77] = np.inf                            # non-finite values are skipped
    small = rng.normal(0, 3, 1000).astype(np.float32)
    small[999] = small.max() + 2.0              # the winner sits past every workgroup but the first
    tiny = np.array([np.nan, -1.0, -1.0], np.float32)
    bufs = [N.DeviceBuffer.from_numpy(a) for a in (big, small, tiny)]
    token = N.DeviceBuffer.zeros(16)
    before = N.Device.allocation_count()
    got = []
    for a, b in zip((big, small, tiny), bufs):
        rc, err = N.argmax_static(b, a.size, token)
        assert rc == 0 and err == 0
        got.append(int(token.numpy(np.uint32, 1)[0]))
    assert N.Device.allocation_count() == before, "the static entry point allocated"
    want = [N.argmax(b, a.size) for a, b in zip((big, small, tiny), bufs)]
    assert got == want == [5, 999, 1]
    assert got == [O.greedy_argmax(a, skip_nonfinite=True) for a in (big, small, tiny)]
    # the same two calls again, after the candidate array has held other contents
    for a, b, w in zip((big, small), bufs, want):
        rc, err = N.argmax_static(b, a.size, token)
        assert rc == 0 and int(token.numpy(np.uint32, 1)[0]) == w


def test_argmax_static_rejects_bad_arguments_without_launching():
    lib = abi.load()
    logits = N.DeviceBuffer.zeros(64)
    token = N.DeviceBuffer.from_numpy(np.array([12345], np.uint32))
    err = C.c_int32(0)
    over = abi.NERVA_HIP_ARGMAX_STATIC_MAX_COUNT + 1
    assert lib.nerva_hip_argmax_static(logits.ptr, over, token.ptr, None, C.byref(err)) == -1 and err.value == 1
    assert lib.nerva_hip_argmax_static(logits.ptr, 0, token.ptr, None, C.byref(err)) == -1
    assert lib.nerva_hip_argmax_static(None, 4, token.ptr, None, C.byref(err)) == -1
    assert lib.nerva_hip_argmax_static(logits.ptr, 4, None, None, C.byref(err)) == -1
    N.Device.synchronize()
    assert int(token.numpy(np.uint32, 1)[0]) == 12345
