"""cai_argmax_noalloc (the entry point that allocates nothing) against cai_argmax, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

from helpers.device import dev

pytestmark = pytest.mark.gpu


class DevBuf:
    def __init__(self, cai, nbytes):
        self.cai, self.p = cai, C.c_void_p()
        cai.check(cai.load().cai_dev_alloc(nbytes, C.byref(self.p)))

    def close(self):
        self.cai.check(self.cai.load().cai_dev_free(self.p))


def _noalloc(cai, xd, out_d, x):
    L = cai.load()
    cai.check(L.cai_dev_upload(xd.p, C.c_void_p(x.ctypes.data), x.nbytes))
    cai.check(L.cai_argmax_noalloc(xd.p, x.size, out_d.p))
    cai.check(L.cai_sync())
    got = np.zeros(1, np.int32)
    cai.check(L.cai_dev_download(C.c_void_p(got.ctypes.data), out_d.p, 4))
    return int(got[0])


def _existing(cai, x):
    got = C.c_int32(-1)
    cai.check(cai.load().cai_argmax(C.c_void_p(x.ctypes.data), x.size, C.byref(got), 0))
    return got.value


def test_two_calls_in_a_row_second_smaller():
    cai = dev()
    rng = np.random.default_rng(424242)
    big = rng.standard_normal(152064).astype(np.float32)
    big[150000] = 50.0                      # winner in a high slice: a stale slot would beat everything in the next call
    small = rng.standard_normal(5000).astype(np.float32)
    small[[17, 4100]] = 9.0                 # a tie across two slices: the lower index wins
    xd, out_d = DevBuf(cai, big.nbytes), DevBuf(cai, 4)
    try:
        assert _noalloc(cai, xd, out_d, big) == _existing(cai, big) == 150000
        assert _noalloc(cai, xd, out_d, small) == _existing(cai, small) == 17
        for n in (1, 63, 4096, 4097, 49152):
            x = rng.standard_normal(n).astype(np.float32)
            assert _noalloc(cai, xd, out_d, x) == _existing(cai, x) == int(np.argmax(x))
    finally:
        xd.close(); out_d.close()


def test_sizes_beyond_the_fixed_scratch_are_refused():
    cai = dev()
    out_d = DevBuf(cai, 4)
    try:
        rc = cai.load().cai_argmax_noalloc(out_d.p, 4096 * 1024 + 1, out_d.p)   # refused before anything is launched
        assert rc == -1 and "exceed" in cai.last_error()
    finally:
        out_d.close()
