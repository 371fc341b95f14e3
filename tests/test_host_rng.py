"""Host logic (no GPU): the library's restatement of numpy's legacy MT19937
stream gives the block coordinates np.random.seed / np.random.randint give
(the calls of gt_sp/utils.py:290-295)."""
import ctypes

import numpy as np
import pytest

from torchgt_amd import _lib


@pytest.mark.parametrize("seed", [0, 1, 7, 12345, 2**31 + 5])
def test_legacy_randint_stream_matches_numpy(seed):
    highs = np.array([2, 2, 1, 3, 256, 1000, 1, 4096, 54321, 7, 2**20, 5, 1, 1, 9] * 50, dtype=np.int64)
    out = np.empty_like(highs)
    L = _lib.lib()
    rc = L.tgt_np_legacy_randint(seed, highs.ctypes.data_as(ctypes.c_void_p), len(highs),
                                 out.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    np.random.seed(seed)
    expect = np.array([np.random.randint(0, int(h)) for h in highs], dtype=np.int64)
    np.testing.assert_array_equal(out, expect)


def test_legacy_randint_crosses_state_refill():
    highs = np.full(2000, 3, dtype=np.int64)       # > 624 draws: the state is regenerated several times
    out = np.empty_like(highs)
    assert _lib.lib().tgt_np_legacy_randint(3, highs.ctypes.data_as(ctypes.c_void_p), len(highs),
                                            out.ctypes.data_as(ctypes.c_void_p)) == 0
    rs = np.random.RandomState(3)
    np.testing.assert_array_equal(out, [rs.randint(0, 3) for _ in range(2000)])
