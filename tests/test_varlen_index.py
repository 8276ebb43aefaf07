"""Integer index oracle: closed forms vs brute force, exhaustively on small cases and on the
reference's own stress lists (tests/test_varlen.py:60-73)."""
import itertools
import random

import numpy as np
import pytest

from oracle import varlen_index as VI


def cu_of(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def test_chunk_size_rule():
    assert [VI.chunk_size_for(t) for t in (1, 15, 16, 17, 32, 33, 64, 65, 10 ** 6)] == [16, 16, 16, 32, 32, 64, 64, 64, 64]


@pytest.mark.parametrize("bt", [2, 3, 4])
def test_exhaustive_small(bt):
    for n in (1, 2, 3):
        for lens in itertools.product(range(1, 2 * bt + 2), repeat=n):
            cu = cu_of(lens)
            a, b = VI.chunk_tables_closed(cu, bt), VI.chunk_tables_brute(cu, bt)
            assert a[0].dtype == np.int32 and np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    for lens in itertools.product(range(1, 7), repeat=3):
        cu = cu_of(lens)
        for wl, shift in [(-1, 0), (0, 0), (1, 2), (2, 0), (3, 4), (2, 3)]:
            for x, y in zip(VI.token_tables_closed(cu, wl, shift), VI.token_tables_brute(cu, wl, shift)):
                assert np.array_equal(x, y)


def test_reference_stress_lists():
    random.seed(0)
    cases = [[128] * 4, [128, 64, 200, 10], [4096, 2048, 1, 1024, 2],
             [random.randint(1, 100) for _ in range(256)], [1, 2000, 3, 50, 4, 3000, 2, 7]]
    for lens in cases:
        cu = cu_of(lens)
        a, b = VI.chunk_tables_closed(cu, 64), VI.chunk_tables_brute(cu, 64)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        assert a[1][-1] == sum((L + 63) // 64 for L in lens)
    lens = [1, 200, 3, 50, 4, 300, 2, 7]
    cu = cu_of(lens)
    for x, y in zip(VI.token_tables_closed(cu, 31, 32), VI.token_tables_brute(cu, 31, 32)):
        assert np.array_equal(x, y)
