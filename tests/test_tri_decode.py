"""The triangular index decode of the triplet kernels (csrc/staf_common.hpp: tri_decode, the branch for up to 255
neighbours): j = trunc((t - sqrt(t^2 - 8 nn - 4)) / 2) with t = 2 m - 1, in single precision, is the row of pair nn
for every m <= 255 and every nn -- also when the square root is off by up to two units in the last place, which
covers the hardware instruction's stated 1 ulp.  The reference enumerates the pairs row by row
(STAF/src/descriptor_builder/reforce.cu.cc:137-146); that numbering is the ground truth here."""
import numpy as np
import pytest


def rows_by_enumeration(m):
    j = np.repeat(np.arange(m - 1), np.arange(m - 1, 0, -1))
    k = np.concatenate([np.arange(a + 1, m) for a in range(m - 1)]) if m > 1 else np.zeros(0, int)
    return j, k


@pytest.mark.parametrize("ulps", [-2, -1, 0, 1, 2])
def test_biased_root_gives_the_row_without_correction(ulps):
    for m in range(2, 256):
        j_true, k_true = rows_by_enumeration(m)
        nn = np.arange(m * (m - 1) // 2, dtype=np.int64)
        t = 2 * m - 1
        root = np.sqrt((t * t - 4 - 8 * nn).astype(np.float32))
        for _ in range(abs(ulps)):
            root = np.nextafter(root, np.float32(np.inf if ulps > 0 else -np.inf))
        j = ((np.float32(t) - root) * np.float32(0.5)).astype(np.int32)   # the conversion truncates
        k = nn - ((j.astype(np.int64) * (t - j)) >> 1) + j + 1
        assert np.array_equal(j, j_true), m
        assert np.array_equal(k, k_true), m
