"""Device-side ColumnPartHyb: index arrays bit-exact with the oracle."""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets
from sparsetir_amd._lib import SparseTIRError
from helpers import coo_pairs, decode_hyb, random_csr

pytestmark = pytest.mark.gpu


def _device_hyb(dev, m, n, indptr, indices, parts, buckets):
    r, c, k = st.column_part_hyb(m, n, torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev),
                                 parts, buckets)
    tonp = lambda nest: [[a.cpu().numpy() for a in p] for p in nest]
    return tonp(r), tonp(c), tonp(k)


@pytest.mark.parametrize("m,n,nnz,parts,buckets,seed", [
    (1000, 1000, 10000, 4, [1, 2, 4], 0),
    (2000, 1500, 60000, 2, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512], 1),
    (513, 77, 9000, 16, [1, 2, 4, 8, 16, 32], 2),
    (100, 100, 0, 3, [1, 2], 3),
    (64, 4096, 20000, 5, [3, 5, 9], 5),
    (300, 300, 5000, 1, [1], 6),
    (50, 7, 300, 7, [1, 2, 4], 7),
    (63, 63, 900, 2, [1, 2, 4, 8], 8),
    (65, 200, 5000, 3, [1, 2], 9),
])
def test_device_column_part_hyb_bit_exact(dev, m, n, nnz, parts, buckets, seed):
    indptr, indices = random_csr(m, n, nnz, seed, skew=1.1)
    got = _device_hyb(dev, m, n, indptr, indices, parts, buckets)
    want = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    for name, g, w in zip(["rows", "cols", "mask"], got, want):
        for p in range(parts):
            for b in range(len(buckets)):
                assert g[p][b].shape == w[p][b].shape, (name, p, b)
                assert np.array_equal(g[p][b], w[p][b]), (name, p, b)


def test_device_column_part_hyb_config2(dev):
    g = datasets.config2()
    got = _device_hyb(dev, g["m"], g["n"], g["indptr"], g["indices"], g["num_col_parts"], g["buckets"])
    want = oracle.column_part_hyb(g["m"], g["n"], g["indptr"], g["indices"], g["num_col_parts"], g["buckets"])
    for gq, wq in zip(got, want):
        for gp, wp in zip(gq, wq):
            for a, b in zip(gp, wp):
                assert np.array_equal(a, b)
    assert np.array_equal(decode_hyb(*got), coo_pairs(g["indptr"], g["indices"]))


def test_device_column_part_hyb_rejects_unsorted_and_out_of_range(dev):
    indptr, indices = random_csr(50, 40, 600, 3, sort=False)
    with pytest.raises(SparseTIRError, match="ascend"):
        _device_hyb(dev, 50, 40, indptr, indices, 2, [1, 2, 4])
    bad = np.asarray([0, 50], np.int32)
    with pytest.raises(SparseTIRError, match="outside"):
        _device_hyb(dev, 2, 40, np.asarray([0, 1, 2], np.int32), bad, 2, [1, 2])
