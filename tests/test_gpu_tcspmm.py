"""GPU parity of SpMM over the condensed format (ConDense -> MFMA) against the float64 closed
form and the oracle's condense.  Tolerance: rtol 2e-2 (fp16 inputs, fp32 accumulation)."""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets, ops
from sparsetir_amd._lib import SparseTIRError
from helpers import random_csr, spmm_f64

pytestmark = pytest.mark.gpu


def _run(dev, indptr, indices, n, feat, weighted, out_dtype, seed=0):
    t, g = 32, 16
    gptr, tiles, mask = st.condense(indptr, indices, t, g)
    want_fmt = oracle.condense(indptr, indices, t, g)
    for a, b in zip((gptr, tiles, mask), want_fmt):
        assert np.array_equal(a, b)
    m = len(indptr) - 1
    mb = len(gptr) - 1
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, feat)).astype(np.float16)
    a = mask.astype(np.float16)
    vals = np.ones(len(indices), np.float32)
    if weighted:
        # weights per stored (row, col): look the value up through the condensed arrays
        import scipy.sparse as sp
        vals = (0.5 + rng.random(len(indices))).astype(np.float16).astype(np.float32)
        dense = sp.csr_matrix((vals, indices, indptr), shape=(m, n)).toarray()
        for tile in range(mb):
            for grp in range(gptr[tile], gptr[tile + 1]):
                rl, sl = np.nonzero(mask[grp])
                a[grp, rl, sl] = dense[tile * t + rl, tiles[grp, sl]]
    td = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)
    c = torch.full((mb * t * feat,), float("nan"), dtype=out_dtype, device=dev)
    f = ops.build_tcspmm(mb, tiles.shape[0], feat, t, g, n, out_dtype)
    f(td(a.ravel()), td(x.ravel()), c, td(gptr), td(tiles.ravel()))
    torch.cuda.synchronize()
    got = c.float().cpu().numpy().reshape(mb * t, feat)
    want = spmm_f64(indptr, indices, vals, x.astype(np.float32))
    scale = spmm_f64(indptr, indices, np.abs(vals), np.abs(x.astype(np.float32)))
    assert np.all(got[m:] == 0)  # rows added to fill the last tile
    bound = 1e-5 * scale + (2e-2 * np.abs(want) if out_dtype == torch.float16 else 0) + 1e-30
    assert np.all(np.abs(got[:m] - want) <= bound)


@pytest.mark.parametrize("feat", [32, 64, 128, 256, 160])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_tcspmm_small(dev, feat, out_dtype):
    m, n = 1000, 777
    indptr, indices = random_csr(m, n, 20000, feat, skew=1.0)
    _run(dev, indptr, indices, n, feat, weighted=(feat % 64 == 0), out_dtype=out_dtype, seed=feat)


def test_tcspmm_config2_graph(dev):
    g = datasets.config2()
    _run(dev, g["indptr"], g["indices"], g["n"], 128, weighted=False, out_dtype=torch.float32)


def test_tcspmm_empty_tiles_and_errors(dev):
    m, n = 96, 50
    indptr = np.zeros(m + 1, np.int32)
    indptr[40:] = 3  # only row 39 has entries
    indices = np.asarray([1, 7, 9], np.int32)
    _run(dev, indptr, indices, n, 64, weighted=False, out_dtype=torch.float16)
    z = lambda k, dt: torch.zeros(k, dtype=dt, device=dev)
    f = ops.build_tcspmm(1, 1, 32, 16, 16, 4)
    with pytest.raises(SparseTIRError, match="t=32"):
        f(z(256, torch.float16), z(128, torch.float16), z(512, torch.float16), z(2, torch.int32), z(16, torch.int32))


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_tcspmm_hub_tile(dev, out_dtype):
    """One row with 9000 distinct columns: its tile has 563 groups = 282 steps, which the fp32
    path cuts into equal units that meet in atomics; C starts as NaN, so the rows of that tile
    must be cleared first.  Another tile lies just above the length of one unit.  Two feature
    tiles, the second one partial."""
    m, n, feat = 200, 20000, 160
    rng = np.random.default_rng(3)
    deg = rng.integers(0, 12, m)
    deg[77] = 9000
    deg[150] = 530   # 34 groups = 17 steps: just above one unit
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    indices = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]).astype(np.int32)
    _run(dev, indptr, indices, n, feat, weighted=False, out_dtype=out_dtype, seed=9)


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("tiles,feat", [(40, 96), (9, 64), (67, 32)])
def test_tcspmm_every_tile_long(dev, tiles, feat, out_dtype):
    """Rows of about 40 entries over 3000 columns: every row tile has more than a thousand
    distinct columns, i.e. 35 to 40 steps.  With fp16 output a workgroup of the launch for long
    tiles then works on several tiles in turn (it looks at eight, a whole grid apart); tile counts
    that are and are not multiples of eight, and a last tile with fewer than 32 rows."""
    m, n = tiles * 32 - 5, 3000
    indptr, indices = random_csr(m, n, 40 * m, tiles, skew=0.0)
    _run(dev, indptr, indices, n, feat, weighted=False, out_dtype=out_dtype, seed=tiles)
