"""GPU parity of SpMM over the condensed format (ConDense -> MFMA) against the float64 closed
form and the oracle's condense.  Tolerance: rtol 2e-2 (fp16 inputs, fp32 accumulation)."""
import numpy as np
import pytest
import torch

import ctypes

import oracle
import sparsetir_amd as st
from sparsetir_amd import _lib, datasets, ops
from sparsetir_amd._lib import SparseTIRError
from helpers import random_csr, spmm_f64

pytestmark = pytest.mark.gpu
STIR_F16, STIR_F32 = 0, 2  # include/sparsetir_amd.h


def _run(dev, indptr, indices, n, feat, weighted, out_dtype, seed=0, t=32):
    g = 16
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
    want = spmm_f64(indptr, indices, vals, x.astype(np.float32))
    scale = spmm_f64(indptr, indices, np.abs(vals), np.abs(x.astype(np.float32)))
    bound = 1e-5 * scale + (2e-2 * np.abs(want) if out_dtype == torch.float16 else 0) + 1e-30
    d_a, d_x, d_ptr, d_tiles = td(a.ravel()), td(x.ravel()), td(gptr), td(tiles.ravel())

    def check(c, what):
        torch.cuda.synchronize()
        got = c.float().cpu().numpy().reshape(mb * t, feat)
        assert np.all(got[m:] == 0), what  # rows added to fill the last tile
        assert np.all(np.abs(got[:m] - want) <= bound), what

    # the built operator: it makes a plan from the group counts at its first call
    c = torch.full((mb * t * feat,), float("nan"), dtype=out_dtype, device=dev)
    f = ops.build_tcspmm(mb, tiles.shape[0], feat, t, g, n, out_dtype)
    f(d_a, d_x, c, d_ptr, d_tiles)
    check(c, "operator, first call")
    c.fill_(float("nan"))
    f(d_a, d_x, c, d_ptr, d_tiles)
    check(c, "operator, with its plan")
    # calls back to back leave the plan's piece counters at zero each time, and the sums of the
    # partial tiles do not depend on which workgroup finishes last: the same bits every time
    again = [torch.full_like(c, float("nan")) for _ in range(4)]
    for y in again:
        f(d_a, d_x, y, d_ptr, d_tiles)
    torch.cuda.synchronize()
    for y in again:
        assert torch.equal(y, c), "operator, repeated calls"
    # and the entry point that takes no plan
    c.fill_(float("nan"))
    vp = lambda v: ctypes.c_void_p(v.data_ptr() if v.numel() else 0)
    _lib.check(_lib.lib().stir_tc_spmm_f16(STIR_F16 if out_dtype == torch.float16 else STIR_F32, mb, t, g, feat,
                                           tiles.shape[0], vp(d_a), vp(d_x), vp(c), vp(d_ptr), vp(d_tiles),
                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    check(c, "without a plan")


# tile sizes: 8 and 16 are what the reference condenses with (tile_size = mma_m of m8n32k16 and
# m16n16k16, examples/spmm/bench_tc_spmm.py:584-585,670), 32 fills the 32x32x16 instruction
TILES = [8, 16, 32]


@pytest.mark.parametrize("t", TILES)
@pytest.mark.parametrize("feat", [32, 64, 128, 256, 160])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_tcspmm_small(dev, feat, out_dtype, t):
    m, n = 1000 + t // 8, 777  # the last tile is partial at every tile size
    indptr, indices = random_csr(m, n, 20000, feat, skew=1.0)
    _run(dev, indptr, indices, n, feat, weighted=(feat % 64 == 0), out_dtype=out_dtype, seed=feat, t=t)


@pytest.mark.parametrize("t,out_dtype", [(8, torch.float16), (16, torch.float16), (32, torch.float32),
                                         (16, torch.float32)])
def test_tcspmm_config2_graph(dev, t, out_dtype):
    g = datasets.config2()
    _run(dev, g["indptr"], g["indices"], g["n"], 128, weighted=False, out_dtype=out_dtype, t=t)


def test_tcspmm_empty_tiles_and_errors(dev):
    m, n = 96, 50
    indptr = np.zeros(m + 1, np.int32)
    indptr[40:] = 3  # only row 39 has entries
    indices = np.asarray([1, 7, 9], np.int32)
    _run(dev, indptr, indices, n, 64, weighted=False, out_dtype=torch.float16)
    z = lambda k, dt: torch.zeros(k, dtype=dt, device=dev)
    _run(dev, indptr, indices, n, 64, weighted=False, out_dtype=torch.float16, t=8)
    _run(dev, indptr, indices, n, 32, weighted=False, out_dtype=torch.float32, t=16)
    # a tile size without a matrix-core shape, and a group size other than the k extent
    for t, g in ((4, 16), (16, 8)):
        f = ops.build_tcspmm(1, 1, 32, t, g, 4)
        with pytest.raises(SparseTIRError, match="t in"):
            f(z(t * g, torch.float16), z(128, torch.float16), z(t * 32, torch.float16), z(2, torch.int32),
              z(g, torch.int32))


@pytest.mark.parametrize("t", TILES)
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_tcspmm_hub_tile(dev, out_dtype, t):
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
    _run(dev, indptr, indices, n, feat, weighted=False, out_dtype=out_dtype, seed=9, t=t)


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("tiles,feat,t", [(40, 96, 32), (9, 64, 32), (67, 32, 32), (40, 96, 16), (67, 32, 16)])
def test_tcspmm_every_tile_long(dev, tiles, feat, out_dtype, t):
    """Rows of about 40 entries over 3000 columns: every row tile has more than a thousand
    distinct columns, i.e. 35 to 40 steps.  With fp16 output a workgroup of the launch for long
    tiles then works on several tiles in turn (it looks at eight, a whole grid apart); tile counts
    that are and are not multiples of eight, and a last tile with fewer than 32 rows."""
    m, n = tiles * 32 - 5, 3000
    per_row = 40 * 32 // t  # 16-row tiles of 80 entries per row reach the same 35 to 40 steps
    indptr, indices = random_csr(m, n, per_row * m, tiles, skew=0.0)
    _run(dev, indptr, indices, n, feat, weighted=False, out_dtype=out_dtype, seed=tiles, t=t)


@pytest.mark.parametrize("t", [32, 8])
def test_tcspmm_plan_entry_points(dev, t):
    """stir_tc_plan_create / stir_tc_spmm_f16_planned through the C ABI: one plan used at three
    feature widths in turn (its memory for partial tiles grows with the widest), a plan for a
    matrix without long tiles, the row-tile count checked against the plan's, and an in-place
    change of the group counts followed by the operator's invalidate()."""
    L = _lib.lib()
    g = 16
    m, n = 300, 12000
    rng = np.random.default_rng(41)
    deg = rng.integers(0, 10, m)
    deg[5], deg[130], deg[131], deg[299] = 7000, 2200, 300, 4100   # tiles of 219, 76 and 129 steps
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    indices = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]).astype(np.int32)
    gptr, tiles, mask = st.condense(indptr, indices, t, g)
    mb, nnzb = len(gptr) - 1, tiles.shape[0]
    td = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)
    vp = lambda v: ctypes.c_void_p(v.data_ptr() if v.numel() else 0)
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    d_a, d_ptr, d_tiles = td(mask.astype(np.float16).ravel()), td(gptr), td(tiles.ravel())
    plan = ctypes.c_void_p()
    _lib.check(L.stir_tc_plan_create(ctypes.byref(plan), mb, vp(d_ptr), stream()))
    try:
        for feat, dt in ((64, torch.float16), (256, torch.float32), (96, torch.float16), (256, torch.float16)):
            x = rng.standard_normal((n, feat)).astype(np.float16)
            c = torch.full((mb * t * feat,), float("nan"), dtype=dt, device=dev)
            _lib.check(L.stir_tc_spmm_f16_planned(plan, STIR_F16 if dt == torch.float16 else STIR_F32, mb, t, g, feat,
                                                  nnzb, vp(d_a), vp(td(x.ravel())), vp(c), vp(d_ptr), vp(d_tiles),
                                                  stream()))
            torch.cuda.synchronize()
            got = c.float().cpu().numpy().reshape(mb * t, feat)[:m]
            ones = np.ones(len(indices), np.float32)
            want = spmm_f64(indptr, indices, ones, x.astype(np.float32))
            scale = spmm_f64(indptr, indices, ones, np.abs(x.astype(np.float32)))
            rtol = 2e-2 if dt == torch.float16 else 0.0
            assert np.all(np.abs(got - want) <= rtol * np.abs(want) + 1e-5 * scale + 1e-30), (feat, dt)
        assert L.stir_tc_spmm_f16_planned(plan, STIR_F16, mb + 1, t, g, 64, nnzb, vp(d_a), vp(d_a), vp(d_a),
                                          vp(d_ptr), vp(d_tiles), stream()) == -1
        assert b"row tiles" in L.stir_last_error()
        assert L.stir_tc_spmm_f16_planned(plan, 1, mb, t, g, 64, nnzb, vp(d_a), vp(d_a), vp(d_a), vp(d_ptr),
                                          vp(d_tiles), stream()) == -1  # bf16 output does not exist
        assert b"out_dtype" in L.stir_last_error()
    finally:
        L.stir_tc_plan_destroy(plan)

    # no long tile at all: the plan is empty and the launch is the first kernel alone
    indptr2, indices2 = random_csr(200, 500, 1500, 7, skew=0.0)
    _run(dev, indptr2, indices2, 500, 64, weighted=False, out_dtype=torch.float16, t=t)

    # the operator after its indptr array was rewritten in place: invalidate() makes a new plan
    feat = 64
    x = rng.standard_normal((n, feat)).astype(np.float16)
    f = ops.build_tcspmm(mb, nnzb, feat, t, g, n, torch.float16)
    c = torch.zeros(mb * t * feat, dtype=torch.float16, device=dev)
    f(d_a, td(x.ravel()), c, d_ptr, d_tiles)
    # the rows of tile 0 (the longest) and of tile 6 change places: the same groups, other tiles long
    rows = [*range(192, 224), *range(32, 192), *range(0, 32), *range(224, m)]
    indptr3 = np.concatenate([[0], np.cumsum(deg[rows])]).astype(np.int32)
    indices3 = np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in rows])
    gptr3, tiles3, mask3 = st.condense(indptr3, indices3, t, g)
    assert tiles3.shape[0] == nnzb  # the same number of groups: the arrays can be rewritten in place
    ones = np.ones(len(indices3), np.float32)
    want3 = spmm_f64(indptr3, indices3, ones, x.astype(np.float32))
    scale3 = spmm_f64(indptr3, indices3, ones, np.abs(x.astype(np.float32)))

    def agrees():
        c.fill_(float("nan"))
        f(d_a, td(x.ravel()), c, d_ptr, d_tiles)
        torch.cuda.synchronize()
        got = c.float().cpu().numpy().reshape(mb * t, feat)[:m]
        return np.all(np.abs(got - want3) <= 2e-2 * np.abs(want3) + 1e-5 * scale3 + 1e-30)

    # rewritten through torch: the operator notices by itself
    d_ptr.copy_(td(gptr3)), d_tiles.copy_(td(tiles3.ravel())), d_a.copy_(td(mask3.astype(np.float16).ravel()))
    assert agrees()
    # rewritten behind torch's back (a plain hipMemcpy to the array's address): invalidate() is the
    # caller's part
    import ctypes as ct
    hip = ct.CDLL("libamdhip64.so")
    back = np.ascontiguousarray(gptr)
    assert hip.hipMemcpy(ct.c_void_p(d_ptr.data_ptr()), back.ctypes.data_as(ct.c_void_p), ct.c_size_t(back.nbytes), 1) == 0
    d_tiles.copy_(td(tiles.ravel())), d_a.copy_(td(mask.astype(np.float16).ravel()))
    f.invalidate()
    c.fill_(float("nan"))
    f(d_a, td(x.ravel()), c, d_ptr, d_tiles)
    torch.cuda.synchronize()
    got = c.float().cpu().numpy().reshape(mb * t, feat)[:m]
    ones = np.ones(len(indices), np.float32)
    want = spmm_f64(indptr, indices, ones, x.astype(np.float32))
    scale = spmm_f64(indptr, indices, ones, np.abs(x.astype(np.float32)))
    assert np.all(np.abs(got - want) <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30)

