"""GPU parity of SDDMM and its row-lookup preprocess against the oracle.
Tolerance: fp32, |got - want| <= 1e-5 * sum_k |a_k b_k| per nonzero (float64 closed form)."""
import numpy as np
import pytest
import torch

import oracle
from sparsetir_amd import datasets, ops
from helpers import random_csr, sddmm_f64

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _run(dev, indptr, indices, a, b, feat):
    m, n, nnz = len(indptr) - 1, b.shape[0], len(indices)
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    pre = ops.build_sddmm_preproc(m, n, feat, nnz)
    f = ops.build_sddmm(m, n, feat, nnz)
    mid = torch.full((nnz,), -7, dtype=torch.int32, device=dev)
    c = torch.full((nnz,), float("nan"), dtype=torch.float32, device=dev)
    args = [t(a.ravel()), t(b.ravel()), c, t(indptr), t(indices), mid]
    pre(*args)
    f(*args)
    torch.cuda.synchronize()
    return c.cpu().numpy(), mid.cpu().numpy()


@pytest.mark.parametrize("feat", [16, 32, 64, 128, 256, 512, 40, 3, 4, 96, 384, 260])
def test_sddmm_feature_widths(dev, feat):
    m, n = 901, 1203
    indptr, indices = random_csr(m, n, 25000, feat, skew=1.1)
    rng = np.random.default_rng(feat)
    a = rng.standard_normal((m, feat), dtype=np.float32)
    b = rng.standard_normal((n, feat), dtype=np.float32)
    got, mid = _run(dev, indptr, indices, a, b, feat)
    assert np.array_equal(mid, oracle.sddmm_mid(indptr, len(indices)))
    want = sddmm_f64(indptr, indices, a, b)
    rows = np.repeat(np.arange(m), np.diff(indptr))
    scale = np.einsum("ek,ek->e", np.abs(a).astype(np.float64)[rows], np.abs(b).astype(np.float64)[indices])
    assert np.all(np.abs(got - want) <= RTOL * scale + 1e-30)
    ref = oracle.sddmm(a, b, indices, mid, feat)
    assert np.all(np.abs(got - ref) <= 2 * RTOL * scale + 1e-30)


def test_sddmm_edge_shapes(dev):
    for m, n, nnz in [(1, 1, 1), (4, 4, 0), (70, 3, 150), (3, 500, 63), (3, 500, 65)]:
        indptr, indices = random_csr(m, n, nnz, 1)
        rng = np.random.default_rng(1)
        a = rng.standard_normal((m, 64), dtype=np.float32)
        b = rng.standard_normal((n, 64), dtype=np.float32)
        got, mid = _run(dev, indptr, indices, a, b, 64)
        assert np.array_equal(mid, oracle.sddmm_mid(indptr, len(indices)))
        if len(indices):
            assert np.allclose(got, sddmm_f64(indptr, indices, a, b), rtol=1e-4, atol=1e-4)


def test_sddmm_config3_shape_small_scale(dev):
    g = datasets.config3(scale=0.01)
    feat = 64
    a = datasets.features(g["m"], feat, 1)
    b = datasets.features(g["n"], feat, 2)
    got, mid = _run(dev, g["indptr"], g["indices"], a, b, feat)
    want = sddmm_f64(g["indptr"], g["indices"], a, b)
    rows = np.repeat(np.arange(g["m"]), np.diff(g["indptr"]))
    assert np.array_equal(mid, rows)
    scale = np.einsum("ek,ek->e", np.abs(a).astype(np.float64)[rows], np.abs(b).astype(np.float64)[g["indices"]])
    assert np.all(np.abs(got - want) <= RTOL * scale + 1e-30)


def test_sddmm_scaled_by_edge_values(dev):
    m, n, feat = 400, 300, 64
    indptr, indices = random_csr(m, n, 9000, 5, skew=1.0)
    rng = np.random.default_rng(5)
    a = rng.standard_normal((m, feat), dtype=np.float32)
    b = rng.standard_normal((n, feat), dtype=np.float32)
    e = rng.random(len(indices), dtype=np.float32)
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    nnz = len(indices)
    c = torch.empty(nnz, device=dev)
    mid = torch.empty(nnz, dtype=torch.int32, device=dev)
    args = [t(a.ravel()), t(b.ravel()), c, t(indptr), t(indices), mid]
    ops.build_sddmm_preproc(m, n, feat, nnz)(*args)
    ops.build_sddmm_scaled(m, n, feat, nnz)(*args, t(e))
    torch.cuda.synchronize()
    want = sddmm_f64(indptr, indices, a, b) * e
    rows = np.repeat(np.arange(m), np.diff(indptr))
    scale = np.einsum("ek,ek->e", np.abs(a).astype(np.float64)[rows], np.abs(b).astype(np.float64)[indices]) * e
    assert np.all(np.abs(c.cpu().numpy() - want) <= 2 * RTOL * scale + 1e-30)


def test_sddmm_preproc_empty_row_runs_and_hub_rows(dev):
    """Row lookup where 512 consecutive nonzeros span thousands of rows (long runs of empty rows:
    the per-nonzero fallback) and where one row holds thousands of nonzeros."""
    rng = np.random.default_rng(21)
    deg = np.zeros(40000, np.int64)
    deg[rng.choice(40000, 300, replace=False)] = rng.integers(1, 6, 300)   # sparse region
    deg[100] = 5000                                                         # hub
    deg[20000:20400] = rng.integers(0, 40, 400)                             # dense region
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    nnz = int(indptr[-1])
    pre = ops.build_sddmm_preproc(40000, 10, 16, nnz)
    mid = torch.full((nnz,), -7, dtype=torch.int32, device=dev)
    z = lambda k, dt=torch.float32: torch.zeros(k, dtype=dt, device=dev)
    pre(z(40000 * 16), z(10 * 16), z(nnz), torch.from_numpy(indptr).to(dev), z(nnz, torch.int32), mid)
    torch.cuda.synchronize()
    assert np.array_equal(mid.cpu().numpy(), np.repeat(np.arange(40000), deg))
    assert np.array_equal(mid.cpu().numpy(), oracle.sddmm_mid(indptr, nnz))
