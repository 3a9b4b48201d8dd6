"""The fp32 kernels against the float64 closed form with a literal rtol of 1e-5 on the result.

The other GPU tests bound the error by 1e-5 of the summed magnitudes, sum |a||x|, because an rtol
against the result says nothing where terms cancel.  With inputs that cannot cancel (edge values,
features and weights all non-negative) the summed magnitude *is* the result, and the bound turns
into the plain statement |got - want| <= 1e-5 * |want| for every output element: that is what is
asserted here, on the configurations' own graphs (hub rows of thousands of nonzeros included)."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import sparsetir_amd as st
from sparsetir_amd import datasets, ops
from helpers import rgms_f64, sddmm_f64, spmm_f64
from test_gpu_sddmm import _run as _run_sddmm
from test_gpu_spmm import _hyb_as_coo, _hyb_setup, _run_csr, _run_hyb

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _literal(got, want, what):
    got = got.astype(np.float64)
    assert np.all(want >= 0) and want.max() > 0
    err = np.abs(got - want)
    bad = err > RTOL * np.abs(want)
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} elements beyond rtol {RTOL}, worst relative error " \
                          f"{(err[bad] / np.abs(want[bad])).max():.3e}"


def test_csr_spmm_config1_literal_rtol(dev):
    g = datasets.config1()
    x = np.abs(g["x"])
    got = _run_csr(dev, g["indptr"], g["indices"], g["values"], x, g["feat"])
    _literal(got, spmm_f64(g["indptr"], g["indices"], g["values"], x), "csr config 1")


@pytest.mark.parametrize("feat", [32, 128])
def test_csr_and_hyb_spmm_config2_literal_rtol(dev, feat):
    g = datasets.config2()
    m, n, parts, buckets = g["m"], g["n"], g["num_col_parts"], g["buckets"]
    assert np.diff(g["indptr"]).max() > 5000  # hub rows: thousands of terms per output element
    x = np.abs(datasets.features(n, feat, seed=11))
    triples = _hyb_setup(dev, g["indptr"], g["indices"], m, n, parts, buckets, weighted=False, seed=0,
                         device_format=True)
    ones = np.ones(len(g["indices"]), np.float32)
    want = spmm_f64(g["indptr"], g["indices"], ones, x)
    got, _ = _run_hyb(dev, m, n, feat, parts, buckets, triples, x)
    _literal(got, want, f"hyb config 2, feat {feat}")
    _literal(_run_csr(dev, g["indptr"], g["indices"], ones, x, feat), want, f"csr config 2, feat {feat}")
    # one partition (what format.suggest_decomposition returns): every bucket but the last stores
    triples1 = _hyb_setup(dev, g["indptr"], g["indices"], m, n, 1, buckets, weighted=True, seed=3, device_format=True)
    r, c, v = _hyb_as_coo(triples1)
    a64 = sp.csr_matrix((v.astype(np.float64), (r, c)), shape=(m, n))
    got1, _ = _run_hyb(dev, m, n, feat, 1, buckets, triples1, x)
    _literal(got1, a64 @ x.astype(np.float64), f"hyb config 2, one partition, weighted, feat {feat}")


def test_sddmm_literal_rtol(dev):
    g = datasets.config3(scale=0.02)
    m, n, feat = g["m"], g["n"], 64
    rng = np.random.default_rng(5)
    a = np.abs(rng.standard_normal((m, feat), dtype=np.float32))
    b = np.abs(rng.standard_normal((n, feat), dtype=np.float32))
    got, _ = _run_sddmm(dev, g["indptr"], g["indices"], a, b, feat)
    _literal(got, sddmm_f64(g["indptr"], g["indices"], a, b), "sddmm")


@pytest.mark.parametrize("deterministic", [False, True])
def test_rgms_csf_f32_literal_rtol(dev, deterministic):
    cfg = datasets.config5(n=20000, num_rels=9, num_edges=200000, seed=7)
    R, n, fin, fout = 9, cfg["n"], 32, 32
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    rng = np.random.default_rng(2)
    x = np.abs(rng.standard_normal((n, fin), dtype=np.float32))
    w = np.abs(rng.standard_normal((R, fout, fin), dtype=np.float32)) * 0.1
    a = 0.5 + rng.random(len(csf[3]), dtype=np.float32)
    t = lambda z: torch.from_numpy(np.ascontiguousarray(z)).to(dev)
    f = ops.build_rgms_csf(n, n, R, fin, fout, len(csf[1]), len(csf[3]), deterministic=deterministic)
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(t(a), t(w.ravel()), t(x.ravel()), y, *[t(c) for c in csf])
    torch.cuda.synchronize()
    want = rgms_f64(*csf, a, x, np.ascontiguousarray(w.transpose(0, 2, 1)), n)
    got = y.cpu().numpy().reshape(n, fout)
    keep = want > 0  # rows without edges stay zero
    assert np.all(got[~keep] == 0)
    _literal(np.where(keep, got, 1.0), np.where(keep, want, 1.0), f"rgms csf fp32, deterministic={deterministic}")
