"""GPU parity of RGMS with an fp16 Y (the reference's tensor-core operator built with dtype
"float16", examples/rgms/rgcn/bench_rgcn_tensorcore.py:564-607) against the float64 closed form.

Tolerance: fp16 inputs and one rounding of the result to fp16 per store (rtol 2e-2 on the result);
elements that are summed with fp16 atomics are rounded once per addition, which is bounded by
2^-11 of the summed magnitudes per addition: atol 4e-3 of the summed magnitudes."""
import numpy as np
import pytest
import torch

import sparsetir_amd as st
from sparsetir_amd import datasets, ops, packed
from sparsetir_amd._lib import SparseTIRError
from helpers import random_csf, rgms_f64
from test_gpu_rgms import _csf_from_pairs, slots_of

pytestmark = pytest.mark.gpu


def _ell3d(dev, csf, R, group, buckets, weighted, seed):
    rows_bkt = [max(1, group // b) for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    rng = np.random.default_rng(seed)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    triples, mids, wts = [], [], []
    for b in range(len(buckets)):
        a = mask[b].astype(np.float32)
        if weighted:
            a = a * (0.5 + rng.random(a.shape, dtype=np.float32))
        a16 = a.astype(np.float16)
        wts.append(a16.astype(np.float64))
        triples += [t(a16.ravel()), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    return rows_bkt, ptr, rows, cols, mask, wts, triples, mids


def _closed_form(R, m, fout, ptr, rows, cols, wts, x64, w64):
    """Y[row] += a * X[col] @ W[rel] in float64 straight from the ELL3D arrays, and the same with
    absolute values (the magnitude of the summed terms)."""
    want, scale = np.zeros((m, fout)), np.zeros((m, fout))
    for b in range(len(cols)):
        G, rb, cb = cols[b].shape
        rel = np.repeat(np.arange(R), np.diff(ptr[b]))
        for r in range(R):
            g = np.nonzero(rel == r)[0]
            if len(g) == 0:
                continue
            a = wts[b][g].reshape(-1, cb)
            c = cols[b][g].reshape(-1, cb)
            agg = np.einsum("es,esk->ek", a, x64[c])
            agg_abs = np.einsum("es,esk->ek", a, np.abs(x64[c]))
            dest = rows[b][g].reshape(-1)
            np.add.at(want, dest, agg @ w64[r])
            np.add.at(scale, dest, agg_abs @ np.abs(w64[r]))
    return want, scale


def _case(dev, csf, m, n, R, fin, fout, group, buckets, weighted, seed, static=False, y0=None, calls=1):
    rows_bkt, ptr, rows, cols, mask, wts, triples, mids = _ell3d(dev, csf, R, group, buckets, weighted, seed)
    rng = np.random.default_rng(seed + 1)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = t(rng.standard_normal((n, fin), dtype=np.float32)).half()
    w = t(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).half()
    f = ops.build_rgms(m, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols], static_weights=static,
                       out_dtype=torch.float16)
    y = torch.zeros(m * fout, dtype=torch.float16, device=dev) if y0 is None else y0.clone()
    for _ in range(calls):
        f(w.reshape(-1), x.reshape(-1), y, *triples, *mids)
    torch.cuda.synchronize()
    want, scale = _closed_form(R, m, fout, ptr, rows, cols, wts, x.double().cpu().numpy(), w.double().cpu().numpy())
    base = np.zeros((m, fout)) if y0 is None else y0.double().cpu().numpy().reshape(m, fout)
    want, scale = base + calls * want, np.abs(base) + calls * scale
    got = y.double().cpu().numpy().reshape(m, fout)
    err = np.abs(got - want)
    assert np.all(err <= 2e-2 * np.abs(want) + 4e-3 * scale + 1e-30), f"worst {err.max():.3e}"
    return got, want, slots_of(mask)


@pytest.mark.parametrize("group,buckets,fin,fout,weighted", [
    (256, [1, 2, 4, 8, 16], 32, 32, False),
    (32, [1, 2, 4, 8, 16, 32], 32, 64, True),
    (16, [1, 2, 4], 16, 32, True),
    (12, [1, 3, 6], 48, 32, True),
    (64, [2, 64], 64, 96, False),
])
def test_rgms_f16_out_small(dev, group, buckets, fin, fout, weighted):
    """Below 8192 slots: one packed fp16 atomic per ELL row and pair of output features, every
    bucket width's way of summing an ELL row."""
    R, n = 5, 300
    csf = random_csf(R, n, 900, seed=group)
    _, want, slots = _case(dev, csf, n, n, R, fin, fout, group, buckets, weighted, seed=group)
    assert slots < 8192 and np.abs(want).max() > 0


@pytest.mark.parametrize("static", [False, True])
def test_rgms_f16_out_config5_reduced(dev, static):
    """The resident destination-tile kernel (W in LDS): tiles written once, rounded once."""
    cfg = datasets.config5(n=20000, num_rels=9, num_edges=200000, seed=7)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    _, _, slots = _case(dev, csf, cfg["m"], cfg["n"], 9, 32, 32, 256, [1, 2, 4, 8, 16], True, seed=3, static=static)
    assert slots >= 8192


def test_rgms_f16_out_adds_to_y(dev):
    """The operator adds to what Y holds, over two calls."""
    cfg = datasets.config5(n=6000, num_rels=5, num_edges=60000, seed=9)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    y0 = (torch.randn(cfg["m"] * 64, device=dev) * 0.5).half()
    _case(dev, csf, cfg["m"], cfg["n"], 5, 32, 64, 64, [1, 4, 16], True, seed=5, y0=y0, calls=2)


@pytest.mark.parametrize("fin,fout,group,buckets", [
    (32, 32, 256, [1, 2, 4, 8, 16]),   # W in LDS
    (16, 64, 64, [1, 2, 4, 64]),
    (128, 32, 32, [2, 8, 32]),         # feat_in above 64: W read from memory, four wavefronts per unit
])
def test_rgms_f16_out_hub_rows(dev, fin, fout, group, buckets):
    """Output rows not a multiple of 32 and one row that receives thousands of edges in three
    relations: its tile is cut into pieces that meet in packed fp16 atomics."""
    n, R = 5001, 7
    rng = np.random.default_rng(fin + fout)
    pairs = []
    for r in range(R):
        e = 0 if r == 3 else 20000
        dst, src = rng.integers(0, n, e), rng.integers(0, n, e)
        if r in (0, 1, 5):
            dst = np.concatenate([dst, np.full(3000, 77)])
            src = np.concatenate([src, rng.choice(n, 3000, replace=False)])
        pairs.append((dst, src))
    csf = _csf_from_pairs(pairs, n)
    got, want, slots = _case(dev, csf, n, n, R, fin, fout, group, buckets, True, seed=fin)
    assert slots >= 8192 and np.abs(want[77]).max() > 0


def test_rgms_f16_out_rejects(dev):
    with pytest.raises(SparseTIRError):
        ops.build_rgms(64, 64, 2, 32, 32, [4], [4], [1], dtype=torch.bfloat16, out_dtype=torch.float16)
    f = ops.build_rgms(64, 64, 2, 32, 32, [4], [4], [1], out_dtype=torch.float16)
    z16 = lambda k: torch.zeros(k, dtype=torch.float16, device=dev)
    zi = lambda k: torch.zeros(k, dtype=torch.int32, device=dev)
    with pytest.raises(SparseTIRError):  # an fp32 Y where the operator was built for fp16
        f(z16(2 * 32 * 32), z16(64 * 32), torch.zeros(64 * 32, device=dev), z16(16), zi(4), zi(16), zi(1))


def test_packed_rgms_f16_out(dev):
    """sparsetir.rgms picks the output type from Y's dtype; same values as the operator class."""
    cfg = datasets.config5(n=3000, num_rels=4, num_edges=30000, seed=2)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    R, fin, fout, buckets = 4, 32, 32, [1, 2, 4, 8]
    rows_bkt, ptr, rows, cols, mask, wts, triples, mids = _ell3d(dev, csf, R, 64, buckets, True, seed=1)
    rng = np.random.default_rng(8)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = t(rng.standard_normal((cfg["n"], fin), dtype=np.float32)).half().reshape(-1)
    w = t(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).half().reshape(-1)
    y = torch.zeros(cfg["m"] * fout, dtype=torch.float16, device=dev)
    packed.get_global_func("sparsetir.rgms")(w, x, y, *triples, *mids, fin, fout)
    torch.cuda.synchronize()
    want, scale = _closed_form(R, cfg["m"], fout, ptr, rows, cols, wts, x.double().cpu().numpy().reshape(-1, fin),
                               w.double().cpu().numpy().reshape(R, fin, fout))
    err = np.abs(y.double().cpu().numpy().reshape(cfg["m"], fout) - want)
    assert np.all(err <= 2e-2 * np.abs(want) + 4e-3 * scale + 1e-30), f"worst {err.max():.3e}"
