"""Plan reuse of the plan-based operators.  The reference's built operators hold no state and read
their index arrays at every call (examples/spmm/bench_spmm.py:225-229,
examples/rgms/rgcn/bench_rgcn_tensorcore.py:852); here plans are kept per set of arrays, so these
tests pin what a caller of the reference may do without knowing of plans: alternate between graphs,
rewrite index arrays in place, free arrays and get the addresses back."""
import ctypes
import gc

import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import _lib, ops, packed
from sparsetir_amd._lib import SparseTIRError
from helpers import random_csf, random_csr, rgms_f64, spmm_f64

pytestmark = pytest.mark.gpu


def _td(dev):
    return lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)


def _hyb_case(dev, seed, parts, m=1500, n=1500, nnz=30000, buckets=(1, 2, 4, 8)):
    """Device triples of a decomposed random graph and the float64 result for weights 1."""
    td = _td(dev)
    indptr, indices = random_csr(m, n, nnz, seed, skew=1.0)
    rows, cols, mask = st.column_part_hyb(m, n, indptr, indices, parts, list(buckets))
    triples, nrows = [], []
    for p in range(parts):
        for b in range(len(buckets)):
            triples += [td(mask[p][b].astype(np.float32).ravel()), td(rows[p][b]), td(cols[p][b].ravel())]
            nrows.append(int(rows[p][b].shape[0]))
    return dict(m=m, n=n, indptr=indptr, indices=indices, parts=parts, buckets=list(buckets), triples=triples,
                nrows=nrows)


def _hyb_want(case, x, triples=None):
    """float64 closed form of what the (possibly rewritten) triples describe: every slot adds
    A * X[col] to its row."""
    trip = case["triples"] if triples is None else triples
    m, feat = case["m"], x.shape[1]
    want, scale = np.zeros((m, feat)), np.zeros((m, feat))
    nb = len(case["buckets"])
    for k in range(len(trip) // 3):
        a, r, c = (t.cpu().numpy() for t in trip[3 * k:3 * k + 3])
        w = case["buckets"][k % nb]
        if r.size == 0:
            continue
        contrib = (a.reshape(-1, w, 1).astype(np.float64) * x[c.reshape(-1, w)].astype(np.float64))
        np.add.at(want, r, contrib.sum(1))
        np.add.at(scale, r, np.abs(contrib).sum(1))
    return want, scale


def _rgms_case(dev, seed, R=6, n=3000, edges=30000, fin=32, fout=32, group=32, buckets=(1, 2, 4, 8)):
    td = _td(dev)
    csf = random_csf(R, n, edges, seed=seed)
    rb = [group // b for b in buckets]
    iptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, list(buckets))
    assert sum(c.size for c in cols) >= 8192  # large enough for the indexed kernel
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((R, fin, fout)) * 0.1).astype(np.float16)
    x = rng.standard_normal((n, fin)).astype(np.float16)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [td(mask[k].astype(np.float16).ravel()), td(rows[k].ravel()), td(cols[k].ravel())]
        mids.append(td(np.repeat(np.arange(R, dtype=np.int32), np.diff(iptr[k]))))
    want = rgms_f64(*csf, np.ones(len(csf[3]), np.float32), x.astype(np.float32), w.astype(np.float32), n)
    scale = rgms_f64(*csf, np.ones(len(csf[3]), np.float32), np.abs(x.astype(np.float32)),
                     np.abs(w.astype(np.float32)), n)
    return dict(R=R, n=n, fin=fin, fout=fout, rb=rb, buckets=list(buckets), groups=[c.shape[0] for c in cols],
                triples=triples, mids=mids, w=td(w.ravel()), x=td(x.ravel()), want=want, scale=scale)


def _rgms_ok(case, y):
    got = y.cpu().numpy().reshape(case["n"], case["fout"])
    return np.all(np.abs(got - case["want"]) <= 2e-2 * np.abs(case["want"]) + 1e-3 * case["scale"] + 1e-30)


@pytest.mark.parametrize("static", [0, 1])
def test_packed_operators_alternating_two_graphs_build_two_plans(dev, static):
    """Two graphs in turn, ten rounds, through "sparsetir.rgms" and "sparsetir.hyb_csrmm": each
    operator makes exactly two plans (one per graph), with and without the static-structure
    promise, and every result is right.  Tolerances: hyb fp32 1e-5 of the summed magnitudes; RGMS
    fp16 rtol 2e-2 plus 1e-3 of the summed magnitudes."""
    promise = packed.get_global_func("sparsetir.static_structure")
    packed.get_global_func("sparsetir.invalidate_plans")()
    promise(static)
    try:
        rg = [_rgms_case(dev, 31), _rgms_case(dev, 32, R=4, n=2500)]
        hy = [_hyb_case(dev, 41, parts=2), _hyb_case(dev, 42, parts=8, m=1200, n=1300)]
        feat = 64
        xs = [torch.randn(c["n"] * feat, device=dev) for c in hy]
        wants = [_hyb_want(c, x.cpu().numpy().reshape(-1, feat)) for c, x in zip(hy, xs)]
        f_rgms = packed.get_global_func("sparsetir.rgms")
        f_hyb = packed.get_global_func("sparsetir.hyb_csrmm")
        before = packed.plan_builds()
        for rnd in range(10):
            for c in rg:
                y = torch.zeros(c["n"] * c["fout"], device=dev)
                f_rgms(c["w"], c["x"], y, *c["triples"], *c["mids"], c["fin"], c["fout"])
                torch.cuda.synchronize()
                assert _rgms_ok(c, y), (rnd, "rgms")
            for c, x, (want, scale) in zip(hy, xs, wants):
                out = torch.zeros(c["m"] * feat, device=dev)
                f_hyb(x, out, *c["triples"], feat, c["parts"])
                torch.cuda.synchronize()
                got = out.cpu().numpy().reshape(c["m"], feat)
                assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30), (rnd, "hyb", c["parts"])
        assert packed.plan_builds() - before == 4
    finally:
        promise(0)
        packed.get_global_func("sparsetir.invalidate_plans")()


def test_packed_plan_cache_evicts_the_plan_used_longest_ago(dev):
    """Nine array sets through one operator: the ninth plan replaces the first one's, which is
    rebuilt when its arrays come again; the eight used last are all found."""
    packed.get_global_func("sparsetir.invalidate_plans")()
    f_hyb = packed.get_global_func("sparsetir.hyb_csrmm")
    cases = [_hyb_case(dev, 60 + i, parts=1, m=300, n=300, nnz=3000) for i in range(9)]
    feat = 32
    x = torch.randn(300 * feat, device=dev)

    def call(c):
        out = torch.zeros(c["m"] * feat, device=dev)
        f_hyb(x, out, *c["triples"], feat, c["parts"])

    before = packed.plan_builds()
    for c in cases:
        call(c)
    assert packed.plan_builds() - before == 9
    for c in cases[1:]:
        call(c)  # all cached
    assert packed.plan_builds() - before == 9
    call(cases[0])  # evicted by the ninth
    assert packed.plan_builds() - before == 10
    torch.cuda.synchronize()
    packed.get_global_func("sparsetir.invalidate_plans")()


@pytest.mark.parametrize("parts", [2, 8])
def test_packed_hyb_columns_rewritten_in_place(dev, parts):
    """Without the static-structure promise the packed hyb operator reads its arrays at every call,
    as the reference's does: column ids rewritten in place between two calls (same addresses, same
    sizes) give the sums for the new columns.  2 partitions would run as phases without atomics and
    8 as merged rows with copied column ids if plans kept what they derive from the contents."""
    packed.get_global_func("sparsetir.invalidate_plans")()
    c = _hyb_case(dev, 71, parts=parts)
    feat = 64
    x = torch.randn(c["n"] * feat, device=dev)
    xh = x.cpu().numpy().reshape(-1, feat)
    f_hyb = packed.get_global_func("sparsetir.hyb_csrmm")

    def agrees():
        out = torch.zeros(c["m"] * feat, device=dev)
        f_hyb(x, out, *c["triples"], feat, parts)
        torch.cuda.synchronize()
        want, scale = _hyb_want(c, xh)
        return np.all(np.abs(out.cpu().numpy().reshape(c["m"], feat) - want) <= 1e-5 * scale + 1e-30)

    assert agrees()
    before = packed.plan_builds()
    # every column id mirrored inside its partition's range, and rows of two buckets made to
    # collide (an output row fed by two ELL rows of one bucket: the phases' single-writer rule
    # would no longer hold)
    width = (c["n"] + parts - 1) // parts
    for k in range(len(c["triples"]) // 3):
        cols, rows = c["triples"][3 * k + 2], c["triples"][3 * k + 1]
        p = k // len(c["buckets"])
        lo, hi = p * width, min(c["n"], (p + 1) * width)
        cols.copy_(lo + (hi - 1 - cols).clamp(min=0) % (hi - lo))
        if rows.numel() > 1:
            rows[1:2] = rows[0:1]
    assert agrees()
    assert packed.plan_builds() == before  # the same plan: addresses and sizes only
    packed.get_global_func("sparsetir.invalidate_plans")()


def test_packed_static_structure_keeps_the_index_until_invalidated(dev):
    """With "sparsetir.static_structure"(1) the RGMS plan keeps its edge index: source nodes
    rewritten in place go unnoticed until "sparsetir.invalidate_plans"; without the promise (the
    default) the next call already sees them."""
    promise = packed.get_global_func("sparsetir.static_structure")
    inval = packed.get_global_func("sparsetir.invalidate_plans")
    g = packed.get_global_func("sparsetir.rgms")
    c = _rgms_case(dev, 81)
    n, fout = c["n"], c["fout"]

    def run():
        y = torch.zeros(n * fout, device=dev)
        g(c["w"], c["x"], y, *c["triples"], *c["mids"], c["fin"], fout)
        torch.cuda.synchronize()
        return y

    def shift_sources():
        for k in range(len(c["buckets"])):
            c["triples"][3 * k + 2].copy_((c["triples"][3 * k + 2] + 1) % n)

    inval()
    try:
        y0 = run()
        assert _rgms_ok(c, y0)
        shift_sources()
        y1 = run()  # default: arrays read afresh
        assert not torch.allclose(y1, y0, rtol=1e-3, atol=1e-3)
        fresh = torch.zeros(n * fout, device=dev)
        ops.build_rgms(n, n, c["R"], c["fin"], fout, c["rb"], c["buckets"], c["groups"])(
            c["w"], c["x"], fresh, *c["triples"], *c["mids"])
        torch.cuda.synchronize()
        assert torch.allclose(y1, fresh, rtol=1e-4, atol=1e-4)
        promise(1)
        y2 = run()
        assert torch.allclose(y2, fresh, rtol=1e-4, atol=1e-4)
        shift_sources()
        y3 = run()  # promised static: the old index is still used
        assert torch.allclose(y3, y2, rtol=1e-6, atol=1e-6)
        inval()
        y4 = run()
        assert not torch.allclose(y4, y2, rtol=1e-3, atol=1e-3)
    finally:
        promise(0)
        inval()


def test_operator_objects_notice_in_place_changes_and_keep_their_arrays(dev):
    """ops.HybCsrMM / ops.Rgms / ops.TcSpMM key their plans by address and by the version counter
    torch keeps per tensor, and a plan keeps its arrays alive.  So: index arrays rewritten through
    torch give the new result without invalidate(); alternating two graphs builds two plans; and a
    TcSpMM called with a second indptr of the same size after the first was dropped cannot mistake
    it for the first (the allocator cannot hand out the address of an array that is still held)."""
    # hyb, 2 partitions (phases without atomics while the row arrays allow it)
    c = _hyb_case(dev, 91, parts=2)
    feat = 32
    x = torch.randn(c["n"] * feat, device=dev)
    xh = x.cpu().numpy().reshape(-1, feat)
    f = ops.build_hyb_csrmm(c["m"], c["n"], feat, 2, c["buckets"], c["nrows"])

    def hyb_agrees():
        out = torch.zeros(c["m"] * feat, device=dev)
        f(x, out, *c["triples"])
        torch.cuda.synchronize()
        want, scale = _hyb_want(c, xh)
        return np.all(np.abs(out.cpu().numpy().reshape(c["m"], feat) - want) <= 1e-5 * scale + 1e-30)

    assert hyb_agrees() and hyb_agrees() and f.plan_builds == 1
    for k in range(len(c["triples"]) // 3):  # two ELL rows of one bucket now feed the same output row
        rows = c["triples"][3 * k + 1]
        if rows.numel() > 1:
            rows[1:2] = rows[0:1]
    assert hyb_agrees() and f.plan_builds == 2

    # RGMS: two graphs in turn
    rg = [_rgms_case(dev, 92), _rgms_case(dev, 93)]
    g = ops.build_rgms(rg[0]["n"], rg[0]["n"], rg[0]["R"], 32, 32, rg[0]["rb"], rg[0]["buckets"], rg[0]["groups"])
    g2 = ops.build_rgms(rg[1]["n"], rg[1]["n"], rg[1]["R"], 32, 32, rg[1]["rb"], rg[1]["buckets"], rg[1]["groups"])
    same_shape = rg[0]["groups"] == rg[1]["groups"]
    for rnd in range(10):
        for case, op in zip(rg, (g, g if same_shape else g2)):
            y = torch.zeros(case["n"] * 32, device=dev)
            op(case["w"], case["x"], y, *case["triples"], *case["mids"])
            torch.cuda.synchronize()
            assert _rgms_ok(case, y), rnd
    assert g.plan_builds + (0 if same_shape else g2.plan_builds) == 2
    # ... and source nodes rewritten through torch are noticed
    case = rg[0]
    for k in range(len(case["buckets"])):
        case["triples"][3 * k + 2].add_(1).remainder_(case["n"])
    y = torch.zeros(case["n"] * 32, device=dev)
    g(case["w"], case["x"], y, *case["triples"], *case["mids"])
    torch.cuda.synchronize()
    assert not _rgms_ok(case, y)  # the old closed form no longer describes the arrays
    fresh = torch.zeros_like(y)
    ops.build_rgms(case["n"], case["n"], case["R"], 32, 32, case["rb"], case["buckets"], case["groups"])(
        case["w"], case["x"], fresh, *case["triples"], *case["mids"])
    torch.cuda.synchronize()
    assert torch.allclose(y, fresh, rtol=1e-4, atol=1e-4)

    # TcSpMM: two indptr arrays of equal size, the first one dropped between the calls
    t, grp, featc = 32, 16, 64
    m, n = 320, 9000
    rng = np.random.default_rng(94)
    td = _td(dev)
    L = _lib.lib()
    results = []
    mats = []
    for hub in (3, 200):  # a hub row in another tile: other tiles are long
        deg = rng.integers(0, 8, m)
        deg[hub] = 6000
        indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
        indices = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]).astype(np.int32)
        mats.append((indptr, indices))
    xc = rng.standard_normal((n, featc)).astype(np.float16)
    d_x = td(xc.ravel())
    op = None
    for indptr, indices in mats:
        gptr, tiles, mask = st.condense(indptr, indices, t, grp)
        mb, nnzb = len(gptr) - 1, tiles.shape[0]
        if op is None or (op.mb, op.nnzb) != (mb, nnzb):
            op = ops.build_tcspmm(mb, nnzb, featc, t, grp, n, torch.float16)
        d_ptr, d_a, d_t = td(gptr), td(mask.astype(np.float16).ravel()), td(tiles.ravel())
        c1 = torch.full((mb * t * featc,), float("nan"), dtype=torch.float16, device=dev)
        op(d_a, d_x, c1, d_ptr, d_t)
        c2 = torch.full_like(c1, float("nan"))
        _lib.check(L.stir_tc_spmm_f16(0, mb, t, grp, featc, nnzb, ctypes.c_void_p(d_a.data_ptr()),
                                      ctypes.c_void_p(d_x.data_ptr()), ctypes.c_void_p(c2.data_ptr()),
                                      ctypes.c_void_p(d_ptr.data_ptr()), ctypes.c_void_p(d_t.data_ptr()),
                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        ones = np.ones(len(indices), np.float32)
        want = spmm_f64(indptr, indices, ones, xc.astype(np.float32))
        scale = spmm_f64(indptr, indices, ones, np.abs(xc.astype(np.float32)))
        for got in (c1, c2):
            gg = got.float().cpu().numpy().reshape(mb * t, featc)[:m]
            assert np.all(np.abs(gg - want) <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30)
        del d_ptr, d_a, d_t, c1, c2
        gc.collect()


def test_packed_format_fill_must_match_its_sizes_call(dev):
    """The device format passes keep the layout of their scratch between .sizes and .fill: a .fill
    with other arrays, sizes or bucket lists, or with outputs of other lengths than .sizes
    returned, is refused on the host before anything is launched."""
    td = _td(dev)
    # ColumnPartHyb
    m = n = 500
    indptr, indices = random_csr(m, n, 8000, 5, skew=1.0)
    d_ptr, d_idx = td(indptr), td(indices)
    buckets = np.asarray([1, 2, 4], np.int32)
    nrows = np.zeros(2 * 3, np.int64)
    sizes = packed.get_global_func("tir.sparse.ColumnPartHyb.sizes")
    fill = packed.get_global_func("tir.sparse.ColumnPartHyb.fill")
    sizes(m, n, d_ptr, d_idx, 2, buckets, nrows)

    def outs(counts, widths):
        o = []
        for k, r in enumerate(counts):
            w = int(widths[k % len(widths)])
            o += [torch.zeros(int(r), dtype=torch.int32, device=dev), torch.zeros(int(r) * w, dtype=torch.int32, device=dev),
                  torch.zeros(int(r) * w, dtype=torch.int32, device=dev)]
        return o

    other_b = np.asarray([1, 2, 8], np.int32)
    with pytest.raises(SparseTIRError, match="differ from those of the .sizes call"):
        fill(m, n, d_ptr, d_idx, 2, other_b, *outs(nrows, other_b))
    d_idx2 = d_idx.clone()
    with pytest.raises(SparseTIRError, match="differ from those of the .sizes call"):
        fill(m, n, d_ptr, d_idx2, 2, buckets, *outs(nrows, buckets))
    wrong = nrows.copy()
    wrong[0] += 1
    with pytest.raises(SparseTIRError, match="the .sizes call returned"):
        fill(m, n, d_ptr, d_idx, 2, buckets, *outs(wrong, buckets))
    good = outs(nrows, buckets)
    fill(m, n, d_ptr, d_idx, 2, buckets, *good)  # the matching call still works
    torch.cuda.synchronize()
    rows, cols, mask = oracle.column_part_hyb(m, n, indptr, indices, 2, [1, 2, 4])
    for p in range(2):
        for q in range(3):
            k = p * 3 + q
            assert np.array_equal(good[3 * k].cpu().numpy(), rows[p][q])
            assert np.array_equal(good[3 * k + 1].cpu().numpy(), cols[p][q].ravel())

    # CSFToELL3D
    csf = random_csf(5, 200, 3000, 6)
    d_csf = [td(a) for a in csf]
    rb, cb = np.asarray([4, 2, 1], np.int32), np.asarray([1, 2, 4], np.int32)
    groups = np.zeros(3, np.int64)
    packed.get_global_func("tir.sparse.CSFToELL3D.sizes")(*d_csf, rb, cb, groups)

    def csf_outs(gr, rbk, cbk):
        o = []
        for b in range(3):
            g = int(gr[b])
            o += [torch.zeros(6, dtype=torch.int32, device=dev), torch.zeros(g * int(rbk[b]), dtype=torch.int32, device=dev),
                  torch.zeros(g * int(rbk[b]) * int(cbk[b]), dtype=torch.int32, device=dev),
                  torch.zeros(g * int(rbk[b]) * int(cbk[b]), dtype=torch.int32, device=dev)]
        return o

    csf_fill = packed.get_global_func("tir.sparse.CSFToELL3D.fill")
    rb2 = np.asarray([8, 2, 1], np.int32)
    with pytest.raises(SparseTIRError, match="differ from those of the .sizes call"):
        csf_fill(*d_csf, rb2, cb, *csf_outs(groups, rb2, cb))
    g_wrong = groups.copy()
    g_wrong[1] += 2
    with pytest.raises(SparseTIRError, match="the .sizes call returned"):
        csf_fill(*d_csf, rb, cb, *csf_outs(g_wrong, rb, cb))
    csf_fill(*d_csf, rb, cb, *csf_outs(groups, rb, cb))

    # ConDense
    t, g = 16, 16
    gptr = torch.empty((m + t - 1) // t + 1, dtype=torch.int32, device=dev)
    ng = np.zeros(1, np.int64)
    packed.get_global_func("tir.sparse.ConDense.sizes")(d_ptr, d_idx, t, g, gptr, ng)
    cd_fill = packed.get_global_func("tir.sparse.ConDense.fill")
    k = int(ng[0])
    z = lambda cnt: torch.zeros(cnt, dtype=torch.int32, device=dev)
    with pytest.raises(SparseTIRError, match="differ from those of the .sizes call"):
        cd_fill(d_ptr, d_idx2, t, g, z(k * g), z(k * t * g), gptr)
    with pytest.raises(SparseTIRError, match="the .sizes call returned"):
        cd_fill(d_ptr, d_idx, t, g, z((k + 1) * g), z((k + 1) * t * g), gptr)
    tiles, mask = z(k * g), z(k * t * g)
    cd_fill(d_ptr, d_idx, t, g, tiles, mask, gptr)
    torch.cuda.synchronize()
    want = oracle.condense(indptr, indices, t, g)
    assert np.array_equal(tiles.cpu().numpy(), want[1].ravel()) and np.array_equal(mask.cpu().numpy(), want[2].ravel())
