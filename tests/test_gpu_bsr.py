"""GPU parity of BSR SpMM (MFMA, fp16/bf16 in, fp32 accumulate) against the oracle.
Tolerance: rtol 2e-2 on the result plus 2e-2 of the summed term magnitudes per element."""
import numpy as np
import pytest
import torch

import oracle
from sparsetir_amd import datasets, ops
from sparsetir_amd._lib import SparseTIRError
from helpers import bsr_f64

pytestmark = pytest.mark.gpu
RTOL = 2e-2


def _run(dev, cfg, dtype, out_dtype=None):
    mb, nb, blk, feat = cfg["mb"], cfg["nb"], cfg["blk"], cfg["feat"]
    a = torch.from_numpy(cfg["data"]).to(dev).to(dtype)
    x = torch.from_numpy(cfg["x"]).to(dev).to(dtype)
    od = dtype if out_dtype is None else out_dtype
    y = torch.full((mb * blk * feat,), float("nan"), dtype=od, device=dev)
    f = ops.build_bsrmm(mb, nb, len(cfg["indices"]), blk, feat, dtype, od)
    f(a.reshape(-1), x.reshape(-1), y, torch.from_numpy(cfg["indptr"]).to(dev),
      torch.from_numpy(cfg["indices"]).to(dev))
    torch.cuda.synchronize()
    # the values the kernel actually saw (rounded to the storage type), as float32
    a32 = a.float().cpu().numpy()
    x32 = x.float().cpu().numpy()
    return y.float().cpu().numpy().reshape(mb * blk, feat), a32, x32


def _check(got, cfg, a32, x32, out_is_16bit, what):
    mb, nb, blk = cfg["mb"], cfg["nb"], cfg["blk"]
    want = bsr_f64(cfg["indptr"], cfg["indices"], a32, x32, mb, nb, blk)
    scale = bsr_f64(cfg["indptr"], cfg["indices"], np.abs(a32), np.abs(x32), mb, nb, blk)
    # fp32 accumulation of exactly representable products: error ~1e-6*scale; a 16-bit output
    # adds one rounding of the result (2^-8 relative for bf16)
    bound = 1e-5 * scale + (RTOL * np.abs(want) if out_is_16bit else 0) + 1e-30
    err = np.abs(got - want)
    assert np.all(err <= bound), f"{what}: worst {np.max(err - bound):.3e}"
    ref = oracle.bsrmm(a32, x32, cfg["indptr"], cfg["indices"], blk, cfg["feat"])
    assert np.all(np.abs(got - ref) <= RTOL * np.abs(ref) + RTOL * scale)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("out32", [False, True])
def test_bsr_small(dev, dtype, out32):
    cfg = datasets.config4(seed=11, mb=9, nb=7, blk=32, density=0.4, feat=160)
    got, a32, x32 = _run(dev, cfg, dtype, torch.float32 if out32 else None)
    _check(got, cfg, a32, x32, not out32, f"{dtype} out32={out32}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bsr_config4(dev, dtype):
    cfg = datasets.config4()
    got, a32, x32 = _run(dev, cfg, dtype)
    _check(got, cfg, a32, x32, True, f"config4 {dtype}")


def test_bsr_block64_and_empty_rows(dev):
    cfg = datasets.config4(seed=6, mb=6, nb=5, blk=64, density=0.3, feat=96)
    assert (np.diff(cfg["indptr"]) == 0).any()  # the fixture holds a block row without blocks
    got, a32, x32 = _run(dev, cfg, torch.float16, torch.float32)
    _check(got, cfg, a32, x32, False, "blk=64")
    empty = datasets.config4(seed=6, mb=4, nb=4, blk=32, density=0.0, feat=32)
    got, _, _ = _run(dev, empty, torch.float16)
    assert np.all(got == 0)


@pytest.mark.parametrize("blk,feat,dtype,out32", [
    (64, 1056, torch.bfloat16, False),   # two slices per workgroup, two accumulators per wavefront
    (128, 160, torch.float16, True),     # two slices per workgroup, four k steps per block
    (96, 64, torch.float16, False),      # 96 rows: one slice per workgroup
    (128, 1280, torch.float16, False),   # block rows dealt to XCDs, five feature tiles of 256
    (256, 384, torch.bfloat16, True),    # four slices per block row in that order, a partial second feature tile
])
def test_bsr_tall_blocks(dev, blk, feat, dtype, out32):
    """Blocks of 64 rows and more: a workgroup takes two 32-row slices when blk is a multiple of 64;
    from 128 rows on (and more than one feature tile) the block rows are dealt to XCDs, 13 block
    rows here: neither a multiple of 8 nor below it."""
    cfg = datasets.config4(seed=blk, mb=13 if blk >= 128 else 5, nb=6, blk=blk, density=0.35, feat=feat)
    got, a32, x32 = _run(dev, cfg, dtype, torch.float32 if out32 else None)
    _check(got, cfg, a32, x32, not out32, f"blk={blk} feat={feat} {dtype}")


@pytest.mark.parametrize("mb,nb,blk,feat,dtype", [
    (160, 12, 32, 512, torch.float16),    # one accumulator per wavefront
    (48, 20, 32, 1536, torch.bfloat16),   # two accumulators per wavefront
    (24, 10, 64, 1536, torch.float16),    # two slices per workgroup as well
    (9, 6, 128, 2080, torch.float16),     # 128-row blocks, last feature tile partial
    (10, 4, 256, 1024, torch.bfloat16),   # 256-row blocks
])
def test_bsr_many_workgroups(dev, mb, nb, blk, feat, dtype):
    """More than two workgroups per CU: the kernel whose wavefronts split the feature axis (small
    launches take the one whose wavefronts split the steps of a block row)."""
    cfg = datasets.config4(seed=mb, mb=mb, nb=nb, blk=blk, density=0.3, feat=feat)
    assert mb * (blk // 32) * ((feat + 127) // 128) > 512
    got, a32, x32 = _run(dev, cfg, dtype)
    _check(got, cfg, a32, x32, True, f"mb={mb} blk={blk} feat={feat} {dtype}")


@pytest.mark.parametrize("dtype,out32,varied", [(torch.float16, False, False), (torch.bfloat16, True, True)])
def test_bsr_launch_swept_in_step(dev, dtype, out32, varied):
    """A launch large enough for the kernel in which as many workgroups as are resident loop over
    tiles, every workgroup ranking the block rows by length on its own (X rows of one feature tile
    beyond 3 MB, at least 8 feature tiles, several tiles per resident workgroup).  Every block row
    must be computed exactly once: compared on the GPU against the same sum formed block by block in
    fp32 by torch, for all rows.  `varied`: block rows of very different lengths, empty ones and
    one beyond the 1024 length classes of the ranking."""
    mb, nb, blk, feat = 1100, 208, 32, 2048
    rng = np.random.default_rng(17)
    if varied:
        nb = 1300
        dens = rng.choice([0.0, 0.002, 0.01, 0.03], size=mb)
        present = rng.random((mb, nb)) < dens[:, None]
        present[7, :] = True         # 1300 blocks: the last length class
        present[8, :1023] = True
        present[9, :1024] = True
    else:
        present = rng.random((mb, nb)) < 0.05
    indptr = np.zeros(mb + 1, np.int32)
    np.cumsum(present.sum(axis=1), out=indptr[1:])
    indices = np.nonzero(present)[1].astype(np.int32)
    nnzb = len(indices)
    assert nb * blk * 256 * 2 > 3 << 20 and feat // 256 >= 8
    gen = torch.Generator(device=dev).manual_seed(3)
    a = (torch.randn(nnzb * blk * blk, device=dev, generator=gen) * 0.02).to(dtype)
    x = torch.randn(nb * blk * feat, device=dev, generator=gen).to(dtype)
    od = torch.float32 if out32 else dtype
    y = torch.full((mb * blk * feat,), float("nan"), dtype=od, device=dev)
    d_ptr, d_idx = torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev)
    ops.build_bsrmm(mb, nb, nnzb, blk, feat, dtype, od)(a, x, y, d_ptr, d_idx)
    torch.cuda.synchronize()
    # reference: per stored block one fp32 product, summed per block row (index_add), in chunks
    rows_of = torch.repeat_interleave(torch.arange(mb, device=dev), torch.from_numpy(np.diff(indptr)).to(dev))
    want = torch.zeros(mb, blk, feat, device=dev)
    scale = torch.zeros(mb, blk, feat, device=dev)
    a3, x3 = a.view(nnzb, blk, blk).float(), x.view(nb, blk, feat).float()
    for lo in range(0, nnzb, 2048):
        hi = min(nnzb, lo + 2048)
        xb = x3[d_idx[lo:hi].long()]
        want.index_add_(0, rows_of[lo:hi], torch.bmm(a3[lo:hi], xb))
        scale.index_add_(0, rows_of[lo:hi], torch.bmm(a3[lo:hi].abs(), xb.abs()))
    got = y.view(mb, blk, feat).float()
    bound = 2e-5 * scale + (0.0 if out32 else RTOL * want.abs()) + 1e-30
    bad = (got - want).abs() > bound
    assert not bool(bad.any()), f"{int(bad.sum())} elements off, rows {torch.nonzero(bad.any(2).any(1))[:8].ravel().tolist()}"
    # a block row without blocks is written as zeros
    empty = torch.from_numpy(np.diff(indptr) == 0).to(dev)
    assert bool((got[empty] == 0).all())


@pytest.mark.parametrize("blk,feat,dtype,out32", [
    (16, 512, torch.float16, False),    # the reference's schedule splits both block axes by 16
    (16, 160, torch.bfloat16, True),    # an odd number of 16-column chunks in most block rows, a partial feature tile
    (48, 96, torch.float16, True),      # a multiple of 16 that is not one of 32: three slices, three chunks per block
    (80, 256, torch.bfloat16, False),
])
def test_bsr_blocks_of_16_rows(dev, blk, feat, dtype, out32):
    """Block sides that are multiples of 16 (examples/blocksparse/bsr_spmm.py:379-380 splits the
    block axes by 16): the 16-row slices run on the 16x16x32 matrix-core instruction, two
    16-column chunks per step."""
    cfg = datasets.config4(seed=blk + feat, mb=11, nb=13, blk=blk, density=0.3, feat=feat)
    got, a32, x32 = _run(dev, cfg, dtype, torch.float32 if out32 else None)
    _check(got, cfg, a32, x32, not out32, f"blk={blk} feat={feat} {dtype}")


def test_bsr_rejects_unsupported(dev):
    z = lambda k, dt: torch.zeros(k, dtype=dt, device=dev)
    f = ops.build_bsrmm(1, 1, 1, 8, 32)
    with pytest.raises(SparseTIRError, match="blk"):
        f(z(64, torch.float16), z(256, torch.float16), z(256, torch.float16), z(2, torch.int32), z(1, torch.int32))


def test_dbsr_doubly_compressed(dev):
    """Only the non-empty block rows are stored; block rows without blocks keep their content."""
    cfg = datasets.config4(seed=8, mb=12, nb=9, blk=32, density=0.15, feat=96)
    counts = np.diff(cfg["indptr"])
    keep = np.nonzero(counts > 0)[0].astype(np.int32)
    assert len(keep) < cfg["mb"]  # some block rows are empty and are not stored
    ptr1 = np.concatenate([[0], np.cumsum(counts[keep])]).astype(np.int32)
    a = torch.from_numpy(cfg["data"]).to(dev).half()
    x = torch.from_numpy(cfg["x"]).to(dev).half()
    y = torch.full((cfg["mb"] * 32 * 96,), 7.0, dtype=torch.float32, device=dev)
    f = ops.build_dbsrmm(cfg["mb"], cfg["nb"], len(keep), len(cfg["indices"]), 32, 96, torch.float16, torch.float32)
    t = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)
    f(a.reshape(-1), x.reshape(-1), y, t(np.asarray([0, len(keep)], np.int32)), t(keep), t(ptr1), t(cfg["indices"]))
    torch.cuda.synchronize()
    got = y.cpu().numpy().reshape(cfg["mb"], 32, 96)
    want = bsr_f64(cfg["indptr"], cfg["indices"], a.float().cpu().numpy(), x.float().cpu().numpy(),
                   cfg["mb"], cfg["nb"], 32).reshape(cfg["mb"], 32, 96)
    empty = np.setdiff1d(np.arange(cfg["mb"]), keep)
    assert np.all(got[empty] == 7.0)
    assert np.allclose(got[keep], want[keep], rtol=1e-4, atol=1e-4)
