"""The built operators: what ``tvm.build(mod, target=...)`` hands the reference's scripts.

Each ``build_*`` function returns a callable that takes the same flat device arrays, in the
same order, as the operator the reference builds for that kernel, and launches the
hand-written gfx950 kernel through the C ABI on torch's current stream:

  build_csrmm         f(A, B, C, indptr, indices)             examples/spmm/bench_spmm_naive.py:121-129
  build_hyb_csrmm     f(B, C, A_0, rows_0, cols_0, ...)       examples/spmm/bench_spmm.py:208-225
  build_sddmm_preproc f(A, B, C, indptr, indices, mid)        examples/sddmm/bench_sddmm.py:106-115
  build_sddmm         f(A, B, C, indptr, indices, mid)        examples/sddmm/bench_sddmm.py:170-171
  build_bsrmm         f(A, X, Y, indptr, indices)             examples/blocksparse/bsr_spmm.py:427-433
  build_dbsrmm        f(A, X, Y, indptr_0, indices_0, indptr_1, indices_1)
                                                               examples/blocksparse/bsr_spmm.py:66-102
  build_tcspmm        f(A, B, C, indptr, indices)             examples/spmm/bench_tc_spmm.py:650-656
  build_rgms          f(W, X, Y, (A_k, rows_k, cols_k)..., mids_k...)
                                                               examples/rgms/rgcn/bench_rgcn_tensorcore.py:840-852
  build_rgms_f32      same arguments in fp32, W [R, Fout, Fin]  examples/rgms/rgcn/bench_rgcn_composable.py:208-221
  build_rgms_csf      f(A, W, X, Y, indptr_i, indices_i, indptr_j, indices_j)
                                                               examples/rgms/rgcn/bench_rgcn_non_composable.py:109

Arrays are torch CUDA tensors (device memory and streams only).  Arguments are checked the
way the reference's generated host stub checks DLTensors (src/tir/transforms/arg_binder.cc:152+):
one dimension, exact dtype, exact length, contiguous, all on one device.  Operators also offer
``time_evaluator(number)``, the reference's protocol of one discarded call followed by the
mean of ``number`` back-to-back launches between device events
(src/runtime/profiling.cc:742-797).
"""
import collections
import ctypes
import operator

import torch

from . import _lib


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None and t.numel() > 0 else 0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class _PlanCache:
    """The plans an operator used last, found again by key (addresses and torch version counters
    of the arrays a plan was made from).  At most ``capacity`` are kept: one more destroys the plan
    whose last use lies furthest back, so a caller that alternates between a few graphs
    (mini-batches, training and validation sets) builds each plan once.  ``builds`` counts the
    plans made.  An entry keeps its arrays alive: their addresses cannot be handed to other arrays
    while a plan made from them exists."""
    capacity = 8

    def __init__(self, destroy):
        self._destroy = destroy
        self._plans = collections.OrderedDict()  # key -> (plan, arrays kept alive)
        self.builds = 0

    def get(self, key):
        hit = self._plans.get(key)
        if hit is None:
            return None
        self._plans.move_to_end(key)
        return hit[0]

    def put(self, key, plan, keep):
        while len(self._plans) >= self.capacity:
            _, (old, _) = self._plans.popitem(last=False)
            self._destroy(old)
        self._plans[key] = (plan, keep)
        self.builds += 1

    def clear(self):
        while self._plans:
            _, (old, _) = self._plans.popitem()
            self._destroy(old)

    def __len__(self):
        return len(self._plans)


def _addr(t):
    return t.data_ptr() if t.numel() else 0


# A plan key is made at every call, over dozens of arrays for a decomposed matrix: C-level maps
# (10 us for 60 arrays) rather than a Python loop (25 us, the run time of a small launch).
_data_ptrs = torch.Tensor.data_ptr
_version_of = operator.attrgetter("_version")


def _same_objects(a, b):
    return b is not None and len(a) == len(b) and all(map(operator.is_, a, b))


class _Operator:
    name = "main"
    entry_name = "main"

    def _check(self, args, spec):
        """spec: list of (label, dtype, length).  Returns the device all arrays live on."""
        if len(args) != len(spec):
            raise _lib.SparseTIRError(f"{self.name}: num_args should be {len(spec)}")
        first = args[0]
        if isinstance(first, torch.Tensor) and first.is_cuda:
            idx = first.get_device()
            for t, (_, dtype, length) in zip(args, spec):
                # one combined test per array; anything odd is diagnosed by the slow path below
                if not (isinstance(t, torch.Tensor) and t.dtype == dtype and t.ndim == 1
                        and t.shape[0] == length and t.is_contiguous() and t.get_device() == idx):
                    break
            else:
                return first.device
        return self._check_slow(args, spec)

    def _check_slow(self, args, spec):
        dev = None
        for i, (t, (label, dtype, length)) in enumerate(zip(args, spec)):
            if not isinstance(t, torch.Tensor):
                raise _lib.SparseTIRError(f"{self.name}: Expect arg[{i}] to be pointer")
            if not t.is_cuda:
                raise _lib.SparseTIRError(f"{self.name}: arg[{i}] ({label}) must be a device array")
            if t.dim() != 1:
                raise _lib.SparseTIRError(f"{self.name}: {label}.ndim is expected to equal 1")
            if t.dtype != dtype:
                raise _lib.SparseTIRError(
                    f"{self.name}: {label}.dtype is expected to be {dtype}, got {t.dtype}")
            if t.shape[0] != length:
                raise _lib.SparseTIRError(
                    f"{self.name}: {label}.shape[0] is expected to be {length}, got {t.shape[0]}")
            if not t.is_contiguous():
                raise _lib.SparseTIRError(f"{self.name}: {label} is expected to be compact")
            if dev is None:
                dev = t.device
            elif t.device != dev:
                raise _lib.SparseTIRError(f"{self.name}: all arrays must be on one device")
        return dev

    def time_evaluator(self, number=100):
        """Returns g(*args) -> mean seconds per call over ``number`` launches after one
        discarded call, timed with device events on the current stream."""
        def run(*args):
            self(*args)
            start = torch.cuda.Event(enable_timing=True)
            stop = torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(number):
                self(*args)
            stop.record()
            stop.synchronize()
            return start.elapsed_time(stop) / 1e3 / number
        return run


class CsrMM(_Operator):
    name = "csrmm"

    def __init__(self, m, n, feat, nnz):
        self.m, self.n, self.feat, self.nnz = int(m), int(n), int(feat), int(nnz)
        self.L = _lib.lib()

    def __call__(self, *args):
        f32, i32 = torch.float32, torch.int32
        dev = self._check(args, [("A", f32, self.nnz), ("B", f32, self.n * self.feat),
                                 ("C", f32, self.m * self.feat), ("indptr", i32, self.m + 1),
                                 ("indices", i32, self.nnz)])
        a, b, c, indptr, indices = args
        with torch.cuda.device(dev):
            _lib.check(self.L.stir_csr_spmm_f32(self.m, self.n, self.feat, self.nnz, _ptr(a),
                                                _ptr(b), _ptr(c), _ptr(indptr), _ptr(indices),
                                                _stream()))


class HybCsrMM(_Operator):
    """All ELL buckets of all column partitions in one launch.  ``nrows`` lists the ELL rows
    of every bucket, partition-major, the quantity the reference specialises the kernel with
    (examples/spmm/bench_spmm.py:146-152).

    The operator keeps the plans of the array sets it was called with last (see :class:`_PlanCache`),
    keyed by the addresses of the (A_k, rows_k, cols_k) arrays and the version counters torch keeps
    for rows_k and cols_k: with 2 to 4 column partitions a plan remembers whether the row arrays
    allowed dropping atomics, with more than 4 it holds a list of every output row's slots made from
    the row and column arrays (the weights A_k are read at every call).  In-place changes made
    through torch are therefore noticed; after rewriting row or column arrays by other means (a
    kernel of the caller's, another library) call :meth:`invalidate` -- the reference's operator
    reads them afresh on every call."""
    name = "hyb_csrmm"

    def __init__(self, m, n, feat, num_col_parts, buckets, nrows):
        self.m, self.n, self.feat = int(m), int(n), int(feat)
        self.parts, self.buckets = int(num_col_parts), [int(b) for b in buckets]
        self.nrows = [int(r) for r in nrows]
        if len(self.nrows) != self.parts * len(self.buckets):
            raise _lib.SparseTIRError("hyb_csrmm: nrows must have num_col_parts*len(buckets) entries")
        self.L = _lib.lib()
        self._plans = _PlanCache(self.L.stir_hyb_plan_destroy)
        self._spec_cache = None
        self._last_args, self._last_dev = None, None

    @property
    def plan_builds(self):
        return self._plans.builds

    def _spec(self):
        f32, i32 = torch.float32, torch.int32
        spec = [("B", f32, self.n * self.feat), ("C", f32, self.m * self.feat)]
        nb = len(self.buckets)
        for k, r in enumerate(self.nrows):
            w = self.buckets[k % nb]
            tag = f"{k // nb}_{k % nb}"
            spec += [(f"A_{tag}", f32, r * w), (f"rows_{tag}", i32, r), (f"cols_{tag}", i32, r * w)]
        return spec

    def invalidate(self):
        """Forget every plan made from the arrays of earlier calls."""
        self._plans.clear()
        self._last_args = None

    def __del__(self):
        try:
            self._plans.clear()
        except Exception:
            pass

    def __call__(self, *args):
        if self._spec_cache is None:
            self._spec_cache = self._spec()
        b, c, triples = args[0], args[1], args[2:]
        # addresses of all arrays; torch's count of in-place changes for the row and column arrays
        try:
            key = (tuple(map(_data_ptrs, triples)), tuple(map(_version_of, triples[1::3])),
                   tuple(map(_version_of, triples[2::3])))
        except (TypeError, AttributeError):  # an argument that is no tensor: the check says which
            self._check(args, self._spec_cache)
            raise
        if _same_objects(triples, self._last_args) and self._plans.get((self._last_dev,) + key) is not None:
            # the tensor objects of the last, checked call, unchanged (and kept alive by their plan):
            # only B and C are new
            dev = self._check(args[:2], self._spec_cache[:2])
            if dev != self._last_dev:
                raise _lib.SparseTIRError(f"{self.name}: all arrays must be on one device")
        else:
            dev = self._check(args, self._spec_cache)
            self._last_args, self._last_dev = triples, dev
        key = (dev,) + key
        with torch.cuda.device(dev):
            plan = self._plans.get(key)
            if plan is None:
                nk = len(self.nrows)
                widths = (ctypes.c_int32 * len(self.buckets))(*self.buckets)
                nrows = (ctypes.c_int64 * max(nk, 1))(*self.nrows)
                plan = ctypes.c_void_p()
                A = _lib.ptr_table([_addr(t) for t in triples[0::3]])
                R = _lib.ptr_table([_addr(t) for t in triples[1::3]])
                Cc = _lib.ptr_table([_addr(t) for t in triples[2::3]])
                _lib.check(self.L.stir_hyb_plan_create(ctypes.byref(plan), self.m, self.n, self.parts,
                                                       len(self.buckets), widths, nrows, A, R, Cc))
                self._plans.put(key, plan, triples)  # the plan stores pointers into these arrays
            _lib.check(self.L.stir_hyb_spmm_f32(plan, self.feat, _ptr(b), _ptr(c), _stream()))


class SddmmPreproc(_Operator):
    name = "sddmm_preproc"

    def __init__(self, m, n, feat, nnz):
        self.m, self.n, self.feat, self.nnz = int(m), int(n), int(feat), int(nnz)
        self.L = _lib.lib()

    def _spec(self):
        f32, i32 = torch.float32, torch.int32
        return [("A", f32, self.m * self.feat), ("B", f32, self.n * self.feat),
                ("C", f32, self.nnz), ("indptr", i32, self.m + 1), ("indices", i32, self.nnz),
                ("mid", i32, self.nnz)]

    def __call__(self, *args):
        dev = self._check(args, self._spec())
        a, b, c, indptr, indices, mid = args
        with torch.cuda.device(dev):
            _lib.check(self.L.stir_sddmm_preproc(self.m, self.nnz, _ptr(indptr), _ptr(mid), _stream()))


class Sddmm(SddmmPreproc):
    name = "sddmm"

    def __call__(self, *args):
        dev = self._check(args, self._spec())
        a, b, c, indptr, indices, mid = args
        with torch.cuda.device(dev):
            _lib.check(self.L.stir_sddmm_f32(self.m, self.n, self.feat, self.nnz, _ptr(a), _ptr(b),
                                             _ptr(c), _ptr(indptr), _ptr(indices), _ptr(mid),
                                             _stream()))


class SddmmScaled(SddmmPreproc):
    """C[e] = E[e] * <A[mid[e], :], B[indices[e], :]>: f(A, B, C, indptr, indices, mid, E)."""
    name = "sddmm_scaled"

    def __call__(self, *args):
        dev = self._check(args, self._spec() + [("E", torch.float32, self.nnz)])
        a, b, c, indptr, indices, mid, e = args
        with torch.cuda.device(dev):
            _lib.check(self.L.stir_sddmm_scaled_f32(self.m, self.n, self.feat, self.nnz, _ptr(a), _ptr(b),
                                                    _ptr(c), _ptr(indptr), _ptr(indices), _ptr(mid), _ptr(e),
                                                    _stream()))


_DT = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


class BsrMM(_Operator):
    name = "bsrmm"

    def __init__(self, mb, nb, nnzb, blk, feat, dtype=torch.float16, out_dtype=None):
        self.mb, self.nb, self.nnzb, self.blk, self.feat = map(int, (mb, nb, nnzb, blk, feat))
        self.dtype = dtype
        self.out_dtype = dtype if out_dtype is None else out_dtype
        if dtype not in (torch.float16, torch.bfloat16):
            raise _lib.SparseTIRError("bsrmm: inputs must be float16 or bfloat16")
        self.L = _lib.lib()

    def __call__(self, *args):
        i32 = torch.int32
        dev = self._check(args, [("A", self.dtype, self.nnzb * self.blk * self.blk),
                                 ("X", self.dtype, self.nb * self.blk * self.feat),
                                 ("Y", self.out_dtype, self.mb * self.blk * self.feat),
                                 ("indptr", i32, self.mb + 1), ("indices", i32, self.nnzb)])
        a, x, y, indptr, indices = args
        with torch.cuda.device(dev):
            _lib.check(self.L.stir_bsr_spmm(_DT[self.dtype], _DT[self.out_dtype], self.mb, self.nb,
                                            self.blk, self.feat, self.nnzb, _ptr(a), _ptr(x), _ptr(y),
                                            _ptr(indptr), _ptr(indices), _stream()))


class DBsrMM(_Operator):
    """Doubly-compressed BSR SpMM: f(A, X, Y, indptr_0, indices_0, indptr_1, indices_1), the
    argument list of the reference's dbsrmm (examples/blocksparse/bsr_spmm.py:66-102)."""
    name = "dbsrmm"

    def __init__(self, mb, nb, nnz_rows, nnzb, blk, feat, dtype=torch.float16, out_dtype=None):
        self.mb, self.nb, self.nr, self.nnzb, self.blk, self.feat = map(int, (mb, nb, nnz_rows, nnzb, blk, feat))
        self.dtype = dtype
        self.out_dtype = dtype if out_dtype is None else out_dtype
        self.L = _lib.lib()

    def __call__(self, *args):
        i32 = torch.int32
        dev = self._check(args, [("A", self.dtype, self.nnzb * self.blk * self.blk),
                                 ("X", self.dtype, self.nb * self.blk * self.feat),
                                 ("Y", self.out_dtype, self.mb * self.blk * self.feat),
                                 ("indptr_0", i32, 2), ("indices_0", i32, self.nr),
                                 ("indptr_1", i32, self.nr + 1), ("indices_1", i32, self.nnzb)])
        a, x, y, _, rows, indptr, indices = args
        with torch.cuda.device(dev):
            _lib.check(self.L.stir_dbsr_spmm(_DT[self.dtype], _DT[self.out_dtype], self.nr, self.nb, self.blk,
                                             self.feat, self.nnzb, _ptr(a), _ptr(x), _ptr(y), _ptr(rows),
                                             _ptr(indptr), _ptr(indices), _stream()))


class TcSpMM(_Operator):
    """SpMM over the condensed (t x 1 tiles, g per group) format on the matrix cores.

    The operator keeps a plan made from the group counts on the first call with a given ``indptr``
    array (keyed by its address): the row tiles with many groups, longest first, cut into pieces
    that are summed in fp32 and rounded once.  In-place changes of ``indptr`` made through torch
    are noticed (its version counter is part of the key); after rewriting it by other means (a
    kernel of the caller's, another library) call :meth:`invalidate` -- the reference's operator
    reads the array on every call.  The first call
    of a plan allocates and synchronises the stream, so it cannot be part of a captured graph;
    later calls can."""
    name = "tcspmm"

    def __init__(self, mb, nnzb, feat, tile_size, group_size, num_b_rows, out_dtype=torch.float16):
        self.mb, self.nnzb, self.feat = int(mb), int(nnzb), int(feat)
        self.t, self.g, self.brows = int(tile_size), int(group_size), int(num_b_rows)
        self.out_dtype = out_dtype
        self.L = _lib.lib()
        self._plans = _PlanCache(self.L.stir_tc_plan_destroy)

    @property
    def plan_builds(self):
        return self._plans.builds

    def invalidate(self):
        """Forget the plans made from the contents ``indptr`` arrays had at earlier calls."""
        self._plans.clear()

    def __del__(self):
        try:
            self._plans.clear()
        except Exception:
            pass

    def __call__(self, *args):
        f16, i32 = torch.float16, torch.int32
        dev = self._check(args, [("A", f16, self.nnzb * self.t * self.g), ("B", f16, self.brows * self.feat),
                                 ("C", self.out_dtype, self.mb * self.t * self.feat),
                                 ("indptr", i32, self.mb + 1), ("indices", i32, self.nnzb * self.g)])
        a, b, c, indptr, indices = args
        with torch.cuda.device(dev):
            if self.t not in (8, 16, 32) or self.g != 16:  # refused by the library with its own message
                _lib.check(self.L.stir_tc_spmm_f16(_DT[self.out_dtype], self.mb, self.t, self.g, self.feat,
                                                   self.nnzb, _ptr(a), _ptr(b), _ptr(c), _ptr(indptr),
                                                   _ptr(indices), _stream()))
                return
            # torch counts the in-place changes it knows of: rewriting indptr with torch calls makes a new plan
            key = (dev, indptr.data_ptr(), indptr._version)
            plan = self._plans.get(key)
            if plan is None:
                plan = ctypes.c_void_p()
                _lib.check(self.L.stir_tc_plan_create(ctypes.byref(plan), self.mb, _ptr(indptr), _stream()))
                # the array stays alive with the plan: its address cannot be handed to another
                # indptr array (same size, version 0) that the key would take for this one
                self._plans.put(key, plan, indptr)
            _lib.check(self.L.stir_tc_spmm_f16_planned(plan, _DT[self.out_dtype], self.mb, self.t, self.g,
                                                       self.feat, self.nnzb,
                                                       _ptr(a), _ptr(b), _ptr(c), _ptr(indptr), _ptr(indices),
                                                       _stream()))


class Rgms(_Operator):
    """RGMS on ELL3D buckets.  ``groups`` lists the group count of every bucket, ``rows_bkt`` /
    ``cols_bkt`` the ELL rows per group and slots per ELL row.

    The operator keeps the plans of the array sets it was called with last (see :class:`_PlanCache`),
    keyed by the arrays' addresses and the version counters torch keeps for the index arrays.  From
    8192 slots on, a plan holds an edge index derived from the contents of the rows / cols / mids
    arrays: in-place changes made through torch are noticed, after changing them by other means
    call :meth:`invalidate`, or the old structure keeps being used (the reference's operator reads
    the arrays on every call).  The
    edge weights ``A_k``, ``W`` and ``X`` are read on every call -- unless the operator was built
    with ``static_weights=True``, the promise that the ``A_k`` keep the values of the first call
    (the reference's use: its ``A_k`` is the 0/1 mask); zero-weight padding slots are then left out
    of the index and the weights live inside it.  The first call of a plan allocates and
    synchronises the stream, so it cannot be part of a captured graph."""
    name = "rgms"

    _in_dtype = torch.float16
    _fns = ("stir_rgms_plan_create", "stir_rgms_f16", "stir_rgms_plan_destroy")

    _out_dtype = torch.float32

    def __init__(self, m, n, num_rels, feat_in, feat_out, rows_bkt, cols_bkt, groups, dtype=None,
                 static_weights=False, out_dtype=None):
        self._static = bool(static_weights)
        if dtype is not None and self._in_dtype is torch.float16:
            if dtype not in (torch.float16, torch.bfloat16):
                raise _lib.SparseTIRError("rgms: dtype must be torch.float16 or torch.bfloat16")
            if dtype is torch.bfloat16:  # same kernel on the bf16 matrix-core instruction
                self._in_dtype = dtype
                self._fns = ("stir_rgms_plan_create", "stir_rgms_bf16", "stir_rgms_plan_destroy")
        if out_dtype not in (None, torch.float32):
            # the reference's operator built with dtype "float16" (bench_rgcn_tensorcore.py:564-607)
            if out_dtype is not torch.float16 or self._in_dtype is not torch.float16:
                raise _lib.SparseTIRError("rgms: out_dtype must be torch.float32, or torch.float16 with fp16 inputs")
            self._out_dtype = out_dtype
            self._fns = ("stir_rgms_plan_create", "stir_rgms_f16_out_f16", "stir_rgms_plan_destroy")
        self.m, self.n, self.R = int(m), int(n), int(num_rels)
        self.fin, self.fout = int(feat_in), int(feat_out)
        self.rb, self.cb = [int(v) for v in rows_bkt], [int(v) for v in cols_bkt]
        self.groups = [int(v) for v in groups]
        self.L = _lib.lib()
        self._plans = _PlanCache(getattr(self.L, self._fns[2]))
        self._spec_cache = None
        self._last_args, self._last_dev = None, None

    @property
    def plan_builds(self):
        return self._plans.builds

    def _spec(self):
        f16, f32, i32 = self._in_dtype, torch.float32, torch.int32
        spec = [("W", f16, self.R * self.fin * self.fout), ("X", f16, self.n * self.fin),
                ("Y", self._out_dtype, self.m * self.fout)]
        for k, g in enumerate(self.groups):
            spec += [(f"A_{k}", f16, g * self.rb[k] * self.cb[k]), (f"rows_{k}", i32, g * self.rb[k]),
                     (f"cols_{k}", i32, g * self.rb[k] * self.cb[k])]
        for k, g in enumerate(self.groups):
            spec.append((f"mids_{k}", i32, g))
        return spec

    def invalidate(self):
        """Forget the plans (and edge indices) made from the arrays of earlier calls."""
        self._plans.clear()
        self._last_args = None

    def __del__(self):
        try:
            self._plans.clear()
        except Exception:
            pass

    def __call__(self, *args):
        w, x, y, rest = args[0], args[1], args[2], args[3:]
        nb = len(self.groups)
        triples, mids = rest[:3 * nb], rest[3 * nb:]
        # index arrays: address and torch's count of in-place changes; weights: address only, unless
        # the plan keeps them inside its index
        if self._spec_cache is None:
            self._spec_cache = self._spec()
        try:
            key = (tuple(map(_data_ptrs, rest)), tuple(map(_version_of, triples[1::3])),
                   tuple(map(_version_of, triples[2::3])), tuple(map(_version_of, mids)),
                   tuple(map(_version_of, triples[0::3])) if self._static else ())
        except (TypeError, AttributeError):  # an argument that is no tensor: the check says which
            self._check(args, self._spec_cache)
            raise
        if _same_objects(rest, self._last_args) and self._plans.get((self._last_dev,) + key) is not None:
            # the tensor objects of the last, checked call, unchanged (and kept alive by their plan):
            # only W, X and Y are new
            dev = self._check(args[:3], self._spec_cache[:3])
            if dev != self._last_dev:
                raise _lib.SparseTIRError(f"{self.name}: all arrays must be on one device")
        else:
            dev = self._check(args, self._spec_cache)
            self._last_args, self._last_dev = rest, dev
        key = (dev,) + key
        with torch.cuda.device(dev):
            plan = self._plans.get(key)
            if plan is None:
                plan = ctypes.c_void_p()
                rb = (ctypes.c_int32 * nb)(*self.rb)
                cb = (ctypes.c_int32 * nb)(*self.cb)
                groups = (ctypes.c_int64 * nb)(*self.groups)
                tab = lambda ts: _lib.ptr_table([_addr(t) for t in ts])
                _lib.check(getattr(self.L, self._fns[0])(ctypes.byref(plan), nb, rb, cb, groups,
                                                         tab(triples[0::3]), tab(triples[1::3]),
                                                         tab(triples[2::3]), tab(mids)))
                self._plans.put(key, plan, rest)
                if self._static and self._in_dtype is not torch.float32:
                    _lib.check(self.L.stir_rgms_plan_set_static_weights(plan, 1))
                if getattr(self, "_deterministic", False):
                    _lib.check(self.L.stir_rgms_f32_plan_set_deterministic(plan, 1))
            _lib.check(getattr(self.L, self._fns[1])(plan, self.m, self.n, self.R, self.fin, self.fout,
                                                     _ptr(w), _ptr(x), _ptr(y), _stream()))


class RgmsF32(Rgms):
    """fp32 RGMS on ELL3D buckets with W laid out [R, feat_out, feat_in]: the composable operator of
    examples/rgms/rgcn/bench_rgcn_composable.py:208-221, same argument order as :class:`Rgms`.
    From 8192 slots on (and for feature sizes up to 64) a plan builds, at its first call, an edge
    index by 64-row tile of Y, and every tile is summed on chip in a fixed order and written once:
    no atomics, the same bits on every run, and about a tenth faster than the form with atomics
    (no counterpart in the reference, whose operator adds with atomics).  ``deterministic=False``
    keeps the atomic form at every size: nothing is derived from what the index arrays hold."""
    name = "rgms_f32"
    _in_dtype = torch.float32
    _fns = ("stir_rgms_f32_plan_create", "stir_rgms_f32", "stir_rgms_f32_plan_destroy")

    def __init__(self, *args, deterministic=True, **kwargs):
        super().__init__(*args, **kwargs)
        self._deterministic = bool(deterministic)


class RgmsCsf(_Operator):
    """fp32 RGMS over the CSF arrays: f(A, W, X, Y, indptr_i, indices_i, indptr_j, indices_j), the
    non-composable operator of examples/rgms/rgcn/bench_rgcn_non_composable.py:82-112.

    By default the operator keeps plans, keyed by the addresses of the five graph arrays and torch's
    version counters of the four index arrays; from 8192 edges on (feature sizes up to 64) a plan
    holds an edge index by 64-row tile of Y (built by the first call: it allocates and synchronises)
    and Y is accumulated into without atomics: sums that come out the same, bit for bit, on every
    run, about a sixth faster than with atomics (no counterpart in the reference).
    ``deterministic=False`` is the stateless form, like the reference's operator: every call reads
    the arrays and adds to Y with atomics.  The edge values ``A`` are read on every call either way."""
    name = "rgms_csf"

    def __init__(self, m, n, num_rels, feat_in, feat_out, nnz_i, nnz_j, deterministic=True):
        self.m, self.n, self.R = int(m), int(n), int(num_rels)
        self.fin, self.fout, self.nnz_i, self.nnz_j = int(feat_in), int(feat_out), int(nnz_i), int(nnz_j)
        self.deterministic = bool(deterministic)
        self.L = _lib.lib()
        self._plans = _PlanCache(self.L.stir_rgms_csf_f32_plan_destroy)

    @property
    def plan_builds(self):
        return self._plans.builds

    def invalidate(self):
        """Forget the plans (and edge indices) made from the arrays of earlier calls."""
        self._plans.clear()

    def __del__(self):
        try:
            self._plans.clear()
        except Exception:
            pass

    def __call__(self, *args):
        f32, i32 = torch.float32, torch.int32
        dev = self._check(args, [("A", f32, self.nnz_j), ("W", f32, self.R * self.fout * self.fin),
                                 ("X", f32, self.n * self.fin), ("Y", f32, self.m * self.fout),
                                 ("indptr_i", i32, self.R + 1), ("indices_i", i32, self.nnz_i),
                                 ("indptr_j", i32, self.nnz_i + 1), ("indices_j", i32, self.nnz_j)])
        a, w, x, y, pi, ii, pj, ij = args
        if not self.deterministic:
            with torch.cuda.device(dev):
                _lib.check(self.L.stir_rgms_csf_f32(self.m, self.n, self.R, self.fin, self.fout, self.nnz_i,
                                                    self.nnz_j, _ptr(a), _ptr(w), _ptr(x), _ptr(y), _ptr(pi),
                                                    _ptr(ii), _ptr(pj), _ptr(ij), _stream()))
            return
        graph = (a, pi, ii, pj, ij)
        key = (dev, tuple(map(_data_ptrs, graph)), tuple(map(_version_of, graph[1:])))
        with torch.cuda.device(dev):
            plan = self._plans.get(key)
            if plan is None:
                plan = ctypes.c_void_p()
                _lib.check(self.L.stir_rgms_csf_f32_plan_create(ctypes.byref(plan), self.nnz_i, self.nnz_j, _ptr(a),
                                                                _ptr(pi), _ptr(ii), _ptr(pj), _ptr(ij)))
                self._plans.put(key, plan, graph)
            _lib.check(self.L.stir_rgms_csf_f32_planned(plan, self.m, self.n, self.R, self.fin, self.fout, _ptr(w),
                                                        _ptr(x), _ptr(y), _stream()))


def build_csrmm(m, n, feat, nnz):
    return CsrMM(m, n, feat, nnz)


def build_hyb_csrmm(m, n, feat, num_col_parts, buckets, nrows):
    return HybCsrMM(m, n, feat, num_col_parts, buckets, nrows)


def build_sddmm_preproc(m, n, feat, nnz):
    return SddmmPreproc(m, n, feat, nnz)


def build_sddmm(m, n, feat, nnz):
    return Sddmm(m, n, feat, nnz)


def build_sddmm_scaled(m, n, feat, nnz):
    return SddmmScaled(m, n, feat, nnz)


def build_bsrmm(mb, nb, nnzb, blk, feat, dtype=torch.float16, out_dtype=None):
    return BsrMM(mb, nb, nnzb, blk, feat, dtype, out_dtype)


def build_dbsrmm(mb, nb, nnz_rows, nnzb, blk, feat, dtype=torch.float16, out_dtype=None):
    return DBsrMM(mb, nb, nnz_rows, nnzb, blk, feat, dtype, out_dtype)


def build_tcspmm(mb, nnzb, feat, tile_size, group_size, num_b_rows, out_dtype=torch.float16):
    return TcSpMM(mb, nnzb, feat, tile_size, group_size, num_b_rows, out_dtype)


def build_rgms(m, n, num_rels, feat_in, feat_out, rows_bkt, cols_bkt, groups, dtype=torch.float16,
               static_weights=False, out_dtype=torch.float32):
    return Rgms(m, n, num_rels, feat_in, feat_out, rows_bkt, cols_bkt, groups, dtype, static_weights, out_dtype)


def build_rgms_f32(m, n, num_rels, feat_in, feat_out, rows_bkt, cols_bkt, groups, deterministic=True):
    return RgmsF32(m, n, num_rels, feat_in, feat_out, rows_bkt, cols_bkt, groups, deterministic=deterministic)


def build_rgms_csf(m, n, num_rels, feat_in, feat_out, nnz_i, nnz_j, deterministic=True):
    return RgmsCsf(m, n, num_rels, feat_in, feat_out, nnz_i, nnz_j, deterministic)
