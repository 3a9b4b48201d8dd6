// TVM PackedFunc adapters: unpack TVMValue/DLTensor arguments, validate them the way the
// reference's generated host stubs do, and call the plain C ABI.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "../../include/sparsetir_amd.h"
#include "../../include/sparsetir_amd_packed.h"

namespace {

thread_local void* g_stream = nullptr;
void (*g_error_hook)(const char*) = nullptr;

int packed_fail(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  stir::set_error("%s", buf);
  if (g_error_hook) g_error_hook(buf);
  return -1;
}

// Forward a failure of the plain C ABI (message already recorded) to the hook.
int forward(int rc) {
  if (rc != 0 && g_error_hook) g_error_hook(stir_last_error());
  return rc;
}

enum Where { kHost, kDevice };

struct Arr {
  void* data = nullptr;
  int64_t len = 0;
  int device_type = 0, device_id = 0;
};

struct Args {
  const char* fn;
  TVMValue* v;
  int* tc;
  int n;
  bool ok = true;
  int dev_type = -1, dev_id = -1;

  // Array argument i: one dimension, given dtype, compact, on the expected side.
  Arr arr(int i, const char* name, uint8_t code, uint8_t bits, Where where) {
    Arr a;
    if (!ok) return a;
    const int t = tc[i];
    if (t != kTVMDLTensorHandle && t != kTVMNDArrayHandle && t != kTVMOpaqueHandle && t != kTVMNullptr) {
      ok = false;
      packed_fail("%s: Expect arg[%d] to be pointer", fn, i);
      return a;
    }
    const DLTensor* d = t == kTVMNullptr ? nullptr : static_cast<const DLTensor*>(v[i].v_handle);
    if (!d) {
      ok = false;
      packed_fail("%s: %s is expected to be a tensor, got null", fn, name);
      return a;
    }
    if (d->ndim != 1) {
      ok = false;
      packed_fail("%s: %s.ndim is expected to equal 1", fn, name);
      return a;
    }
    if (d->dtype.code != code || d->dtype.bits != bits || d->dtype.lanes != 1) {
      ok = false;
      packed_fail("%s: %s.dtype is expected to be code %d bits %d lanes 1, got code %d bits %d lanes %d", fn,
                  name, code, bits, d->dtype.code, d->dtype.bits, d->dtype.lanes);
      return a;
    }
    if (d->shape[0] < 0) {
      ok = false;
      packed_fail("%s: %s.shape[0]=%lld is negative", fn, name, (long long)d->shape[0]);
      return a;
    }
    if (d->strides && d->shape[0] > 1 && d->strides[0] != 1) {
      ok = false;
      packed_fail("%s: %s.strides: expected to be compact array", fn, name);
      return a;
    }
    const bool on_dev = d->device.device_type == kDLROCM || d->device.device_type == kDLCUDA;
    const bool on_host = d->device.device_type == kDLCPU || d->device.device_type == kDLROCMHost ||
                         d->device.device_type == kDLCUDAHost;
    if ((where == kDevice && !on_dev) || (where == kHost && !on_host)) {
      ok = false;
      packed_fail("%s: %s is expected to be on the %s", fn, name, where == kDevice ? "GPU (kDLROCM)" : "CPU");
      return a;
    }
    if (where == kDevice) {
      if (dev_type < 0) {
        dev_type = d->device.device_type;
        dev_id = d->device.device_id;
      } else if (dev_type != (int)d->device.device_type || dev_id != d->device.device_id) {
        ok = false;
        packed_fail("%s: Argument %s.device_id has an unsatisfied constraint: all arrays on one device", fn,
                    name);
        return a;
      }
    }
    a.data = d->data ? static_cast<char*>(d->data) + d->byte_offset : nullptr;
    a.len = d->shape[0];
    a.device_type = d->device.device_type;
    a.device_id = d->device.device_id;
    return a;
  }

  // Device or host, whichever the tensor is on (format pass accepts both).
  bool on_device(int i) const {
    const int t = tc[i];
    if (t != kTVMDLTensorHandle && t != kTVMNDArrayHandle && t != kTVMOpaqueHandle) return false;
    const DLTensor* d = static_cast<const DLTensor*>(v[i].v_handle);
    return d && (d->device.device_type == kDLROCM || d->device.device_type == kDLCUDA);
  }

  int64_t integer(int i, const char* name) {
    if (!ok) return 0;
    if (tc[i] != kTVMArgInt) {
      ok = false;
      packed_fail("%s: Expect arg[%d] (%s) to be int", fn, i, name);
      return 0;
    }
    return v[i].v_int64;
  }

  bool count(int want) {
    if (n != want) {
      ok = false;
      packed_fail("%s: num_args should be %d", fn, want);
    }
    return ok;
  }

  bool len(const Arr& a, const char* name, int64_t want) {
    if (ok && a.len != want) {
      ok = false;
      packed_fail("%s: Argument %s.shape[0] has an unsatisfied constraint: %lld == %lld", fn, name,
                  (long long)a.len, (long long)want);
    }
    return ok;
  }
};

// Makes the arrays' device current for the call and restores the previous one.
struct DeviceGuard {
  int prev = -1;
  bool switched = false;
  int enter(int dev_id) {
    if (dev_id < 0) return 0;
    STIR_HIP(hipGetDevice(&prev));
    if (prev != dev_id) {
      STIR_HIP(hipSetDevice(dev_id));
      switched = true;
    }
    return 0;
  }
  ~DeviceGuard() {
    if (switched) (void)hipSetDevice(prev);
  }
};

bool fits_i32(int64_t x) { return x >= 0 && x <= INT32_MAX; }

// ---- cached plans for the plan-based kernels.  A plan is found again by the addresses and sizes
// of the arrays it was made from; each operator keeps the kPlanCacheEntries plans used last, so a
// caller that alternates between a few graphs (mini-batches, training and validation sets) builds
// each plan once.  Making a plan beyond that number destroys the one whose last use lies furthest
// back.
struct HybKey {
  std::vector<uintptr_t> ptrs;
  std::vector<int64_t> nums;
  bool operator==(const HybKey& o) const { return ptrs == o.ptrs && nums == o.nums; }
};
constexpr size_t kPlanCacheEntries = 8;
std::mutex g_plan_mutex;   // guards the caches, the promises and the counter below
int64_t g_plan_builds = 0;  // plans made by the PackedFuncs since the library was loaded

template <class Plan>
struct PlanCache {
  struct Entry {
    HybKey key;
    Plan* plan;
    uint64_t used;
  };
  int (*destroy)(Plan*);
  std::vector<Entry> entries;
  uint64_t clock = 0;
  explicit PlanCache(int (*d)(Plan*)) : destroy(d) {}
  Plan* find(const HybKey& key) {
    for (Entry& e : entries)
      if (e.key == key) {
        e.used = ++clock;
        return e.plan;
      }
    return nullptr;
  }
  void insert(const HybKey& key, Plan* plan) {
    if (entries.size() >= kPlanCacheEntries) {
      size_t oldest = 0;
      for (size_t i = 1; i < entries.size(); ++i)
        if (entries[i].used < entries[oldest].used) oldest = i;
      destroy(entries[oldest].plan);
      entries.erase(entries.begin() + (std::ptrdiff_t)oldest);
    }
    entries.push_back(Entry{key, plan, ++clock});
    ++g_plan_builds;
  }
  void clear() {
    for (Entry& e : entries) destroy(e.plan);
    entries.clear();
  }
};
PlanCache<stir_hyb_plan> g_hyb_plans(stir_hyb_plan_destroy);
PlanCache<stir_rgms_plan> g_rgms_plans(stir_rgms_plan_destroy);
PlanCache<stir_rgms_f32_plan> g_rgms_f32_plans(stir_rgms_f32_plan_destroy);
PlanCache<stir_rgms_csf_f32_plan> g_rgms_csf_plans(stir_rgms_csf_f32_plan_destroy);  // only under the promise below

// Promises of the caller for the plans made from now on.  Without the first, a cached plan holds
// addresses and sizes only and every call reads the index arrays afresh, as the reference's built
// operators do; with it, plans may keep what they derive from the contents of the index arrays
// (the single-writer finding that drops atomics and the slot lists of hyb, the edge index of
// RGMS; the fp32 RGMS then sums every tile of Y on chip in a fixed order instead of adding with
// atomics).
bool g_static_structure = false;
bool g_rgms_static_weights = false;

}  // namespace

extern "C" {

void stir_set_error_hook(void (*hook)(const char*)) { g_error_hook = hook; }
void stir_set_stream(void* stream) { g_stream = stream; }

int stir_packed_csrmm(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"sparsetir.csrmm", v, tc, n};
  if (!a.count(5)) return -1;
  Arr A = a.arr(0, "A", kDLFloat, 32, kDevice), B = a.arr(1, "B", kDLFloat, 32, kDevice),
      C = a.arr(2, "C", kDLFloat, 32, kDevice), P = a.arr(3, "indptr", kDLInt, 32, kDevice),
      I = a.arr(4, "indices", kDLInt, 32, kDevice);
  if (!a.ok) return -1;
  const int64_t m = P.len - 1, nnz = A.len;
  if (m < 0) return packed_fail("%s: indptr must have at least one entry", a.fn);
  a.len(I, "indices", nnz);
  if (!a.ok) return -1;
  if (m == 0) return 0;
  if (C.len % m != 0 || C.len == 0) return packed_fail("%s: C.shape[0]=%lld is not a multiple of m=%lld", a.fn, (long long)C.len, (long long)m);
  const int64_t feat = C.len / m;
  if (B.len % feat != 0) return packed_fail("%s: B.shape[0]=%lld is not a multiple of feat=%lld", a.fn, (long long)B.len, (long long)feat);
  const int64_t ncols = B.len / feat;
  if (!fits_i32(m) || !fits_i32(ncols) || !fits_i32(feat)) return packed_fail("%s: sizes exceed int32", a.fn);
  DeviceGuard g;
  if (g.enter(a.dev_id)) return forward(-1);
  return forward(stir_csr_spmm_f32((int32_t)m, (int32_t)ncols, (int32_t)feat, nnz, (const float*)A.data,
                                   (const float*)B.data, (float*)C.data, (const int32_t*)P.data,
                                   (const int32_t*)I.data, g_stream));
}

int stir_packed_hyb_csrmm(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"sparsetir.hyb_csrmm", v, tc, n};
  if (n < 4 || (n - 4) % 3 != 0) return packed_fail("%s: num_args should be 2 + 3*buckets + 2", a.fn);
  const int nk = (n - 4) / 3;
  Arr B = a.arr(0, "B", kDLFloat, 32, kDevice), C = a.arr(1, "C", kDLFloat, 32, kDevice);
  const int64_t feat = a.integer(n - 2, "feat"), parts = a.integer(n - 1, "num_col_parts");
  if (!a.ok) return -1;
  if (feat <= 0 || parts <= 0 || nk % parts != 0)
    return packed_fail("%s: feat=%lld num_col_parts=%lld do not fit %d buckets", a.fn, (long long)feat, (long long)parts, nk);
  if (B.len % feat != 0 || C.len % feat != 0) return packed_fail("%s: B/C lengths are not multiples of feat", a.fn);
  const int nb = nk / (int)parts;
  std::vector<const float*> Ak(nk);
  std::vector<const int32_t*> Rk(nk), Ck(nk);
  std::vector<int64_t> nrows(nk);
  std::vector<int32_t> widths(nb, 0);
  for (int k = 0; k < nk; ++k) {
    Arr Aa = a.arr(2 + 3 * k, "A_k", kDLFloat, 32, kDevice), Rr = a.arr(3 + 3 * k, "rows_k", kDLInt, 32, kDevice),
        Cc = a.arr(4 + 3 * k, "cols_k", kDLInt, 32, kDevice);
    if (!a.ok) return -1;
    a.len(Cc, "cols_k", Aa.len);
    if (!a.ok) return -1;
    nrows[k] = Rr.len;
    Ak[k] = (const float*)Aa.data;
    Rk[k] = (const int32_t*)Rr.data;
    Ck[k] = (const int32_t*)Cc.data;
    if (Rr.len > 0) {
      if (Aa.len % Rr.len != 0) return packed_fail("%s: A_%d length is not a multiple of its row count", a.fn, k);
      const int64_t w = Aa.len / Rr.len;
      if (widths[k % nb] != 0 && widths[k % nb] != w)
        return packed_fail("%s: bucket %d has width %lld in one partition and %d in another", a.fn, k % nb, (long long)w, widths[k % nb]);
      widths[k % nb] = (int32_t)w;
    } else if (Aa.len != 0) {
      return packed_fail("%s: A_%d has slots but no rows", a.fn, k);
    }
  }
  for (int b = 0; b < nb; ++b)
    if (widths[b] == 0) widths[b] = b ? widths[b - 1] : 1;  // width of an empty bucket is immaterial
  DeviceGuard g;
  if (g.enter(a.dev_id)) return forward(-1);
  HybKey key;
  for (int k = 0; k < nk; ++k) {
    key.ptrs.push_back((uintptr_t)Ak[k]);
    key.ptrs.push_back((uintptr_t)Rk[k]);
    key.ptrs.push_back((uintptr_t)Ck[k]);
    key.nums.push_back(nrows[k]);
  }
  for (int b = 0; b < nb; ++b) key.nums.push_back(widths[b]);
  key.nums.push_back(parts);
  key.nums.push_back(C.len / feat);
  key.nums.push_back(B.len / feat);
  key.nums.push_back(a.dev_id);
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  stir_hyb_plan* plan = g_hyb_plans.find(key);
  if (!plan) {
    if (stir_hyb_plan_create_ex(&plan, (int32_t)(C.len / feat), (int32_t)(B.len / feat), (int32_t)parts, nb,
                                widths.data(), nrows.data(), Ak.data(), Rk.data(), Ck.data(),
                                g_static_structure ? 0u : STIR_PLAN_ADDRESSES_ONLY))
      return forward(-1);
    g_hyb_plans.insert(key, plan);
  }
  return forward(stir_hyb_spmm_f32(plan, (int32_t)feat, (const float*)B.data, (float*)C.data, g_stream));
}

static int sddmm_common(const char* fn, bool preproc, TVMValue* v, int* tc, int n) {
  Args a{fn, v, tc, n};
  if (!a.count(6)) return -1;
  Arr A = a.arr(0, "A", kDLFloat, 32, kDevice), B = a.arr(1, "B", kDLFloat, 32, kDevice),
      C = a.arr(2, "C", kDLFloat, 32, kDevice), P = a.arr(3, "indptr", kDLInt, 32, kDevice),
      I = a.arr(4, "indices", kDLInt, 32, kDevice), M = a.arr(5, "mid", kDLInt, 32, kDevice);
  if (!a.ok) return -1;
  const int64_t m = P.len - 1, nnz = C.len;
  if (m < 0) return packed_fail("%s: indptr must have at least one entry", fn);
  a.len(I, "indices", nnz);
  a.len(M, "mid", nnz);
  if (!a.ok) return -1;
  if (nnz == 0) return 0;
  if (m == 0 || A.len % m != 0 || A.len == 0) return packed_fail("%s: A.shape[0] is not a multiple of m", fn);
  const int64_t feat = A.len / m;
  if (B.len % feat != 0) return packed_fail("%s: B.shape[0] is not a multiple of feat", fn);
  if (!fits_i32(m) || !fits_i32(B.len / feat) || !fits_i32(feat)) return packed_fail("%s: sizes exceed int32", fn);
  DeviceGuard g;
  if (g.enter(a.dev_id)) return forward(-1);
  if (preproc) return forward(stir_sddmm_preproc((int32_t)m, nnz, (const int32_t*)P.data, (int32_t*)M.data, g_stream));
  return forward(stir_sddmm_f32((int32_t)m, (int32_t)(B.len / feat), (int32_t)feat, nnz, (const float*)A.data,
                                (const float*)B.data, (float*)C.data, (const int32_t*)P.data,
                                (const int32_t*)I.data, (const int32_t*)M.data, g_stream));
}

int stir_packed_sddmm_preproc(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return sddmm_common("sparsetir.sddmm_preproc", true, v, tc, n);
}
int stir_packed_sddmm(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return sddmm_common("sparsetir.sddmm", false, v, tc, n);
}

// bsrmm (A, X, Y, indptr, indices, blk, feat) and dbsrmm (A, X, Y, indptr_0, indices_0, indptr_1,
// indices_1, blk, feat) differ in the two leading index arrays of the doubly-compressed form
static int packed_bsr_any(const char* name, bool doubly, TVMValue* v, int* tc, int n) {
  Args a{name, v, tc, n};
  const int x = doubly ? 2 : 0;  // index of the extra arguments
  if (!a.count(7 + x)) return -1;
  // the 16-bit type is read from A's dtype: float16 (kDLFloat/16) or bfloat16 (kDLBfloat/16)
  const DLTensor* d0 = (tc[0] == kTVMDLTensorHandle || tc[0] == kTVMNDArrayHandle || tc[0] == kTVMOpaqueHandle)
                           ? static_cast<const DLTensor*>(v[0].v_handle) : nullptr;
  if (!d0) return packed_fail("%s: Expect arg[0] to be pointer", a.fn);
  const bool bf = d0->dtype.code == kDLBfloat;
  const uint8_t code = bf ? kDLBfloat : kDLFloat;
  Arr A = a.arr(0, "A", code, 16, kDevice), X = a.arr(1, "X", code, 16, kDevice);
  const DLTensor* d2 = (tc[2] == kTVMDLTensorHandle || tc[2] == kTVMNDArrayHandle || tc[2] == kTVMOpaqueHandle)
                           ? static_cast<const DLTensor*>(v[2].v_handle) : nullptr;
  if (!d2) return packed_fail("%s: Expect arg[2] to be pointer", a.fn);
  const bool out32 = d2->dtype.code == kDLFloat && d2->dtype.bits == 32;
  Arr Y = out32 ? a.arr(2, "Y", kDLFloat, 32, kDevice) : a.arr(2, "Y", code, 16, kDevice);
  Arr P0, I0;
  if (doubly) {
    P0 = a.arr(3, "indptr_0", kDLInt, 32, kDevice);
    I0 = a.arr(4, "indices_0", kDLInt, 32, kDevice);
  }
  Arr P = a.arr(3 + x, doubly ? "indptr_1" : "indptr", kDLInt, 32, kDevice),
      I = a.arr(4 + x, doubly ? "indices_1" : "indices", kDLInt, 32, kDevice);
  const int64_t blk = a.integer(5 + x, "blk"), feat = a.integer(6 + x, "feat");
  if (!a.ok) return -1;
  const int64_t mb = P.len - 1, nnzb = I.len;  // stored block rows
  if (mb < 0 || blk <= 0 || feat <= 0) return packed_fail("%s: bad sizes", a.fn);
  a.len(A, "A", nnzb * blk * blk);
  if (doubly) {
    a.len(P0, "indptr_0", 2);
    a.len(I0, "indices_0", mb);
    if (a.ok && Y.len % (blk * feat) != 0) return packed_fail("%s: Y.shape[0] is not a multiple of blk*feat", a.fn);
  } else {
    a.len(Y, "Y", mb * blk * feat);
  }
  if (!a.ok) return -1;
  if (X.len % (blk * feat) != 0) return packed_fail("%s: X.shape[0] is not a multiple of blk*feat", a.fn);
  const int64_t nbk = X.len / (blk * feat);
  if (!fits_i32(mb) || !fits_i32(nbk) || !fits_i32(blk) || !fits_i32(feat)) return packed_fail("%s: sizes exceed int32", a.fn);
  DeviceGuard g;
  if (g.enter(a.dev_id)) return forward(-1);
  const int dt = bf ? STIR_BF16 : STIR_F16;
  if (doubly)
    return forward(stir_dbsr_spmm(dt, out32 ? STIR_F32 : dt, (int32_t)mb, (int32_t)nbk, (int32_t)blk,
                                  (int32_t)feat, nnzb, A.data, X.data, Y.data, (const int32_t*)I0.data,
                                  (const int32_t*)P.data, (const int32_t*)I.data, g_stream));
  return forward(stir_bsr_spmm(dt, out32 ? STIR_F32 : dt, (int32_t)mb, (int32_t)nbk, (int32_t)blk, (int32_t)feat,
                               nnzb, A.data, X.data, Y.data, (const int32_t*)P.data, (const int32_t*)I.data,
                               g_stream));
}

int stir_packed_bsrmm(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return packed_bsr_any("sparsetir.bsrmm", false, v, tc, n);
}

int stir_packed_dbsrmm(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return packed_bsr_any("sparsetir.dbsrmm", true, v, tc, n);
}

int stir_packed_tcspmm(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"sparsetir.tcspmm", v, tc, n};
  if (!a.count(8)) return -1;
  Arr A = a.arr(0, "A", kDLFloat, 16, kDevice), B = a.arr(1, "B", kDLFloat, 16, kDevice);
  const DLTensor* d2 = (tc[2] == kTVMDLTensorHandle || tc[2] == kTVMNDArrayHandle || tc[2] == kTVMOpaqueHandle)
                           ? static_cast<const DLTensor*>(v[2].v_handle) : nullptr;
  if (!d2) return packed_fail("%s: Expect arg[2] to be pointer", a.fn);
  const bool out32 = d2->dtype.code == kDLFloat && d2->dtype.bits == 32;
  Arr C = a.arr(2, "C", kDLFloat, out32 ? 32 : 16, kDevice);
  Arr P = a.arr(3, "indptr", kDLInt, 32, kDevice), I = a.arr(4, "indices", kDLInt, 32, kDevice);
  const int64_t feat = a.integer(5, "feat"), t = a.integer(6, "tile_size"), g = a.integer(7, "group_size");
  if (!a.ok) return -1;
  const int64_t mb = P.len - 1;
  if (mb < 0 || feat <= 0 || t <= 0 || g <= 0) return packed_fail("%s: bad sizes", a.fn);
  if (I.len % g != 0) return packed_fail("%s: indices.shape[0] is not a multiple of group_size", a.fn);
  const int64_t nnzb = I.len / g;
  a.len(A, "A", nnzb * t * g);
  a.len(C, "C", mb * t * feat);
  if (!a.ok) return -1;
  if (B.len % feat != 0) return packed_fail("%s: B.shape[0] is not a multiple of feat", a.fn);
  if (!fits_i32(mb) || !fits_i32(feat) || !fits_i32(t) || !fits_i32(g)) return packed_fail("%s: sizes exceed int32", a.fn);
  DeviceGuard guard;
  if (guard.enter(a.dev_id)) return forward(-1);
  return forward(stir_tc_spmm_f16(out32 ? STIR_F32 : STIR_F16, (int32_t)mb, (int32_t)t, (int32_t)g, (int32_t)feat,
                                  nnzb, A.data, B.data, C.data, (const int32_t*)P.data, (const int32_t*)I.data,
                                  g_stream));
}

// fp16 (W [R, fin, fout]) and fp32 (W [R, fout, fin]) forms share the argument list
static int packed_rgms_any(const char* name, bool f32, TVMValue* v, int* tc, int n) {
  Args a{name, v, tc, n};
  const int bits = f32 ? 32 : 16;
  // the 16-bit form takes float16 or bfloat16, read from W's dtype
  const DLTensor* d0 = (n > 0 && (tc[0] == kTVMDLTensorHandle || tc[0] == kTVMNDArrayHandle ||
                                  tc[0] == kTVMOpaqueHandle))
                           ? static_cast<const DLTensor*>(v[0].v_handle) : nullptr;
  const bool bf = !f32 && d0 && d0->dtype.code == kDLBfloat;
  const uint8_t fcode = bf ? kDLBfloat : kDLFloat;
  if (n < 5 || (n - 5) % 4 != 0) return packed_fail("%s: num_args should be 3 + 4*buckets + 2", a.fn);
  const int nb = (n - 5) / 4;
  // the fp16 form also writes an fp16 Y (the reference's operator built with dtype "float16")
  const DLTensor* d2 = (n > 2 && (tc[2] == kTVMDLTensorHandle || tc[2] == kTVMNDArrayHandle ||
                                  tc[2] == kTVMOpaqueHandle))
                           ? static_cast<const DLTensor*>(v[2].v_handle) : nullptr;
  const bool out16 = !f32 && !bf && d2 && d2->dtype.code == kDLFloat && d2->dtype.bits == 16;
  Arr W = a.arr(0, "W", fcode, bits, kDevice), X = a.arr(1, "X", fcode, bits, kDevice),
      Y = a.arr(2, "Y", kDLFloat, out16 ? 16 : 32, kDevice);
  const int64_t fin = a.integer(n - 2, "feat_in"), fout = a.integer(n - 1, "feat_out");
  if (!a.ok) return -1;
  if (fin <= 0 || fout <= 0 || W.len % (fin * fout) != 0 || X.len % fin != 0 || Y.len % fout != 0)
    return packed_fail("%s: W/X/Y lengths do not fit feat_in=%lld feat_out=%lld", a.fn, (long long)fin, (long long)fout);
  std::vector<const void*> Ak(nb);
  std::vector<const int32_t*> Rk(nb), Ck(nb), Mk(nb);
  std::vector<int64_t> groups(nb);
  std::vector<int32_t> rb(nb, 1), cb(nb, 1);
  for (int b = 0; b < nb; ++b) {
    Arr Aa = a.arr(3 + 3 * b, "A_k", fcode, bits, kDevice), Rr = a.arr(4 + 3 * b, "rows_k", kDLInt, 32, kDevice),
        Cc = a.arr(5 + 3 * b, "cols_k", kDLInt, 32, kDevice), Mm = a.arr(3 + 3 * nb + b, "mids_k", kDLInt, 32, kDevice);
    if (!a.ok) return -1;
    a.len(Cc, "cols_k", Aa.len);
    if (!a.ok) return -1;
    groups[b] = Mm.len;
    Ak[b] = Aa.data;
    Rk[b] = (const int32_t*)Rr.data;
    Ck[b] = (const int32_t*)Cc.data;
    Mk[b] = (const int32_t*)Mm.data;
    if (Mm.len > 0) {
      if (Rr.len % Mm.len != 0 || Rr.len == 0 || Aa.len % Rr.len != 0)
        return packed_fail("%s: bucket %d: rows/cols lengths are not multiples of the group count", a.fn, b);
      rb[b] = (int32_t)(Rr.len / Mm.len);
      cb[b] = (int32_t)(Aa.len / Rr.len);
    } else if (Rr.len != 0 || Aa.len != 0) {
      return packed_fail("%s: bucket %d has slots but no groups", a.fn, b);
    }
  }
  DeviceGuard g;
  if (g.enter(a.dev_id)) return forward(-1);
  HybKey key;
  for (int b = 0; b < nb; ++b) {
    key.ptrs.push_back((uintptr_t)Ak[b]);
    key.ptrs.push_back((uintptr_t)Rk[b]);
    key.ptrs.push_back((uintptr_t)Ck[b]);
    key.ptrs.push_back((uintptr_t)Mk[b]);
    key.nums.push_back(groups[b]);
    key.nums.push_back(rb[b]);
    key.nums.push_back(cb[b]);
  }
  key.nums.push_back(a.dev_id);
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  const int32_t mm = (int32_t)(Y.len / fout), nn = (int32_t)(X.len / fin), rr = (int32_t)(W.len / (fin * fout));
  // an edge index also depends on the sizes the launch is given
  key.nums.push_back(mm);
  key.nums.push_back(nn);
  key.nums.push_back(rr);
  if (f32) {
    stir_rgms_f32_plan* plan = g_rgms_f32_plans.find(key);
    if (!plan) {
      std::vector<const float*> Af(nb);
      for (int b = 0; b < nb; ++b) Af[b] = (const float*)Ak[b];
      if (stir_rgms_f32_plan_create(&plan, nb, rb.data(), cb.data(), groups.data(), Af.data(), Rk.data(), Ck.data(),
                                    Mk.data()))
        return forward(-1);
      if (g_static_structure && stir_rgms_f32_plan_set_deterministic(plan, 1)) {
        stir_rgms_f32_plan_destroy(plan);
        return forward(-1);
      }
      g_rgms_f32_plans.insert(key, plan);
    }
    return forward(stir_rgms_f32(plan, mm, nn, rr, (int32_t)fin, (int32_t)fout, (const float*)W.data,
                                 (const float*)X.data, (float*)Y.data, g_stream));
  }
  stir_rgms_plan* plan = g_rgms_plans.find(key);
  if (!plan) {
    if (stir_rgms_plan_create(&plan, nb, rb.data(), cb.data(), groups.data(), Ak.data(), Rk.data(), Ck.data(),
                              Mk.data()))
      return forward(-1);
    // weights inside the index only when the structure may be kept at all
    if ((!g_static_structure && stir_rgms_plan_set_addresses_only(plan, 1)) ||
        (g_static_structure && g_rgms_static_weights && stir_rgms_plan_set_static_weights(plan, 1))) {
      stir_rgms_plan_destroy(plan);
      return forward(-1);
    }
    g_rgms_plans.insert(key, plan);
  }
  if (out16)
    return forward(stir_rgms_f16_out_f16(plan, mm, nn, rr, (int32_t)fin, (int32_t)fout, W.data, X.data, Y.data,
                                         g_stream));
  return forward((bf ? stir_rgms_bf16 : stir_rgms_f16)(plan, mm, nn, rr, (int32_t)fin, (int32_t)fout, W.data, X.data,
                                                       (float*)Y.data, g_stream));
}

int stir_packed_rgms(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return packed_rgms_any("sparsetir.rgms", false, v, tc, n);
}

int stir_packed_rgms_f32(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return packed_rgms_any("sparsetir.rgms_f32", true, v, tc, n);
}

int stir_packed_invalidate_plans(TVMValue*, int*, int n, TVMRetValueHandle, void*) {
  if (n != 0) return packed_fail("sparsetir.invalidate_plans: num_args should be 0");
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  g_hyb_plans.clear();
  g_rgms_plans.clear();
  g_rgms_f32_plans.clear();
  g_rgms_csf_plans.clear();
  return 0;
}

// "sparsetir.static_structure"(on): the promise that the index arrays (rows_k, cols_k, mids_k)
// handed to hyb_csrmm / rgms keep their contents for as long as they keep their addresses
int stir_packed_static_structure(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"sparsetir.static_structure", v, tc, n};
  if (!a.count(1)) return -1;
  const int64_t on = a.integer(0, "on");
  if (!a.ok) return -1;
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  if (g_static_structure != (on != 0)) {
    // the cached plans were made under the other setting
    g_hyb_plans.clear();
    g_rgms_plans.clear();
    g_rgms_f32_plans.clear();
    g_rgms_csf_plans.clear();
  }
  g_static_structure = on != 0;
  return 0;
}

int64_t stir_packed_plan_builds(void) {
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  return g_plan_builds;
}

int stir_packed_rgms_static_weights(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"sparsetir.rgms_static_weights", v, tc, n};
  if (!a.count(1)) return -1;
  const int64_t on = a.integer(0, "on");
  if (!a.ok) return -1;
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  if (g_rgms_static_weights != (on != 0)) g_rgms_plans.clear();  // made under the other setting
  g_rgms_static_weights = on != 0;
  return 0;
}

int stir_packed_rgms_csf(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"sparsetir.rgms_csf", v, tc, n};
  if (!a.count(10)) return -1;
  Arr A = a.arr(0, "A", kDLFloat, 32, kDevice), W = a.arr(1, "W", kDLFloat, 32, kDevice),
      X = a.arr(2, "X", kDLFloat, 32, kDevice), Y = a.arr(3, "Y", kDLFloat, 32, kDevice),
      Pi = a.arr(4, "indptr_i", kDLInt, 32, kDevice), Ii = a.arr(5, "indices_i", kDLInt, 32, kDevice),
      Pj = a.arr(6, "indptr_j", kDLInt, 32, kDevice), Ij = a.arr(7, "indices_j", kDLInt, 32, kDevice);
  const int64_t fin = a.integer(8, "feat_in"), fout = a.integer(9, "feat_out");
  if (!a.ok) return -1;
  if (fin <= 0 || fout <= 0 || W.len % (fin * fout) != 0 || X.len % fin != 0 || Y.len % fout != 0)
    return packed_fail("%s: W/X/Y lengths do not fit feat_in=%lld feat_out=%lld", a.fn, (long long)fin, (long long)fout);
  const int64_t R = W.len / (fin * fout);
  a.len(Pi, "indptr_i", R + 1);
  a.len(Pj, "indptr_j", Ii.len + 1);
  a.len(Ij, "indices_j", A.len);
  if (!a.ok) return -1;
  if (!fits_i32(Y.len / fout) || !fits_i32(X.len / fin) || !fits_i32(R)) return packed_fail("%s: sizes exceed int32", a.fn);
  DeviceGuard g;
  if (g.enter(a.dev_id)) return forward(-1);
  {
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    if (g_static_structure) {  // the plan keeps an edge index made from the four index arrays
      HybKey key;
      for (const Arr* x : {&A, &Pi, &Ii, &Pj, &Ij}) key.ptrs.push_back((uintptr_t)x->data);
      for (int64_t x : {Ii.len, A.len, Y.len / fout, X.len / fin, R, (int64_t)a.dev_id}) key.nums.push_back(x);
      stir_rgms_csf_f32_plan* plan = g_rgms_csf_plans.find(key);
      if (!plan) {
        if (stir_rgms_csf_f32_plan_create(&plan, Ii.len, A.len, (const float*)A.data, (const int32_t*)Pi.data,
                                          (const int32_t*)Ii.data, (const int32_t*)Pj.data, (const int32_t*)Ij.data))
          return forward(-1);
        g_rgms_csf_plans.insert(key, plan);
      }
      return forward(stir_rgms_csf_f32_planned(plan, (int32_t)(Y.len / fout), (int32_t)(X.len / fin), (int32_t)R,
                                               (int32_t)fin, (int32_t)fout, (const float*)W.data,
                                               (const float*)X.data, (float*)Y.data, g_stream));
    }
  }
  return forward(stir_rgms_csf_f32((int32_t)(Y.len / fout), (int32_t)(X.len / fin), (int32_t)R, (int32_t)fin,
                                   (int32_t)fout, Ii.len, A.len, (const float*)A.data, (const float*)W.data,
                                   (const float*)X.data, (float*)Y.data, (const int32_t*)Pi.data,
                                   (const int32_t*)Ii.data, (const int32_t*)Pj.data, (const int32_t*)Ij.data,
                                   g_stream));
}

// ----------------------------------------------------------------------------- format pass

// Scratch of a device format pass, kept per thread between its sizing and its fill call.  It
// belongs to the device it was allocated on: a call for another device starts over.  The sizing
// call leaves the layout of the scratch behind, and that layout follows from its arguments: the
// fill call must come with the same input (`key`: addresses, sizes, bucket lists) and with
// outputs of the lengths the sizing call returned (`counts`), or its kernels would read offsets
// and write lengths that belong to another input.
struct FormatScratch {
  void* ptr = nullptr;
  size_t bytes = 0;
  int dev = -1;
  bool sized = false;
  std::vector<int64_t> key, counts;
  void forget() { sized = false, key.clear(), counts.clear(); }
  void remember(std::vector<int64_t> k, const int64_t* c, size_t n) {
    key = std::move(k);
    counts.assign(c, c + n);
    sized = true;
  }
  // at least `need` bytes on device `dev_id` (which must be current), nullptr when that fails
  void* reserve(int dev_id, size_t need) {
    forget();
    if (ptr && (dev != dev_id || need > bytes)) {
      (void)hipFree(ptr);
      ptr = nullptr;
      bytes = 0;
    }
    if (!ptr) {
      if (hipMalloc(&ptr, std::max<size_t>(need, 256)) != hipSuccess) {
        ptr = nullptr;
        return nullptr;
      }
      bytes = std::max<size_t>(need, 256);
      dev = dev_id;
    }
    return ptr;
  }
  // what the sizing call left for device `dev_id`, or nullptr
  void* get(int dev_id) const { return dev == dev_id && sized ? ptr : nullptr; }
  // the fill call's own key against the sizing call's; false with a recorded message
  bool same_input(const char* fn, const std::vector<int64_t>& k) const {
    if (k == key) return true;
    packed_fail("%s: the arguments differ from those of the .sizes call before it on this thread "
                "(arrays, sizes or bucket lists)", fn);
    return false;
  }
};
static int64_t addr_of(const void* p) { return (int64_t)(uintptr_t)p; }
static thread_local FormatScratch g_hyb_scratch, g_csf_scratch, g_condense_scratch;

static int hyb_format(const char* fn, bool fill, TVMValue* v, int* tc, int n) {
  Args a{fn, v, tc, n};
  if (n < 7) return packed_fail("%s: num_args should be at least 7", fn);
  const bool dev = a.on_device(2);
  const Where w = dev ? kDevice : kHost;
  const int64_t num_rows = a.integer(0, "num_rows"), num_cols = a.integer(1, "num_cols");
  Arr P = a.arr(2, "indptr", kDLInt, 32, w), I = a.arr(3, "indices", kDLInt, 32, w);
  const int64_t parts = a.integer(4, "num_col_parts");
  Arr Bk = a.arr(5, "buckets", kDLInt, 32, kHost);
  if (!a.ok) return -1;
  if (!fits_i32(num_rows) || !fits_i32(num_cols) || parts <= 0 || !fits_i32(parts) || Bk.len <= 0)
    return packed_fail("%s: bad sizes", fn);
  a.len(P, "indptr", num_rows + 1);
  if (!a.ok) return -1;
  const int nb = (int)Bk.len;
  const int64_t nk = parts * nb;
  auto hyb_key = [&]() {
    std::vector<int64_t> k = {num_rows, num_cols, addr_of(P.data), addr_of(I.data), I.len, parts, nb, a.dev_id};
    for (int b = 0; b < nb; ++b) k.push_back(((const int32_t*)Bk.data)[b]);
    return k;
  };
  DeviceGuard g;
  if (dev && g.enter(a.dev_id)) return forward(-1);
  if (!fill) {
    if (!a.count(7)) return -1;
    Arr N = a.arr(6, "nrows_out", kDLInt, 64, kHost);
    if (!a.ok || !a.len(N, "nrows_out", nk)) return -1;
    if (!dev)
      return forward(stir_column_part_hyb_sizes((int32_t)num_rows, (int32_t)num_cols, (const int32_t*)P.data,
                                                (const int32_t*)I.data, (int32_t)parts, (const int32_t*)Bk.data,
                                                nb, (int64_t*)N.data));
    const size_t need = stir_column_part_hyb_device_workspace_bytes((int32_t)num_rows, (int32_t)parts, nb, I.len);
    void* ws = g_hyb_scratch.reserve(a.dev_id, need);
    if (!ws) return packed_fail("%s: cannot allocate %zu bytes of scratch", fn, need);
    const int rc = stir_column_part_hyb_device_sizes((int32_t)num_rows, (int32_t)num_cols, (const int32_t*)P.data,
                                                     (const int32_t*)I.data, (int32_t)parts,
                                                     (const int32_t*)Bk.data, nb, ws, (int64_t*)N.data, g_stream);
    if (rc == 0) g_hyb_scratch.remember(hyb_key(), (const int64_t*)N.data, (size_t)nk);
    return forward(rc);
  }
  if (!a.count(6 + 3 * (int)nk)) return -1;
  std::vector<int32_t*> R(nk), C(nk), M(nk);
  for (int64_t k = 0; k < nk; ++k) {
    Arr r = a.arr(6 + 3 * (int)k, "rows_k", kDLInt, 32, w), c = a.arr(7 + 3 * (int)k, "cols_k", kDLInt, 32, w),
        mk = a.arr(8 + 3 * (int)k, "mask_k", kDLInt, 32, w);
    if (!a.ok) return -1;
    const int64_t width = ((const int32_t*)Bk.data)[k % nb];
    a.len(c, "cols_k", r.len * width);
    a.len(mk, "mask_k", r.len * width);
    if (!a.ok) return -1;
    R[k] = (int32_t*)r.data;
    C[k] = (int32_t*)c.data;
    M[k] = (int32_t*)mk.data;
  }
  if (!dev)
    return forward(stir_column_part_hyb_fill((int32_t)num_rows, (int32_t)num_cols, (const int32_t*)P.data,
                                             (const int32_t*)I.data, (int32_t)parts, (const int32_t*)Bk.data, nb,
                                             R.data(), C.data(), M.data()));
  void* ws = g_hyb_scratch.get(a.dev_id);
  if (!ws) return packed_fail("%s: call tir.sparse.ColumnPartHyb.sizes first on this thread", fn);
  if (!g_hyb_scratch.same_input(fn, hyb_key())) return -1;
  // R[k] has r.len entries; the lengths were read above, so recover them from the arguments
  for (int64_t k = 0; k < nk; ++k) {
    const DLTensor* rk = static_cast<const DLTensor*>(v[6 + 3 * (int)k].v_handle);
    if (rk->shape[0] != g_hyb_scratch.counts[(size_t)k])
      return packed_fail("%s: rows_%lld has %lld entries, the .sizes call returned %lld", fn, (long long)k,
                         (long long)rk->shape[0], (long long)g_hyb_scratch.counts[(size_t)k]);
  }
  int rc = stir_column_part_hyb_device_fill((int32_t)num_rows, (int32_t)num_cols, (const int32_t*)P.data,
                                            (const int32_t*)I.data, (int32_t)parts, (const int32_t*)Bk.data, nb,
                                            ws, R.data(), C.data(), M.data(), g_stream);
  return forward(rc);
}

int stir_packed_column_part_hyb_sizes(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return hyb_format("tir.sparse.ColumnPartHyb.sizes", false, v, tc, n);
}
int stir_packed_column_part_hyb_fill(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return hyb_format("tir.sparse.ColumnPartHyb.fill", true, v, tc, n);
}

static int csf_format(const char* fn, bool fill, TVMValue* v, int* tc, int n) {
  Args a{fn, v, tc, n};
  if (n < 7) return packed_fail("%s: num_args should be at least 7", fn);
  // CSF arrays on the GPU take the device pass and its outputs are device arrays too
  const bool dev = a.on_device(0);
  const Where w = dev ? kDevice : kHost;
  Arr P0 = a.arr(0, "csf_indptr_0", kDLInt, 32, w), I0 = a.arr(1, "csf_indices_0", kDLInt, 32, w),
      P1 = a.arr(2, "csf_indptr_1", kDLInt, 32, w), I1 = a.arr(3, "csf_indices_1", kDLInt, 32, w),
      RB = a.arr(4, "nnz_rows_bkt", kDLInt, 32, kHost), CB = a.arr(5, "nnz_cols_bkt", kDLInt, 32, kHost);
  if (!a.ok) return -1;
  if (RB.len != CB.len) return packed_fail("%s: Input nnz_rows and nnz_cols should have same length.", fn);
  const int nb = (int)CB.len;
  const int64_t rels = P0.len - 1;
  if (rels < 0 || !fits_i32(rels)) return packed_fail("%s: csf_indptr_0 must have at least one entry", fn);
  const int32_t *p0 = (const int32_t*)P0.data, *i0 = (const int32_t*)I0.data, *p1 = (const int32_t*)P1.data,
                *i1 = (const int32_t*)I1.data, *rb = (const int32_t*)RB.data, *cb = (const int32_t*)CB.data;
  if (dev && P1.len != I0.len + 1)
    return packed_fail("%s: csf_indptr_1 must have one entry more than csf_indices_0", fn);
  auto csf_key = [&]() {
    std::vector<int64_t> k = {rels, addr_of(p0), addr_of(i0), addr_of(p1), addr_of(i1), I0.len, I1.len, nb, a.dev_id};
    for (int b = 0; b < nb; ++b) k.push_back(rb[b]), k.push_back(cb[b]);
    return k;
  };
  DeviceGuard g;
  if (dev && g.enter(a.dev_id)) return forward(-1);
  if (!fill) {
    if (!a.count(7)) return -1;
    Arr G = a.arr(6, "groups_out", kDLInt, 64, kHost);
    if (!a.ok || !a.len(G, "groups_out", nb)) return -1;
    if (!dev) return forward(stir_csf_to_ell3d_sizes((int32_t)rels, p0, i0, p1, i1, rb, cb, nb, (int64_t*)G.data));
    const size_t need = stir_csf_to_ell3d_device_workspace_bytes((int32_t)rels, I0.len, nb);
    void* ws = g_csf_scratch.reserve(a.dev_id, need);
    if (!ws) return packed_fail("%s: cannot allocate %zu bytes of scratch", fn, need);
    const int rc = stir_csf_to_ell3d_device_sizes((int32_t)rels, I0.len, I1.len, p0, i0, p1, i1, rb, cb, nb, ws,
                                                  (int64_t*)G.data, g_stream);
    if (rc == 0) g_csf_scratch.remember(csf_key(), (const int64_t*)G.data, (size_t)nb);
    return forward(rc);
  }
  if (!a.count(6 + 4 * nb)) return -1;
  std::vector<int32_t*> OP(nb), R(nb), C(nb), M(nb);
  std::vector<int64_t> groups(nb);
  for (int b = 0; b < nb; ++b) {
    Arr op = a.arr(6 + 4 * b, "indptr_k", kDLInt, 32, w), r = a.arr(7 + 4 * b, "rows_k", kDLInt, 32, w),
        c = a.arr(8 + 4 * b, "cols_k", kDLInt, 32, w), mk = a.arr(9 + 4 * b, "mask_k", kDLInt, 32, w);
    if (!a.ok) return -1;
    a.len(op, "indptr_k", rels + 1);
    a.len(c, "cols_k", r.len * cb[b]);
    a.len(mk, "mask_k", r.len * cb[b]);
    if (!a.ok) return -1;
    if (rb[b] <= 0 || r.len % rb[b] != 0) return packed_fail("%s: rows_k does not hold whole groups", fn);
    groups[b] = r.len / rb[b];
    OP[b] = (int32_t*)op.data;
    R[b] = (int32_t*)r.data;
    C[b] = (int32_t*)c.data;
    M[b] = (int32_t*)mk.data;
  }
  if (!dev)
    return forward(stir_csf_to_ell3d_fill((int32_t)rels, p0, i0, p1, i1, rb, cb, nb, OP.data(), R.data(), C.data(),
                                          M.data()));
  void* ws = g_csf_scratch.get(a.dev_id);
  if (!ws) return packed_fail("%s: call tir.sparse.CSFToELL3D.sizes first on this thread", fn);
  if (!g_csf_scratch.same_input(fn, csf_key())) return -1;
  for (int b = 0; b < nb; ++b)
    if (groups[b] != g_csf_scratch.counts[(size_t)b])
      return packed_fail("%s: rows_%d holds %lld groups, the .sizes call returned %lld", fn, b, (long long)groups[b],
                         (long long)g_csf_scratch.counts[(size_t)b]);
  return forward(stir_csf_to_ell3d_device_fill((int32_t)rels, I0.len, I1.len, p0, i0, p1, i1, rb, cb, nb, ws,
                                               groups.data(), OP.data(), R.data(), C.data(), M.data(), g_stream));
}

int stir_packed_csf_to_ell3d_sizes(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return csf_format("tir.sparse.CSFToELL3D.sizes", false, v, tc, n);
}
int stir_packed_csf_to_ell3d_fill(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  return csf_format("tir.sparse.CSFToELL3D.fill", true, v, tc, n);
}

int stir_packed_condense_sizes(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"tir.sparse.ConDense.sizes", v, tc, n};
  if (!a.count(6)) return -1;
  // CSR arrays on the GPU take the device pass; group_indptr_out is then a device tensor too
  const bool dev = a.on_device(0);
  const Where w = dev ? kDevice : kHost;
  Arr P = a.arr(0, "indptr", kDLInt, 32, w), I = a.arr(1, "indices", kDLInt, 32, w);
  const int64_t t = a.integer(2, "t"), g = a.integer(3, "g");
  Arr GP = a.arr(4, "group_indptr_out", kDLInt, 32, w), NG = a.arr(5, "num_groups_out", kDLInt, 64, kHost);
  if (!a.ok) return -1;
  const int64_t rows = P.len - 1;
  if (rows < 0 || t <= 0 || g <= 0 || !fits_i32(t) || !fits_i32(g)) return packed_fail("%s: bad sizes", a.fn);
  a.len(GP, "group_indptr_out", (rows + t - 1) / t + 1);
  a.len(NG, "num_groups_out", 1);
  if (!a.ok) return -1;
  if (!dev)
    return forward(stir_condense_sizes((int32_t)rows, (const int32_t*)P.data, (const int32_t*)I.data, (int32_t)t,
                                       (int32_t)g, (int32_t*)GP.data, (int64_t*)NG.data));
  DeviceGuard guard;
  if (guard.enter(a.dev_id)) return forward(-1);
  const size_t need = stir_condense_device_workspace_bytes((int32_t)rows, I.len, (int32_t)t);
  void* g_condense_ws = g_condense_scratch.reserve(a.dev_id, need);
  if (!g_condense_ws) return packed_fail("%s: cannot allocate %zu bytes of scratch", a.fn, need);
  const int rc = stir_condense_device_sizes((int32_t)rows, I.len, (const int32_t*)P.data, (const int32_t*)I.data,
                                            (int32_t)t, (int32_t)g, g_condense_ws, (int32_t*)GP.data,
                                            (int64_t*)NG.data, g_stream);
  if (rc == 0)
    g_condense_scratch.remember({rows, addr_of(P.data), addr_of(I.data), I.len, t, g, a.dev_id},
                                (const int64_t*)NG.data, 1);
  return forward(rc);
}

// Device form: (indptr, indices, t, g, tile_indices_out, mask_out, group_indptr) -- the seventh
// argument is the array the sizing call filled.
int stir_packed_condense_fill(TVMValue* v, int* tc, int n, TVMRetValueHandle, void*) {
  Args a{"tir.sparse.ConDense.fill", v, tc, n};
  if (n < 6) return packed_fail("%s: num_args should be at least 6", a.fn);
  const bool dev = a.on_device(0);
  if (!a.count(dev ? 7 : 6)) return -1;
  const Where w = dev ? kDevice : kHost;
  Arr P = a.arr(0, "indptr", kDLInt, 32, w), I = a.arr(1, "indices", kDLInt, 32, w);
  const int64_t t = a.integer(2, "t"), g = a.integer(3, "g");
  Arr TI = a.arr(4, "tile_indices_out", kDLInt, 32, w), MK = a.arr(5, "mask_out", kDLInt, 32, w);
  if (!a.ok) return -1;
  const int64_t rows = P.len - 1;
  if (rows < 0 || t <= 0 || g <= 0 || !fits_i32(t) || !fits_i32(g)) return packed_fail("%s: bad sizes", a.fn);
  if (TI.len % g != 0 || MK.len != TI.len * t) return packed_fail("%s: output lengths do not fit t and g", a.fn);
  if (!dev)
    return forward(stir_condense_fill((int32_t)rows, (const int32_t*)P.data, (const int32_t*)I.data, (int32_t)t,
                                      (int32_t)g, (int32_t*)TI.data, (int32_t*)MK.data));
  Arr GP = a.arr(6, "group_indptr", kDLInt, 32, kDevice);
  if (!a.ok || !a.len(GP, "group_indptr", (rows + t - 1) / t + 1)) return -1;
  void* g_condense_ws = g_condense_scratch.get(a.dev_id);
  if (!g_condense_ws) return packed_fail("%s: call tir.sparse.ConDense.sizes first on this thread", a.fn);
  if (!g_condense_scratch.same_input(a.fn, {rows, addr_of(P.data), addr_of(I.data), I.len, t, g, a.dev_id})) return -1;
  if (TI.len / g != g_condense_scratch.counts[0])
    return packed_fail("%s: tile_indices_out holds %lld groups, the .sizes call returned %lld", a.fn,
                       (long long)(TI.len / g), (long long)g_condense_scratch.counts[0]);
  DeviceGuard guard;
  if (guard.enter(a.dev_id)) return forward(-1);
  return forward(stir_condense_device_fill((int32_t)rows, I.len, (const int32_t*)P.data, (const int32_t*)I.data,
                                           (int32_t)t, (int32_t)g, g_condense_ws, (const int32_t*)GP.data,
                                           TI.len / g, (int32_t*)TI.data, (int32_t*)MK.data, g_stream));
}

// ------------------------------------------------------------------------------ registry

struct PackedEntry {
  const char* name;
  TVMPackedCFunc fn;
};
static const PackedEntry kTable[] = {
    {"sparsetir.csrmm", stir_packed_csrmm},
    {"sparsetir.hyb_csrmm", stir_packed_hyb_csrmm},
    {"sparsetir.sddmm_preproc", stir_packed_sddmm_preproc},
    {"sparsetir.sddmm", stir_packed_sddmm},
    {"sparsetir.bsrmm", stir_packed_bsrmm},
    {"sparsetir.dbsrmm", stir_packed_dbsrmm},
    {"sparsetir.tcspmm", stir_packed_tcspmm},
    {"sparsetir.rgms", stir_packed_rgms},
    {"sparsetir.rgms_f32", stir_packed_rgms_f32},
    {"sparsetir.rgms_csf", stir_packed_rgms_csf},
    {"sparsetir.invalidate_plans", stir_packed_invalidate_plans},
    {"sparsetir.rgms_static_weights", stir_packed_rgms_static_weights},
    {"sparsetir.static_structure", stir_packed_static_structure},
    {"tir.sparse.ColumnPartHyb.sizes", stir_packed_column_part_hyb_sizes},
    {"tir.sparse.ColumnPartHyb.fill", stir_packed_column_part_hyb_fill},
    {"tir.sparse.CSFToELL3D.sizes", stir_packed_csf_to_ell3d_sizes},
    {"tir.sparse.CSFToELL3D.fill", stir_packed_csf_to_ell3d_fill},
    {"tir.sparse.ConDense.sizes", stir_packed_condense_sizes},
    {"tir.sparse.ConDense.fill", stir_packed_condense_fill},
};
static const int kTableSize = (int)(sizeof(kTable) / sizeof(kTable[0]));

int stir_packed_count(void) { return kTableSize; }
const char* stir_packed_name(int i) { return i >= 0 && i < kTableSize ? kTable[i].name : nullptr; }
TVMPackedCFunc stir_packed_func(int i) { return i >= 0 && i < kTableSize ? kTable[i].fn : nullptr; }

int stir_register_all(int (*create_from_cfunc)(TVMPackedCFunc, void*, TVMPackedCFuncFinalizer,
                                               TVMFunctionHandle*),
                      int (*register_global)(const char*, TVMFunctionHandle, int), int override) {
  if (!create_from_cfunc || !register_global) return packed_fail("stir_register_all: null callback");
  for (int i = 0; i < kTableSize; ++i) {
    TVMFunctionHandle h = nullptr;
    int rc = create_from_cfunc(kTable[i].fn, nullptr, nullptr, &h);
    if (rc != 0) return rc;
    rc = register_global(kTable[i].name, h, override);
    if (rc != 0) return rc;
  }
  return 0;
}

}  // extern "C"
