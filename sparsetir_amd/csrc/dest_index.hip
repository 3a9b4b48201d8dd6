// Destination index and the gather-reduce kernel declared in dest_index.h.
#include "dest_index.h"

#include <hipcub/hipcub.hpp>

namespace stir {
namespace {

struct alignas(16) DevBucket {
  const int32_t* rows;
  int64_t row_begin;
};

// Z row q -> its output row: the bucket is found by binary search over row_begin.
__device__ __forceinline__ int dest_of(const DevBucket* __restrict__ tab, int nb, int64_t q) {
  int lo = 0, hi = nb - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tab[mid].row_begin <= q) lo = mid; else hi = mid - 1;
  }
  return tab[lo].rows[q - tab[lo].row_begin];
}

// keys[q] = output row of Z row q, vals[q] = q
__global__ __launch_bounds__(256) void dest_keys_kernel(const DevBucket* __restrict__ tab, int nb, int64_t z_rows,
                                                        int m, int32_t* __restrict__ keys,
                                                        int32_t* __restrict__ vals, int32_t* __restrict__ bad) {
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (q >= z_rows) return;
  int row = dest_of(tab, nb, q);
  if (row < 0 || row >= m) {
    *bad = 1;
    row = 0;
  }
  keys[q] = row;
  vals[q] = (int32_t)q;
}

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }

__device__ __forceinline__ void add4(float4& a, const float4& z) { a.x += z.x, a.y += z.y, a.z += z.z, a.w += z.w; }

// Segmented sum over the list (sorted by output row).  A lane group of 2^lg lanes (one float4 per
// lane and feature step) owns kChunk consecutive list entries whatever rows they belong to, so a
// row with thousands of ELL rows is shared by many groups.  A row that lies inside the chunk is
// added to Y with a plain read-modify-write; the rows at the two ends of the chunk may continue
// in a neighbouring chunk and are added with atomics (G consecutive float4s per instruction).
constexpr int kChunk = 64;
constexpr int kInFlight = 8;  // Z rows requested together per lane
__global__ __launch_bounds__(256) void dest_reduce_kernel(int64_t z_rows, int feat_out, int lg,
                                                          const int32_t* __restrict__ keys,
                                                          const int32_t* __restrict__ list,
                                                          const float* __restrict__ Z, float* __restrict__ Y) {
  const int G = 1 << lg;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t chunk = wave * (kWave >> lg) + (lane >> lg);
  const int64_t x0 = chunk * kChunk;
  if (x0 >= z_rows) return;
  const int64_t x1 = min(z_rows, x0 + kChunk);
  const int gl = lane & (G - 1);
  const bool head_shared = x0 > 0 && keys[x0 - 1] == keys[x0];
  const bool tail_shared = x1 < z_rows && keys[x1] == keys[x1 - 1];
  for (int c = gl * 4; c < feat_out; c += G * 4) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    int cur = keys[x0];
    bool shared = head_shared;
    auto flush = [&](int row, bool atomic) {
      float* y = Y + (int64_t)row * feat_out + c;
      if (atomic) {
        __hip_atomic_fetch_add(y + 0, acc.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_fetch_add(y + 1, acc.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_fetch_add(y + 2, acc.z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_fetch_add(y + 3, acc.w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        float4 v = ld4(y);
        add4(v, acc);
        *reinterpret_cast<float4*>(y) = v;
      }
    };
    for (int64_t x = x0; x < x1; x += kInFlight) {
      int k[kInFlight];
      float4 z[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const bool live = x + u < x1;
        k[u] = live ? keys[x + u] : -1;
        const int q = live ? list[x + u] : 0;
        z[u] = live ? ld4(Z + (int64_t)q * feat_out + c) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        if (k[u] < 0) continue;
        if (k[u] != cur) {
          flush(cur, shared);
          shared = false;
          acc = make_float4(0.f, 0.f, 0.f, 0.f);
          cur = k[u];
        }
        add4(acc, z[u]);
      }
    }
    flush(cur, shared || tail_shared);
  }
}

}  // namespace

void dest_index_free(DestIndex& ix) {
  if (ix.d_keys) (void)hipFree(ix.d_keys);
  if (ix.d_list) (void)hipFree(ix.d_list);
  if (ix.d_Z) (void)hipFree(ix.d_Z);
  ix = DestIndex();
}

int dest_index_prepare(DestIndex& ix, const std::vector<DestBucket>& buckets, int32_t m, int32_t feat_out,
                       hipStream_t stream) {
  int64_t z_rows = 0;
  for (const DestBucket& b : buckets) z_rows += b.ell_rows;
  STIR_REQUIRE(z_rows < (int64_t(1) << 31), "rgms: %lld ELL rows exceed the staging index", (long long)z_rows);
  const int64_t need = z_rows * feat_out;
  if (need > ix.z_floats) {
    if (ix.d_Z) STIR_HIP(hipFree(ix.d_Z));
    ix.d_Z = nullptr;
    ix.z_floats = 0;
    STIR_HIP(hipMalloc(reinterpret_cast<void**>(&ix.d_Z), sizeof(float) * size_t(need)));
    ix.z_floats = need;
  }
  if (ix.m == m && ix.z_rows == z_rows && ix.d_keys) return 0;
  if (ix.d_keys) STIR_HIP(hipFree(ix.d_keys));
  if (ix.d_list) STIR_HIP(hipFree(ix.d_list));
  ix.d_keys = ix.d_list = nullptr;
  ix.m = -1;
  ix.z_rows = z_rows;
  if (z_rows == 0 || m == 0) {
    ix.m = m;
    return 0;
  }
  std::vector<DevBucket> host;
  for (const DestBucket& b : buckets)
    if (b.ell_rows > 0) host.push_back(DevBucket{b.rows, b.row_begin});
  const int nb = (int)host.size();
  // the list is the stable sort of the Z rows by output row, so it is fixed by the format alone
  int end_bit = 1;
  while (end_bit < 31 && (int64_t(1) << end_bit) < m) ++end_bit;
  size_t sort_bytes = 0;
  hipError_t err = hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, (const int32_t*)nullptr, (int32_t*)nullptr,
                                                      (const int32_t*)nullptr, (int32_t*)nullptr, (int)z_rows, 0,
                                                      end_bit, stream);
  DevBucket* d_tab = nullptr;
  int32_t* d_tmp = nullptr;  // bad flag (1), unsorted keys, unsorted vals (z_rows each)
  void* d_sort = nullptr;
  if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&d_tab), sizeof(DevBucket) * host.size());
  if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&d_tmp), sizeof(int32_t) * (1 + 2 * size_t(z_rows)));
  if (err == hipSuccess) err = hipMalloc(&d_sort, sort_bytes ? sort_bytes : 16);
  if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&ix.d_keys), sizeof(int32_t) * size_t(z_rows));
  if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&ix.d_list), sizeof(int32_t) * size_t(z_rows));
  if (err == hipSuccess)
    err = hipMemcpyAsync(d_tab, host.data(), sizeof(DevBucket) * host.size(), hipMemcpyHostToDevice, stream);
  if (err == hipSuccess) err = hipMemsetAsync(d_tmp, 0, sizeof(int32_t), stream);
  int32_t bad = 0;
  if (err == hipSuccess) {
    int32_t* d_bad = d_tmp;
    int32_t* keys = d_tmp + 1;
    int32_t* vals = keys + z_rows;
    hipLaunchKernelGGL(dest_keys_kernel, dim3((unsigned)ceil_div(z_rows, 256)), dim3(256), 0, stream, d_tab, nb,
                       z_rows, m, keys, vals, d_bad);
    err = hipGetLastError();
    if (err == hipSuccess)
      err = hipcub::DeviceRadixSort::SortPairs(d_sort, sort_bytes, (const int32_t*)keys, ix.d_keys,
                                               (const int32_t*)vals, ix.d_list, (int)z_rows, 0, end_bit, stream);
    if (err == hipSuccess) err = hipMemcpyAsync(&bad, d_bad, sizeof(int32_t), hipMemcpyDeviceToHost, stream);
    if (err == hipSuccess) err = hipStreamSynchronize(stream);
  }
  if (d_tab) (void)hipFree(d_tab);
  if (d_tmp) (void)hipFree(d_tmp);
  if (d_sort) (void)hipFree(d_sort);
  if (err != hipSuccess || bad) {
    if (ix.d_keys) (void)hipFree(ix.d_keys);
    if (ix.d_list) (void)hipFree(ix.d_list);
    ix.d_keys = ix.d_list = nullptr;
    if (bad) return fail("rgms: a row id lies outside [0, %d)", m);
    return fail("rgms: building the destination index failed: %s", hipGetErrorString(err));
  }
  ix.m = m;
  return 0;
}

int dest_reduce(const DestIndex& ix, int32_t feat_out, float* d_Y, hipStream_t stream) {
  if (ix.m <= 0 || ix.z_rows == 0) return 0;
  STIR_REQUIRE(feat_out % 4 == 0, "rgms: feat_out=%d must be a multiple of 4", feat_out);
  int lg = 0;
  while ((4 << lg) < feat_out && lg < 6) ++lg;  // 2^lg lanes per chunk
  const int64_t chunks = ceil_div(ix.z_rows, kChunk);
  const int64_t blocks = ceil_div(ceil_div(chunks, kWave >> lg), 4);
  hipLaunchKernelGGL(dest_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, ix.z_rows, feat_out, lg,
                     ix.d_keys, ix.d_list, ix.d_Z, d_Y);
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // namespace stir
