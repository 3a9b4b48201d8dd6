// CSR -> BSR packing on the GPU (square blk x blk blocks), producing the canonical BSR arrays
// scipy's csr_matrix.tobsr gives the reference's BSR example (examples/blocksparse/bsr_spmm.py:441-445):
// block columns ascending inside each block row, absent entries of a stored block zero.
//
// No sort is needed: a bitmap with one bit per (block row, block column) is filled from the
// nonzeros; popcounts give the blocks per block row (-> indptr by a scan), the set bits in
// ascending order are the block column indices, and a nonzero's block position is its block
// row's offset plus the number of set bits below its block column.
#include "common.h"
#include "row_lookup.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

struct PackWs {
  uint32_t* bits;     // [mb][W] one bit per (block row, block col)
  int32_t* wprefix;   // [mb][W] set bits of the block row before word w
  int32_t* rowcnt;    // [mb+1]
  int64_t* total;     // [1]
  int32_t* status;    // [1]
  size_t bytes;
};

size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

PackWs carve(void* p, int64_t mb, int64_t W) {
  PackWs w;
  char* c = static_cast<char*>(p);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* r = c ? c + off : nullptr;
    off += align256(bytes);
    return r;
  };
  const size_t cells = size_t(mb > 0 ? mb : 1) * size_t(W > 0 ? W : 1);
  w.bits = reinterpret_cast<uint32_t*>(take(cells * 4));
  w.wprefix = reinterpret_cast<int32_t*>(take(cells * 4));
  w.rowcnt = reinterpret_cast<int32_t*>(take(size_t(mb + 1) * 4));
  w.total = reinterpret_cast<int64_t*>(take(8));
  w.status = reinterpret_cast<int32_t*>(take(4));
  w.bytes = off;
  return w;
}

constexpr int kPackPerLane = 8;  // a wavefront owns 64 * kPackPerLane consecutive nonzeros

// Sets the bit of every nonzero's block.  Neighbouring lanes hold neighbouring nonzeros, which
// mostly fall into the same block: only the first lane of a run of equal (word, bit) acts, and it
// reads the word first and skips the atomic when the bit is already there -- a block of 1024
// nonzeros costs a handful of atomics instead of 1024 on one address.
__global__ __launch_bounds__(256) void mark_kernel(int m, int n, int blk, int64_t W, int64_t nnz, int32_t first,
                                                   const int32_t* __restrict__ indptr,
                                                   const int32_t* __restrict__ indices,
                                                   uint32_t* __restrict__ bits, int32_t* __restrict__ status) {
  __shared__ int32_t win_all[4][stir::kRowLookupWindow];
  const int lane = threadIdx.x & 63;
  const int64_t end = first + nnz;
  const int64_t e0 = first + ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (kWave * kPackPerLane);
  if (e0 >= end) return;
  const int64_t e_last = min(end, e0 + kWave * kPackPerLane) - 1;
  stir::for_each_nonzero_row<kPackPerLane>(indptr, m, e0, e_last, win_all[threadIdx.x >> 6], lane,
                                           [&](int64_t e, int row, int, bool live) {
    int64_t key = -1;  // (word index, bit); -1: nothing to set
    if (live) {
      const int col = indices[e];
      if (col < 0 || col >= n)
        atomicOr(status, 1);
      else
        key = (((int64_t)(row / blk) * W + (col / blk >> 5)) << 5) | (col / blk & 31);
    }
    const int64_t before = __shfl_up(key, 1, kWave);
    if (key >= 0 && (lane == 0 || before != key)) {
      uint32_t* word = &bits[key >> 5];
      const uint32_t bit = 1u << (key & 31);
      if (!(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & bit)) atomicOr(word, bit);
    }
  });
}

// One wavefront per block row: popcount per word, exclusive prefix over the words.
__global__ __launch_bounds__(256) void count_kernel(int64_t mb, int64_t W, const uint32_t* __restrict__ bits,
                                                    int32_t* __restrict__ wprefix, int32_t* __restrict__ rowcnt) {
  const int lane = threadIdx.x & 63;
  const int64_t I = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (I >= mb) return;
  int carry = 0;
  for (int64_t w0 = 0; w0 < W; w0 += kWave) {
    const int64_t w = w0 + lane;
    const int c = w < W ? __popc(bits[I * W + w]) : 0;
    int incl = c;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const int up = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += up;
    }
    if (w < W) wprefix[I * W + w] = carry + incl - c;
    carry += __shfl(incl, kWave - 1, kWave);
  }
  if (lane == 0) rowcnt[I] = carry;
}

// Exclusive scan of rowcnt[0..mb) into out[0..mb], out[mb] = total.  One workgroup.
__global__ __launch_bounds__(256) void scan_rows_kernel(int64_t mb, const int32_t* __restrict__ rowcnt,
                                                        int32_t* __restrict__ out, int64_t* __restrict__ total) {
  __shared__ int64_t part[256];
  const int64_t chunk = (mb + 255) / 256;
  const int64_t a = chunk * threadIdx.x, b = min(mb, a + chunk);
  int64_t sum = 0;
  for (int64_t i = a; i < b; ++i) sum += rowcnt[i];
  part[threadIdx.x] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    int64_t run = 0;
    for (int t = 0; t < 256; ++t) {
      const int64_t v = part[t];
      part[t] = run;
      run += v;
    }
    total[0] = run;
    out[mb] = (int32_t)run;
  }
  __syncthreads();
  int64_t run = part[threadIdx.x];
  for (int64_t i = a; i < b; ++i) {
    const int32_t v = rowcnt[i];
    out[i] = (int32_t)run;
    run += v;
  }
}

__global__ __launch_bounds__(256) void emit_indices_kernel(int64_t mb, int64_t W, const uint32_t* __restrict__ bits,
                                                           const int32_t* __restrict__ wprefix,
                                                           const int32_t* __restrict__ bsr_indptr,
                                                           int32_t* __restrict__ bsr_indices) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= mb * W) return;
  const int64_t I = t / W, w = t % W;
  uint32_t word = bits[t];
  int64_t pos = (int64_t)bsr_indptr[I] + wprefix[t];
  while (word) {
    const int b = __ffs(word) - 1;
    bsr_indices[pos++] = (int32_t)(w * 32 + b);
    word &= word - 1;
  }
}

template <typename T>
__device__ __forceinline__ T convert(float v);
template <>
__device__ __forceinline__ float convert<float>(float v) { return v; }
template <>
__device__ __forceinline__ _Float16 convert<_Float16>(float v) { return (_Float16)v; }
struct bf16_bits {
  uint16_t u;
};
template <>
__device__ __forceinline__ bf16_bits convert<bf16_bits>(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_bits{uint16_t((u >> 16) | 0x40)};
  u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
  return bf16_bits{uint16_t(u >> 16)};
}

template <typename T>
__global__ __launch_bounds__(256) void scatter_kernel(int m, int blk, int64_t W, int64_t nnz, int32_t first,
                                                      const int32_t* __restrict__ indptr,
                                                      const int32_t* __restrict__ indices,
                                                      const float* __restrict__ values,
                                                      const uint32_t* __restrict__ bits,
                                                      const int32_t* __restrict__ wprefix,
                                                      const int32_t* __restrict__ bsr_indptr, T* __restrict__ data) {
  __shared__ int32_t win_all[4][stir::kRowLookupWindow];
  const int lane = threadIdx.x & 63;
  const int64_t end = first + nnz;
  const int64_t e0 = first + ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (kWave * kPackPerLane);
  if (e0 >= end) return;
  const int64_t e_last = min(end, e0 + kWave * kPackPerLane) - 1;
  stir::for_each_nonzero_row<kPackPerLane>(indptr, m, e0, e_last, win_all[threadIdx.x >> 6], lane,
                                           [&](int64_t e, int row, int, bool live) {
    if (!live) return;
    const int col = indices[e];
    const int I = row / blk, J = col / blk;
    const int64_t cell = (int64_t)I * W + (J >> 5);
    const int64_t pos = (int64_t)bsr_indptr[I] + wprefix[cell] + __popc(bits[cell] & ((1u << (J & 31)) - 1u));
    data[(pos * blk + (row - I * blk)) * blk + (col - J * blk)] = convert<T>(values[e]);
  });
}

int check(const char* who, int32_t m, int32_t n, int32_t blk) {
  STIR_REQUIRE(m >= 0 && n >= 0 && blk > 0, "%s: bad shape %d x %d, blk %d", who, m, n, blk);
  STIR_REQUIRE(m % blk == 0 && n % blk == 0, "%s: shape %d x %d is not a multiple of the block size %d", who, m, n, blk);
  return 0;
}

int read_ends(const int32_t* d_indptr, int32_t m, hipStream_t st, int32_t* first, int64_t* nnz) {
  int32_t ends[2];
  STIR_HIP(hipMemcpyAsync(&ends[0], d_indptr, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(&ends[1], d_indptr + m, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  *first = ends[0];
  *nnz = (int64_t)ends[1] - ends[0];
  STIR_REQUIRE(ends[0] >= 0 && *nnz >= 0, "csr_to_bsr: indptr is not a CSR row pointer");
  return 0;
}

}  // namespace

extern "C" {

size_t stir_csr_to_bsr_workspace_bytes(int32_t m, int32_t n, int32_t blk) {
  if (m < 0 || n < 0 || blk <= 0) return 0;
  return carve(nullptr, m / blk, stir::ceil_div(n / blk, 32)).bytes;
}

int stir_csr_to_bsr_sizes(int32_t m, int32_t n, int32_t blk, const int32_t* d_indptr,
                          const int32_t* d_indices, void* d_workspace, int32_t* d_bsr_indptr,
                          int64_t* nnzb, void* stream) {
  const char* who = "csr_to_bsr";
  if (check(who, m, n, blk)) return -1;
  STIR_REQUIRE(d_indptr && d_workspace && d_bsr_indptr && nnzb, "%s: null pointer argument", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t mb = m / blk, W = stir::ceil_div(n / blk, 32);
  PackWs ws = carve(d_workspace, mb, W);
  *nnzb = 0;
  if (mb == 0) {
    STIR_HIP(hipMemsetAsync(d_bsr_indptr, 0, sizeof(int32_t), st));
    return 0;
  }
  int32_t first;
  int64_t nnz;
  if (read_ends(d_indptr, m, st, &first, &nnz)) return -1;
  STIR_REQUIRE(nnz == 0 || d_indices, "%s: nonzeros but no column array", who);
  STIR_HIP(hipMemsetAsync(ws.bits, 0, size_t(mb) * size_t(W > 0 ? W : 1) * 4, st));
  STIR_HIP(hipMemsetAsync(ws.status, 0, 4, st));
  if (nnz > 0) {
    hipLaunchKernelGGL(mark_kernel, dim3((unsigned)stir::ceil_div(nnz, 4 * kWave * kPackPerLane)), dim3(256), 0, st, m, n, blk, W, nnz,
                       first, d_indptr, d_indices, ws.bits, ws.status);
    STIR_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(count_kernel, dim3((unsigned)stir::ceil_div(mb, 4)), dim3(256), 0, st, mb, W, ws.bits,
                     ws.wprefix, ws.rowcnt);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_rows_kernel, dim3(1), dim3(256), 0, st, mb, ws.rowcnt, d_bsr_indptr, ws.total);
  STIR_LAUNCH_CHECK();
  int32_t status = 0;
  STIR_HIP(hipMemcpyAsync(&status, ws.status, 4, hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(nnzb, ws.total, 8, hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  STIR_REQUIRE(status == 0, "%s: a column index lies outside [0, %d)", who, n);
  STIR_REQUIRE(*nnzb <= INT32_MAX, "%s: %lld blocks exceed int32 indexing", who, (long long)*nnzb);
  return 0;
}

int stir_csr_to_bsr_fill(int32_t m, int32_t n, int32_t blk, const int32_t* d_indptr,
                         const int32_t* d_indices, const float* d_values, void* d_workspace,
                         const int32_t* d_bsr_indptr, int32_t* d_bsr_indices, void* d_bsr_data,
                         int32_t data_dtype, int64_t nnzb, void* stream) {
  const char* who = "csr_to_bsr";
  if (check(who, m, n, blk)) return -1;
  STIR_REQUIRE(data_dtype == STIR_F32 || data_dtype == STIR_F16 || data_dtype == STIR_BF16,
               "%s: data_dtype must be STIR_F32, STIR_F16 or STIR_BF16", who);
  const int64_t mb = m / blk, W = stir::ceil_div(n / blk, 32);
  if (mb == 0 || nnzb == 0) return 0;
  STIR_REQUIRE(d_indptr && d_indices && d_values && d_workspace && d_bsr_indptr && d_bsr_indices && d_bsr_data,
               "%s: null pointer argument", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  PackWs ws = carve(d_workspace, mb, W);
  int32_t first;
  int64_t nnz;
  if (read_ends(d_indptr, m, st, &first, &nnz)) return -1;
  const size_t esize = data_dtype == STIR_F32 ? 4 : 2;
  STIR_HIP(hipMemsetAsync(d_bsr_data, 0, size_t(nnzb) * blk * blk * esize, st));
  hipLaunchKernelGGL(emit_indices_kernel, dim3((unsigned)stir::ceil_div(mb * W, 256)), dim3(256), 0, st, mb, W,
                     ws.bits, ws.wprefix, d_bsr_indptr, d_bsr_indices);
  STIR_LAUNCH_CHECK();
  if (nnz > 0) {
    dim3 grid((unsigned)stir::ceil_div(nnz, 4 * kWave * kPackPerLane)), block(256);
#define STIR_SCATTER(T)                                                                                    \
  hipLaunchKernelGGL((scatter_kernel<T>), grid, block, 0, st, m, blk, W, nnz, first, d_indptr, d_indices,  \
                     d_values, ws.bits, ws.wprefix, d_bsr_indptr, static_cast<T*>(d_bsr_data))
    if (data_dtype == STIR_F32) STIR_SCATTER(float);
    else if (data_dtype == STIR_F16) STIR_SCATTER(_Float16);
    else STIR_SCATTER(bf16_bits);
#undef STIR_SCATTER
    STIR_LAUNCH_CHECK();
  }
  return 0;
}

}  // extern "C"
