// Probes of bench.py, built into libbench_probes.so (not part of the product library): what this
// GPU sustains for the two access patterns the SpMM/SDDMM kernels are made of -- a plain streaming
// copy (also the kernel of known size that the FETCH_SIZE / WRITE_SIZE counters are scaled by) and
// gathers of whole feature rows at pseudo-random row indices (no sparse structure, no arithmetic
// to speak of) -- and the rate at which its matrix cores take v_mfma_f32_32x32x16_f16 from
// registers, the instruction the BSR, TC-SpMM and RGMS kernels are built on.  All return 0 on
// success and -1 on bad arguments or a failed launch.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

__global__ __launch_bounds__(256) void probe_copy_kernel(const float4* __restrict__ src,
                                                         float4* __restrict__ dst, int64_t n16) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n16; i += stride) dst[i] = src[i];
}

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// Every lane group of `lanes` lanes (one float4 per lane) reads `per_group` rows of row_floats
// floats at hashed indices, 8 loads in flight, and sums them; the sum is stored only if it
// equals a value it cannot take, so the loads are not dead code.
__global__ __launch_bounds__(256) void probe_gather_kernel(const float* __restrict__ table, int64_t rows,
                                                           int row_floats, int lanes, int per_group,
                                                           float* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int g = lane / lanes, gl = lane % lanes;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t seed = (uint32_t)(wave * (64 / lanes) + g) * 2654435761u;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int i = 0; i < per_group; i += 8) {
    float4 x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t row = mix32(seed + i + u) % (uint64_t)rows;
      x[u] = *reinterpret_cast<const float4*>(table + row * row_floats + gl * 4);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      acc.x += x[u].x;
      acc.y += x[u].y;
      acc.z += x[u].z;
      acc.w += x[u].w;
    }
  }
  if (acc.x == 1.2345e38f) sink[0] = acc.x + acc.y + acc.z + acc.w;
}

// Every half wavefront adds 1.0 to the 32 floats of `per_group` rows at hashed indices, one
// fp32 atomic per lane and row (no return value, device scope): the scatter of an operator that
// adds 128-byte rows to its output, without the rest of that operator.
__global__ __launch_bounds__(256) void probe_atomic_rows_kernel(float* __restrict__ table, int64_t rows,
                                                                int per_group) {
  const int lane = threadIdx.x & 63;
  const int g = lane >> 5, gl = lane & 31;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t seed = (uint32_t)(wave * 2 + g) * 2654435761u;
  for (int i = 0; i < per_group; ++i) {
    const int64_t row = mix32(seed + i) % (uint64_t)rows;
    __hip_atomic_fetch_add(table + row * 32 + gl, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Every wavefront issues iters x 4 MFMAs on four independent accumulators (operands stay in
// registers; nothing is loaded).  The sum is stored only if it equals a value it cannot take.
__global__ __launch_bounds__(256) void probe_mfma_f16_kernel(int iters, float* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  f16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = (_Float16)(0.001f * (lane + i)), b[i] = (_Float16)(0.002f * (lane - i));
  f32x16 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
#pragma unroll 1
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[t], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) sum += acc[t][v];
  if (sum == 1.2345e38f) sink[0] = sum;
}

// ---- LDS access classes of the BSR tile body (sparsetir_amd/csrc/bsr.hip, bsr_tile), each in a
// kernel of its own with the tile body's addresses, for SQ_LDS_BANK_CONFLICT / SQ_ACTIVE_INST_LDS /
// SQ_INSTS_LDS: CLS 0 the 16-byte stores of the X tile, 1 the 8-byte stores of the A block, 2 the
// 16-byte reads of the A fragment, 3 the transposing reads of X (ds_read_b64_tr_b16), 4 the 16-byte
// stores of the A block of two 32-row slices.  VAR: the column swizzle of the X tile, 0 = column ^
// 2 (k & 3), 1 = none, 2 = column ^ 4 (k & 3) (what the kernels use).  NT: 128 NT features per tile.
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t probe_u32x2 __attribute__((ext_vector_type(2)));
typedef __fp16 probe_tr16x4 __attribute__((__vector_size__(4 * sizeof(__fp16))));

template <int NT, int CLS, int VAR>
__global__ __launch_bounds__(256) void probe_bsr_lds_kernel(int iters, uint32_t* out) {
  constexpr int TF = 128 * NT, FCN = TF / 8, XB = 32 * TF * 2;
  __shared__ __attribute__((aligned(16))) char lds[XB + 4096];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  for (int i = tid; i < (XB + 4096) / 4; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = i;
  __syncthreads();
  auto swizzle = [](int c, int k) { return VAR == 0 ? c ^ (2 * k) : VAR == 1 ? c : c ^ (4 * k); };
  uint32_t xdst[2 * NT];
  for (int q = 0; q < 2 * NT; ++q) {
    const int idx = 64 * (wave * 2 * NT + q) + lane, c = idx % FCN, kk = idx / FCN;
    xdst[q] = (uint32_t)(((kk >> 2) * 4 * FCN + (kk & 3) * FCN + swizzle(c, kk & 3)) * 16);
  }
  const int sl = lane & 15, half16 = (lane >> 4) & 1;
  uint32_t bread[NT];
  for (int t = 0; t < NT; ++t) {
    const int kr = sl >> 2, c = (wave * NT + t) * 4 + 2 * half16 + ((sl & 3) >> 1);
    bread[t] = (uint32_t)(((2 * h) * 4 * FCN + kr * FCN + swizzle(c, kr)) * 16 + (sl & 1) * 8);
  }
  const uint32_t aread = XB + (h * 32 + n) * 16;
  probe_u32x4 acc = {0, 0, 0, 0};
  probe_u32x4 v = {(uint32_t)tid, 1, 2, 3};
  for (int it = 0; it < iters; ++it) {
    if (CLS == 0) {
#pragma unroll
      for (int q = 0; q < 2 * NT; ++q) *reinterpret_cast<probe_u32x4*>(lds + xdst[q]) = v;
      v[0] += 1;
    } else if (CLS == 1) {
      *reinterpret_cast<probe_u32x2*>(lds + XB + tid * 8) = probe_u32x2{v[0], v[1]};
      v[0] += 1;
    } else if (CLS == 2) {
#pragma unroll
      for (int m = 0; m < 2; ++m) acc += *reinterpret_cast<const probe_u32x4*>(lds + aread + m * 1024);
    } else if (CLS == 3) {
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          typedef __attribute__((address_space(3))) probe_tr16x4 LdsTr;
          const char* bp = lds + bread[t] + (4 * m) * FCN * 64;
          const probe_tr16x4 t0 = __builtin_amdgcn_ds_read_tr16_b64_v4f16((LdsTr*)(bp));
          const probe_tr16x4 t1 = __builtin_amdgcn_ds_read_tr16_b64_v4f16((LdsTr*)(bp + FCN * 64));
          const probe_u32x2 lo = __builtin_bit_cast(probe_u32x2, t0), hi = __builtin_bit_cast(probe_u32x2, t1);
          acc += probe_u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    } else {
      *reinterpret_cast<probe_u32x4*>(lds + XB + tid * 16) = v;
      v[0] += 1;
    }
    asm volatile("" ::: "memory");
  }
  __syncthreads();
  if (acc[0] + acc[1] + acc[2] + acc[3] == 0x12345678u) out[tid] = acc[0] + lds[tid];
  if (CLS < 2 || CLS == 4) out[256 + tid] = reinterpret_cast<uint32_t*>(lds)[tid * 3];
}

}  // namespace

extern "C" {

// Launches the LDS access-class kernels of the BSR tile body one after the other (256 workgroups
// of 256 threads, `iters` rounds each; d_out: 512 words): for a counter run, see
// probe_bsr_lds_kernel.  The order of the launches is the order of the template arguments below.
int bench_probe_bsr_lds(int32_t iters, uint32_t* d_out, void* stream) {
  if (!(iters > 0 && d_out)) return -1;
  hipStream_t st = static_cast<hipStream_t>(stream);
#define BENCH_LDS(NT, CLS, VAR) \
  hipLaunchKernelGGL((probe_bsr_lds_kernel<NT, CLS, VAR>), dim3(256), dim3(256), 0, st, iters, d_out)
  BENCH_LDS(2, 0, 2); BENCH_LDS(2, 1, 2); BENCH_LDS(2, 2, 2); BENCH_LDS(2, 3, 2); BENCH_LDS(2, 4, 2);
  BENCH_LDS(1, 0, 2); BENCH_LDS(1, 3, 2);
  BENCH_LDS(2, 3, 0); BENCH_LDS(2, 3, 1);
#undef BENCH_LDS
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// waves_per_simd (1..8) wavefronts on every SIMD of `cus` compute units, each issuing iters x 4
// MFMAs of 32x32x16 (2*32*32*16 flop each); *flop receives the flop of the whole launch.
int bench_probe_mfma_f16(int32_t cus, int32_t waves_per_simd, int32_t iters, float* d_sink, double* flop,
                         void* stream) {
  if (!(cus > 0 && waves_per_simd >= 1 && waves_per_simd <= 8 && iters > 0 && d_sink && flop)) return -1;
  const int blocks = cus * waves_per_simd;  // four wavefronts each, one per SIMD
  *flop = (double)blocks * 4 * (double)iters * 4 * (2.0 * 32 * 32 * 16);
  hipLaunchKernelGGL(probe_mfma_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     iters, d_sink);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// Copies `bytes` (a multiple of 16) from d_src to d_dst.
int bench_probe_copy(const void* d_src, void* d_dst, int64_t bytes, void* stream) {
  if (!(d_src && d_dst && bytes >= 16 && bytes % 16 == 0)) return -1;
  hipLaunchKernelGGL(probe_copy_kernel, dim3(256 * 32), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float4*>(d_src), static_cast<float4*>(d_dst), bytes / 16);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// num_gathers (rounded up to whole wavefronts) reads of row_floats*4 bytes each from a table of
// `rows` rows; row_floats: a power of two in [32, 256].
int bench_probe_gather(const float* d_table, int64_t rows, int32_t row_floats, int64_t num_gathers,
                       float* d_sink, void* stream) {
  if (!(d_table && d_sink && rows > 0 && num_gathers > 0)) return -1;
  if (!(row_floats >= 32 && row_floats <= 256 && (row_floats & (row_floats - 1)) == 0)) return -1;
  const int lanes = row_floats / 4;
  const int groups_per_wave = 64 / lanes;
  const int per_group = 32;
  const int64_t per_wave = (int64_t)per_group * groups_per_wave;
  const int64_t waves = (num_gathers + per_wave - 1) / per_wave;
  const int64_t blocks = (waves + 3) / 4;
  if (blocks >= (int64_t(1) << 31)) return -1;
  hipLaunchKernelGGL(probe_gather_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     static_cast<hipStream_t>(stream), d_table, rows, row_floats, lanes, per_group, d_sink);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// num_rows (rounded up to whole workgroups' worth) additions of a row of 32 floats of 1.0 to
// hashed rows of d_table (rows x 32 floats): 32 fp32 atomics each.
int bench_probe_atomic_rows(float* d_table, int64_t rows, int64_t num_rows, void* stream) {
  if (!(d_table && rows > 0 && num_rows > 0)) return -1;
  const int per_group = 32;
  const int64_t per_block = (int64_t)per_group * 2 * 4;
  const int64_t blocks = (num_rows + per_block - 1) / per_block;
  if (blocks >= (int64_t(1) << 31)) return -1;
  hipLaunchKernelGGL(probe_atomic_rows_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     static_cast<hipStream_t>(stream), d_table, rows, per_group);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // extern "C"
