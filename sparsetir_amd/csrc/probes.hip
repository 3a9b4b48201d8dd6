// Bandwidth probes used by the benchmark to state what this GPU sustains for the two access
// patterns the SpMM/SDDMM kernels are made of: a plain streaming copy, and gathers of whole
// feature rows at pseudo-random row indices (no sparse structure, no arithmetic to speak of).
#include "common.h"
#include "../../include/sparsetir_amd.h"

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

}  // namespace

extern "C" {

int stir_probe_copy(const void* d_src, void* d_dst, int64_t bytes, void* stream) {
  STIR_REQUIRE(d_src && d_dst && bytes >= 16 && bytes % 16 == 0, "probe_copy: need 16-byte multiples");
  hipLaunchKernelGGL(probe_copy_kernel, dim3(256 * 32), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float4*>(d_src), static_cast<float4*>(d_dst), bytes / 16);
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_probe_gather(const float* d_table, int64_t rows, int32_t row_floats, int64_t num_gathers,
                      float* d_sink, void* stream) {
  STIR_REQUIRE(d_table && d_sink && rows > 0 && num_gathers > 0, "probe_gather: bad arguments");
  STIR_REQUIRE(row_floats >= 32 && row_floats <= 256 && (row_floats & (row_floats - 1)) == 0,
               "probe_gather: row_floats=%d must be a power of two in [32, 256]", row_floats);
  const int lanes = row_floats / 4;
  const int groups_per_wave = 64 / lanes;
  const int per_group = 32;
  const int64_t waves = stir::ceil_div(num_gathers, (int64_t)per_group * groups_per_wave);
  const int64_t blocks = stir::ceil_div(waves, 4);
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "probe_gather: too many gathers for one launch");
  hipLaunchKernelGGL(probe_gather_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     static_cast<hipStream_t>(stream), d_table, rows, row_floats, lanes, per_group, d_sink);
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
