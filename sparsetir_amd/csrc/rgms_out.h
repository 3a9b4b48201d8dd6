// How the fp16 RGMS kernels read and write an element of Y: fp32, or fp16 (the output type of the
// reference's tensor-core operator when it is built with dtype "float16",
// examples/rgms/rgcn/bench_rgcn_tensorcore.py:564-607).  Sums are kept in fp32 either way; an fp16
// element is rounded once per store and once per atomic addition.
#pragma once
#include <hip/hip_runtime.h>

namespace stir {

typedef _Float16 y_half2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float y_load(const float* p) { return *p; }
__device__ __forceinline__ float y_load(const _Float16* p) { return (float)*p; }
__device__ __forceinline__ void y_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void y_store(_Float16* p, float v) { *p = (_Float16)v; }

// Atomic addition of `v` at `p` by the lanes for which `on` holds.  Lanes 2k and 2k + 1 of the
// wavefront must address neighbouring elements of one row (the even lane the even element) and
// agree on `on`; every lane of the wavefront that is active must call it.  There is no 16-bit
// atomic addition: the even lane adds both lanes' values with one packed instruction.
__device__ __forceinline__ void y_atomic_add(float* p, float v, bool on, int /*lane*/) {
  if (on) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void y_atomic_add(_Float16* p, float v, bool on, int lane) {
  const float other = __shfl_xor(v, 1, 64);
  if (on && !(lane & 1)) {
    const y_half2 pair = {(_Float16)v, (_Float16)other};
    (void)__builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) y_half2*)p, pair);
  }
}

}  // namespace stir
