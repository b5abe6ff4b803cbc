// Floating-point accumulation into LDS cells shared by many lanes and wavefronts.
//
// On gfx950 the LDS fp32 atomic add (ds_add_f32) measures at ~190 cycles per 64-lane instruction, against ~8 for the
// integer LDS atomics and ~21 for ds_add_f64. Accumulators that take many updates are therefore kept in fp64 (plain
// atomicAdd on a double). Where an fp32 cell has to be updated in place, lds_add(float*) uses a compare-and-swap loop
// on the integer LDS atomic unit: it is lock free (a lane only retries because another lane's update went through),
// so it needs no particular loop shape from the compiler and cannot deadlock a wavefront.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ht {

__device__ __forceinline__ void lds_add(float *p, float v) {
  uint32_t *q = reinterpret_cast<uint32_t *>(p);
  uint32_t seen = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  for (;;) {
    const uint32_t want = __float_as_uint(__uint_as_float(seen) + v);
    if (__hip_atomic_compare_exchange_strong(q, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_WORKGROUP))
      break;
  }
}

__device__ __forceinline__ void lds_add(double *p, double v) { atomicAdd(p, v); }

}  // namespace ht
