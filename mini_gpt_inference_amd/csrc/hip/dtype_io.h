// Loads and stores through a storage type chosen at run time (the dtype codes of common.h), for
// kernels whose arithmetic is float32 whatever their buffers hold: the branch is the same for every
// lane, and the kernels that use it are bound by latency or memory, not by instruction issue.
#pragma once
#include "common.h"

__host__ __device__ __forceinline__ bool dtype_ok(int dtype) { return dtype == MGPT_F32 || dtype == MGPT_BF16; }

__device__ __forceinline__ float load_f(const void* p, int dtype, long i) {
  return dtype == MGPT_F32 ? ((const float*)p)[i] : bf16_to_float(((const bf16_t*)p)[i]);
}

__device__ __forceinline__ void store_f(void* p, int dtype, long i, float v) {
  if (dtype == MGPT_F32) ((float*)p)[i] = v;
  else ((bf16_t*)p)[i] = float_to_bf16(v);
}
