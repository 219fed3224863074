// seq_common.h -- helpers shared by the sequence-engine kernels (libdashinfer_hip_seq.so)
#pragma once
#include "../device_utils.h"
#include "dashinfer_hip_seq.h"

namespace dihip {

// a weight / activation element of run-time type (DIHIP_F32 or DIHIP_BF16) as f32: both conversions are exact
__device__ __forceinline__ float ld_any(const void* p, size_t i, int dt) {
  return dt == DIHIP_F32 ? ((const float*)p)[i] : bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
__device__ __forceinline__ void st_any(void* p, size_t i, int dt, float v) {
  if (dt == DIHIP_F32) ((float*)p)[i] = v;
  else ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(v);
}
inline bool seq_dtype_ok(int dt) { return dt == DIHIP_F32 || dt == DIHIP_BF16; }

// sum over the 256 threads of a block (4 waves), the same value in every thread; `red` = 4 floats of LDS.
// One fixed tree: a row's sum does not depend on the launch it is computed in.
__device__ __forceinline__ float block256_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();  // red may still be read from the call before
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

}  // namespace dihip
