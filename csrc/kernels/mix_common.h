// Helpers of the layer-list models' kernels (mix_*.hip; library _C_mix.so).
//
// These kernels are templated on the activation type: bf16 (raw bits) for a model served
// in bf16, float for one served in full precision.  Norms, scores, softmax, the residual
// stream and the convolution state are fp32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

namespace rfqmix {

typedef uint16_t bf16_t;

__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const bf16_t* p) {
  return __uint_as_float(((uint32_t)*p) << 16);
}
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(bf16_t* p, float v) {
  __hip_bfloat16 b = __float2bfloat16(v);               // round to nearest even
  *p = __builtin_bit_cast(bf16_t, b);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Block-wide sum for blockDim.x a multiple of 64, at most 1024.  scratch >= 16 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  if (lane == 0) scratch[wid] = v;
  __syncthreads();
  float t = (lane < nw) ? scratch[lane] : 0.f;
  t = wave_sum(t);
  __syncthreads();
  return t;
}

}  // namespace rfqmix
