// Shared helpers of the sequence-mixer kernels (recurrent state layers, latent attention,
// learned positions): activations are bf16 or fp32 (template T), every vector parameter,
// state and reduction is fp32.
#pragma once
#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>

namespace sm {

typedef __hip_bfloat16 bf16;

template <typename T> __device__ __forceinline__ float ldf(const T* p, size_t i);
template <> __device__ __forceinline__ float ldf<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldf<bf16>(const bf16* p, size_t i) {
  return __bfloat162float(p[i]);
}
template <typename T> __device__ __forceinline__ void stf(T* p, size_t i, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stf<bf16>(bf16* p, size_t i, float v) {
  p[i] = __float2bfloat16(v);
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) {
  return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x)));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// sum over the block; `red` holds one float per wave (<= 16 waves)
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = 0.0f;
  for (int i = 0; i < nw; i++) s += red[i];
  return s;
}

// entries of a step: one per sequence portion, int32 x 4
struct Entry {
  int row0, n, start, slot;
};
__device__ __forceinline__ Entry load_entry(const int* ent, int e) {
  Entry x;
  x.row0 = ent[4 * e];
  x.n = ent[4 * e + 1];
  x.start = ent[4 * e + 2];
  x.slot = ent[4 * e + 3];
  return x;
}

}  // namespace sm

#define SM_DISPATCH_T(f32, ...)         \
  do {                                  \
    if (f32) {                          \
      typedef float T;                  \
      __VA_ARGS__;                      \
    } else {                            \
      typedef sm::bf16 T;               \
      __VA_ARGS__;                      \
    }                                   \
  } while (0)
