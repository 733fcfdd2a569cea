// Shared helpers of the sequence-mixer kernel library (gfx950): state-space and matrix-state scans,
// latent and windowed attention, top-k routing and the 32-bit residual stream of the layered decoders.
//
// Conventions: wave = 64 lanes; every launcher is `extern "C"`, takes raw device pointers and a
// hipStream_t, never allocates or synchronises (hipGraph-capturable) and returns the launch's
// hipError_t.  Activations come in two storage types chosen by a run-time code (0: bf16,
// 1: f32); all arithmetic is f32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define MX_API extern "C" __attribute__((visibility("default")))
#define MX_RETURN_LAUNCH() return (int)hipGetLastError()

typedef __bf16 bf16;

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16>(const bf16* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16>(bf16* p, float v) { *p = (bf16)v; }

// run BODY with T bound to the storage type of code `dt`
#define MX_DISPATCH(dt, T, ...)        \
  do {                                 \
    if ((dt) == 1) {                   \
      using T = float;                 \
      __VA_ARGS__;                     \
    } else {                           \
      using T = bf16;                  \
      __VA_ARGS__;                     \
    }                                  \
  } while (0)

__device__ __forceinline__ float mx_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ __forceinline__ float mx_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// block-wide sum, blockDim.x <= 1024; scratch: 16 floats of LDS
__device__ __forceinline__ float mx_block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = mx_wave_sum(v);
  if (lane == 0) scratch[wid] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  __syncthreads();
  return t;
}

__device__ __forceinline__ float mx_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float mx_silu(float x) { return x * mx_sigmoid(x); }
// softplus without a clamp: log(1 + e^x), evaluated so that neither tail overflows
__device__ __forceinline__ float mx_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
