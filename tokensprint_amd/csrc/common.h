// Shared device helpers and the C interface conventions of the kernel library.
//
// Every entry point is `extern "C" int ts_<name>(..., hipStream_t stream)`: it checks
// its arguments on the host, launches on the given stream and returns 0, or returns a
// negative code after storing a message that ts_last_error() hands out.  Element types
// travel as codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define TS_F32 0
#define TS_BF16 1

typedef __bf16 bf16_t;

extern "C" const char* ts_last_error();
void ts_set_error(const char* fmt, ...);

#define TS_FAIL(...)            \
  do {                          \
    ts_set_error(__VA_ARGS__);  \
    return -1;                  \
  } while (0)

#define TS_CHECK_LAUNCH(name)                                                   \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) TS_FAIL("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch`
// holds one float per wave.  The order of the additions is fixed by the thread layout,
// so a row's result does not depend on what else is in the launch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

// Dispatch a two-way element type code to a template argument.
#define TS_DISPATCH_TYPE(code, T, ...)                    \
  if ((code) == TS_F32) { typedef float T; __VA_ARGS__; } \
  else if ((code) == TS_BF16) { typedef bf16_t T; __VA_ARGS__; } \
  else TS_FAIL("unknown element type code %d", (int)(code));
