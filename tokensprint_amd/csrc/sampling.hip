// Sampling over float32 logits [R, V]: argmax, and temperature sampling by
// argmax(logit/T - log E) with E ~ Exp(1), which picks token i with probability
// softmax(logits/T)[i].  The noise of (row, vocabulary index) comes from a counter hash
// keyed per row, so a token does not depend on what else is in the batch.
#include <mutex>
#include "common.h"
#include "sampling_static.h"

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

// uniform in (0, 1) from 24 bits
__device__ __forceinline__ float uniform01(uint64_t key, uint32_t index) {
  const uint64_t z = mix64(key + 0x9E3779B97F4A7C15ULL * (uint64_t)(index + 1));
  return ((float)(uint32_t)(z >> 40) + 0.5f) * (1.0f / 16777216.0f);
}

struct Best { float v; int i; };
__device__ __forceinline__ Best better(Best a, Best b) {
  // larger value wins; equal values: lower index
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

constexpr int kSlice = 4096;   // vocabulary entries one workgroup scans

__device__ __forceinline__ Best block_best(Best best, float* sv, int* si) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1)
    best = better(best, Best{__shfl_xor(best.v, o, kWave), __shfl_xor(best.i, o, kWave)});
  const int wave = threadIdx.x / kWave;
  if (threadIdx.x % kWave == 0) { sv[wave] = best.v; si[wave] = best.i; }
  __syncthreads();
  Best b{sv[0], si[0]};
  for (int w = 1; w < (int)(blockDim.x / kWave); ++w) b = better(b, Best{sv[w], si[w]});
  return b;
}

// Stage 1: workgroup (row, slice) finds the best entry of its slice of the vocabulary.
template <bool NOISE>
__global__ __launch_bounds__(256) void pick_slices_kernel(const float* __restrict__ logits,
                                                          const float* __restrict__ temperature,
                                                          const uint64_t* __restrict__ keys,
                                                          float* __restrict__ part_v,
                                                          int* __restrict__ part_i, int vocab) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int r = blockIdx.x, slice = blockIdx.y;
  const float* row = logits + (int64_t)r * vocab;
  const float temp = NOISE ? temperature[r] : 1.f;
  const bool noisy = NOISE && temp > 1e-10f;
  const float inv_t = noisy ? 1.f / temp : 1.f;
  const uint64_t key = NOISE ? keys[r] : 0;
  Best best{-INFINITY, 0x7fffffff};
  const int end = min(vocab, (slice + 1) * kSlice);
  for (int i = slice * kSlice + threadIdx.x; i < end; i += blockDim.x) {
    float s = row[i];
    if (noisy) {
      const float e = fmaxf(-logf(uniform01(key, (uint32_t)i)), 1e-10f);
      s = s * inv_t - logf(e);
    }
    best = better(best, Best{s, i});
  }
  best = block_best(best, sv, si);
  if (threadIdx.x == 0) {
    part_v[(int64_t)r * gridDim.y + slice] = best.v;
    part_i[(int64_t)r * gridDim.y + slice] = best.i;
  }
}

// Stage 2: one workgroup per row picks among the slices' winners.
__global__ __launch_bounds__(256) void pick_final_kernel(const float* __restrict__ part_v,
                                                         const int* __restrict__ part_i,
                                                         int* __restrict__ out, int slices) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int r = blockIdx.x;
  Best best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < slices; i += blockDim.x)
    best = better(best, Best{part_v[(int64_t)r * slices + i], part_i[(int64_t)r * slices + i]});
  best = block_best(best, sv, si);
  if (threadIdx.x == 0) out[r] = best.i;
}

extern "C" int ts_pick_slices(int vocab) { return (vocab + kSlice - 1) / kSlice; }

// `part_v` / `part_i`: scratch of rows * ts_pick_slices(vocab) entries each.
extern "C" int ts_argmax(const float* logits, int* out, float* part_v, int* part_i, int rows,
                         int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) TS_FAIL("argmax: vocab=%d", vocab);
  const int slices = (vocab + kSlice - 1) / kSlice;
  hipLaunchKernelGGL(pick_slices_kernel<false>, dim3(rows, slices), dim3(256), 0, stream,
                     logits, (const float*)nullptr, (const uint64_t*)nullptr, part_v, part_i,
                     vocab);
  hipLaunchKernelGGL(pick_final_kernel, dim3(rows), dim3(256), 0, stream, part_v, part_i, out,
                     slices);
  TS_CHECK_LAUNCH("argmax");
  return 0;
}

// temperature[r] <= 1e-10 means greedy for that row.
extern "C" int ts_sample(const float* logits, const float* temperature, const uint64_t* keys,
                         int* out, float* part_v, int* part_i, int rows, int vocab,
                         hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) TS_FAIL("sample: vocab=%d", vocab);
  const int slices = (vocab + kSlice - 1) / kSlice;
  hipLaunchKernelGGL(pick_slices_kernel<true>, dim3(rows, slices), dim3(256), 0, stream, logits,
                     temperature, keys, part_v, part_i, vocab);
  hipLaunchKernelGGL(pick_final_kernel, dim3(rows), dim3(256), 0, stream, part_v, part_i, out,
                     slices);
  TS_CHECK_LAUNCH("sample");
  return 0;
}

// ---------------------------------------------------------------- no allocation
// The slice winners of ts_sample_static: value and index of each, in one device array of
// the library instead of a workspace of the caller's.  In host code `scratch` is only a
// handle for hipGetSymbolAddress; the address kernels get is looked up once per device.
constexpr int kStaticWinners = 1 << 16;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[(size_t)kStaticWinners * 8];
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

extern "C" int ts_sample_static_capacity() { return kStaticWinners; }

// The device address of `scratch` on the current device (each GPU has its own copy).
static int static_scratch(void** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) TS_FAIL("sample_static: hipGetDevice: %s", hipGetErrorString(e));
  if (device < 0 || device >= kMaxDevices)
    TS_FAIL("sample_static: device %d beyond the %d this library keeps scratch for", device,
            kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      TS_FAIL("sample_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  return 0;
}

extern "C" int ts_sample_static(const float* logits, const float* temperature,
                                const uint64_t* keys, int* out, int rows, int vocab,
                                hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) TS_FAIL("sample_static: vocab=%d", vocab);
  const int slices = (vocab + kSlice - 1) / kSlice;
  if ((int64_t)rows * slices > kStaticWinners)
    TS_FAIL("sample_static: %d rows x %d slices of the vocabulary exceed the %d slice "
            "winners the library's scratch holds; use ts_sample with a workspace",
            rows, slices, kStaticWinners);
  void* base = nullptr;
  if (static_scratch(&base) != 0) return -1;
  float* part_v = (float*)base;
  int* part_i = (int*)((unsigned char*)base + (size_t)kStaticWinners * 4);
  hipLaunchKernelGGL(pick_slices_kernel<true>, dim3(rows, slices), dim3(256), 0, stream, logits,
                     temperature, keys, part_v, part_i, vocab);
  hipLaunchKernelGGL(pick_final_kernel, dim3(rows), dim3(256), 0, stream, part_v, part_i, out,
                     slices);
  TS_CHECK_LAUNCH("sample_static");
  return 0;
}
