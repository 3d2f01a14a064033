// Row-wise kernels: embedding gather, row gather, RMSNorm (with and without the fused
// residual add), SiLU-multiply.  One workgroup per row; sums in float32.
#include "common.h"

// ---------------------------------------------------------------- embedding
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int width) {
  const int64_t t = blockIdx.x;
  const TW* row = table + (int64_t)ids[t] * width;
  float* o = out + t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = to_f32(row[i]);
}

extern "C" int ts_embed(const void* table, int table_type, int vocab, const int* ids,
                        float* out, int num_tokens, int width, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || vocab <= 0) TS_FAIL("embed: bad sizes width=%d vocab=%d", width, vocab);
  TS_DISPATCH_TYPE(table_type, TW,
                   hipLaunchKernelGGL(embed_kernel<TW>, dim3(num_tokens), dim3(256), 0, stream,
                                      (const TW*)table, ids, out, width));
  TS_CHECK_LAUNCH("embed");
  return 0;
}

// ---------------------------------------------------------------- tokens drawn on the device
// ids[i] = drawn[src[i]] where 0 <= src[i] < num_drawn: a step that was launched before
// the host saw the step before it takes its lanes' tokens from where that step's draw
// left them.
__global__ void take_tokens_kernel(int* __restrict__ ids, const int* __restrict__ src,
                                   const int* __restrict__ drawn, int n, int num_drawn) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int s = src[i];
  if (s >= 0 && s < num_drawn) ids[i] = drawn[s];
}

extern "C" int ts_take_tokens(int* ids, const int* src, const int* drawn, int n, int num_drawn,
                              hipStream_t stream) {
  if (n <= 0) return 0;
  if (num_drawn <= 0) TS_FAIL("take_tokens: no drawn tokens to take from");
  hipLaunchKernelGGL(take_tokens_kernel, dim3((n + 63) / 64), dim3(64), 0, stream, ids, src,
                     drawn, n, num_drawn);
  TS_CHECK_LAUNCH("take_tokens");
  return 0;
}

// ---------------------------------------------------------------- row gather
template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ x, const int* __restrict__ rows,
                                   T* __restrict__ out, int width) {
  const int64_t r = blockIdx.x;
  const T* src = x + (int64_t)rows[r] * width;
  T* dst = out + r * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
}

extern "C" int ts_gather_rows(const void* x, int type, const int* rows, void* out,
                              int num_rows, int width, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  TS_DISPATCH_TYPE(type, T,
                   hipLaunchKernelGGL(gather_rows_kernel<T>, dim3(num_rows), dim3(256), 0,
                                      stream, (const T*)x, rows, (T*)out, width));
  TS_CHECK_LAUNCH("gather_rows");
  return 0;
}

// ---------------------------------------------------------------- RMSNorm
// out = x * rsqrt(mean(x^2) + eps) * w.  With `delta`, first resid += delta (float32,
// written back) and the norm is taken of the sum.
template <typename TX, typename TD, typename TO, bool ADD>
__global__ void rmsnorm_kernel(TX* __restrict__ x, const TD* __restrict__ delta,
                               const float* __restrict__ w, TO* __restrict__ out, int width,
                               float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  TX* xr = x + row * width;
  const TD* dr = ADD ? delta + row * width : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = to_f32(xr[i]);
    if (ADD) {
      v += to_f32(dr[i]);
      xr[i] = from_f32<TX>(v);
    }
    ss += v * v;
  }
  const float rstd = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
  TO* o = out + row * width;
  // each thread re-reads what it wrote itself, so no barrier is needed for x
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    o[i] = from_f32<TO>(to_f32(xr[i]) * rstd * w[i]);
}

// The same for a float32 x whose rows are a multiple of 4 wide and fit the registers of a
// workgroup (the residual stream of every model so far): 16-byte loads, each value read
// once and kept, and the stores after the loads, which share a counter with them.
typedef __attribute__((ext_vector_type(4))) float f32x4_rows;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_rows;
__device__ __forceinline__ f32x4_rows load4(const float* p) { return *(const f32x4_rows*)p; }
__device__ __forceinline__ f32x4_rows load4(const bf16_t* p) {
  const bf16x4_rows v = *(const bf16x4_rows*)p;
  return f32x4_rows{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
__device__ __forceinline__ void store4(float* p, f32x4_rows v) { *(f32x4_rows*)p = v; }
__device__ __forceinline__ void store4(bf16_t* p, f32x4_rows v) {
  *(bf16x4_rows*)p = bf16x4_rows{(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
}

template <typename TD, typename TO, bool ADD, int VPT>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(float* __restrict__ x,
                                                          const TD* __restrict__ delta,
                                                          const float* __restrict__ w,
                                                          TO* __restrict__ out, int width,
                                                          float eps) {
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  const int n4 = width / 4;
  f32x4_rows v[VPT];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    v[j] = f32x4_rows{0.f, 0.f, 0.f, 0.f};
    if (i < n4) {
      v[j] = load4(x + base + i * 4);
      if (ADD) {
        const f32x4_rows d = load4(delta + base + i * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[j][e] += d[e];
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += v[j][e] * v[j][e];
  }
  f32x4_rows wv[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    wv[j] = i < n4 ? load4(w + i * 4) : f32x4_rows{0.f, 0.f, 0.f, 0.f};
  }
  const float rstd = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i >= n4) continue;
    if (ADD) store4(x + base + i * 4, v[j]);
    f32x4_rows o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = v[j][e] * rstd * wv[j][e];
    store4(out + base + i * 4, o);
  }
}

// Launches the vector kernel if the row fits; returns false if it does not.
template <typename TD, typename TO, bool ADD>
static bool launch_rmsnorm_vec(float* x, const TD* delta, const float* w, TO* out, int rows,
                               int width, float eps, hipStream_t stream) {
  if (width % 4 || width > 256 * 4 * 8) return false;
  if (((uintptr_t)x | (uintptr_t)delta | (uintptr_t)w | (uintptr_t)out) & 15) return false;
  const int n4 = width / 4;
  const int threads = n4 >= 256 ? 256 : (n4 >= 128 ? 128 : 64);
  const int vpt = (n4 + threads - 1) / threads;
  if (vpt <= 1)
    hipLaunchKernelGGL((rmsnorm_vec_kernel<TD, TO, ADD, 1>), dim3(rows), dim3(threads), 0, stream, x, delta, w, out, width, eps);
  else if (vpt <= 2)
    hipLaunchKernelGGL((rmsnorm_vec_kernel<TD, TO, ADD, 2>), dim3(rows), dim3(threads), 0, stream, x, delta, w, out, width, eps);
  else if (vpt <= 4)
    hipLaunchKernelGGL((rmsnorm_vec_kernel<TD, TO, ADD, 4>), dim3(rows), dim3(threads), 0, stream, x, delta, w, out, width, eps);
  else
    hipLaunchKernelGGL((rmsnorm_vec_kernel<TD, TO, ADD, 8>), dim3(rows), dim3(threads), 0, stream, x, delta, w, out, width, eps);
  return true;
}

extern "C" int ts_rmsnorm(const void* x, int x_type, const float* w, void* out, int out_type,
                          int rows, int width, float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0) TS_FAIL("rmsnorm: width=%d", width);
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  if (x_type == TS_F32) {
    bool done = false;
    TS_DISPATCH_TYPE(out_type, TO, done = launch_rmsnorm_vec<float, TO, false>(
        (float*)x, (const float*)nullptr, w, (TO*)out, rows, width, eps, stream));
    if (done) {
      TS_CHECK_LAUNCH("rmsnorm");
      return 0;
    }
  }
  TS_DISPATCH_TYPE(x_type, TX, TS_DISPATCH_TYPE(out_type, TO,
      hipLaunchKernelGGL((rmsnorm_kernel<TX, float, TO, false>), dim3(rows), dim3(threads), 0,
                         stream, (TX*)x, (const float*)nullptr, w, (TO*)out, width, eps)));
  TS_CHECK_LAUNCH("rmsnorm");
  return 0;
}

extern "C" int ts_add_rmsnorm(float* resid, const void* delta, int delta_type, const float* w,
                              void* out, int out_type, int rows, int width, float eps,
                              hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0) TS_FAIL("add_rmsnorm: width=%d", width);
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  {
    bool done = false;
    TS_DISPATCH_TYPE(delta_type, TD, TS_DISPATCH_TYPE(out_type, TO,
        done = launch_rmsnorm_vec<TD, TO, true>(resid, (const TD*)delta, w, (TO*)out, rows, width,
                                                eps, stream)));
    if (done) {
      TS_CHECK_LAUNCH("add_rmsnorm");
      return 0;
    }
  }
  TS_DISPATCH_TYPE(delta_type, TD, TS_DISPATCH_TYPE(out_type, TO,
      hipLaunchKernelGGL((rmsnorm_kernel<float, TD, TO, true>), dim3(rows), dim3(threads), 0,
                         stream, resid, (const TD*)delta, w, (TO*)out, width, eps)));
  TS_CHECK_LAUNCH("add_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------- SiLU(gate) * up
// gate_up is [rows, 2*inner]: gate in the first half of a row, up in the second.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t total,
                                int inner) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / inner;
    const int c = (int)(i - r * inner);
    const float g = to_f32(gu[r * 2 * inner + c]);
    const float u = to_f32(gu[r * 2 * inner + inner + c]);
    out[i] = from_f32<T>(g / (1.f + expf(-g)) * u);
  }
}

// Eight bfloat16 per thread (inner a multiple of 8): 16-byte loads and stores.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_rows;
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                       int64_t units, int units_per_row) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < units;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / units_per_row;
    const int c = (int)(i - r * units_per_row) * 8;
    const int inner = units_per_row * 8;
    const bf16x8_rows g = *(const bf16x8_rows*)(gu + r * 2 * inner + c);
    const bf16x8_rows u = *(const bf16x8_rows*)(gu + r * 2 * inner + inner + c);
    bf16x8_rows o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float gf = (float)g[j];
      o[j] = (bf16_t)(gf / (1.f + expf(-gf)) * (float)u[j]);
    }
    *(bf16x8_rows*)(out + r * inner + c) = o;
  }
}

extern "C" int ts_silu_mul(const void* gate_up, void* out, int type, int rows, int inner,
                           hipStream_t stream) {
  if (rows <= 0) return 0;
  if (type == TS_BF16 && inner % 8 == 0 && (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0) {
    const int64_t units = (int64_t)rows * (inner / 8);
    const int blocks = (int)((units + 255) / 256 > 16384 ? 16384 : (units + 255) / 256);
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3(blocks), dim3(256), 0, stream,
                       (const bf16_t*)gate_up, (bf16_t*)out, units, inner / 8);
    TS_CHECK_LAUNCH("silu_mul");
    return 0;
  }
  const int64_t total = (int64_t)rows * inner;
  const int blocks = (int)((total + 255) / 256 > 65535 ? 65535 : (total + 255) / 256);
  TS_DISPATCH_TYPE(type, T,
                   hipLaunchKernelGGL(silu_mul_kernel<T>, dim3(blocks), dim3(256), 0, stream,
                                      (const T*)gate_up, (T*)out, total, inner));
  TS_CHECK_LAUNCH("silu_mul");
  return 0;
}
