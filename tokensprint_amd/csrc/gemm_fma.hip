// C[M,N] = A[M,K] * W[N,K]^T with float32 fused multiply-adds only: no matrix-core
// instruction and no reduced-precision mode, whatever the operand types.  This is the
// product of the float32 path and of any bfloat16 run whose weights are held in 32-bit.
// Every output element adds its K products in index order with one accumulator, so its
// value does not depend on M or on which other rows are in the call.
#include "common.h"

constexpr int kTile = 64;   // output tile edge per workgroup
constexpr int kStep = 16;   // K elements staged per iteration

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_fma_kernel(const TA* __restrict__ A,
                                                       const TW* __restrict__ W,
                                                       TC* __restrict__ C, int M, int N, int K) {
  __shared__ float As[kStep][kTile + 4];
  __shared__ float Ws[kStep][kTile + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int64_t m0 = (int64_t)blockIdx.y * kTile, n0 = (int64_t)blockIdx.x * kTile;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += kStep) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int idx = tid + r * 256;
      const int row = idx / kStep, k = idx % kStep;
      const bool kin = k0 + k < K;
      As[k][row] = (kin && m0 + row < M) ? to_f32(A[(m0 + row) * K + k0 + k]) : 0.f;
      Ws[k][row] = (kin && n0 + row < N) ? to_f32(W[(n0 + row) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStep; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t n = n0 + tx * 4 + j;
      if (n < N) C[m * N + n] = from_f32<TC>(acc[i][j]);
    }
  }
}

// Up to 16 rows of A (decode steps): a thread per output column and one workgroup of 64
// threads per 64 columns, so the columns spread over the chip.  A thread walks its row of
// W in 16-byte pieces (the lines it touches stay in the first-level cache until it has
// used them up), the rows of A come through scalar loads, the same for every thread.
// The products of an output element are added in index order, as in the tiled kernel.
typedef __attribute__((ext_vector_type(4))) float f32x4_fma;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_fma;
__device__ __forceinline__ f32x4_fma load4_fma(const float* p) { return *(const f32x4_fma*)p; }
__device__ __forceinline__ f32x4_fma load4_fma(const bf16_t* p) {
  const bf16x4_fma v = *(const bf16x4_fma*)p;
  return f32x4_fma{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

template <typename TA, typename TW, typename TC, int MR>
__global__ __launch_bounds__(64) void gemm_fma_rows_kernel(const TA* __restrict__ A,
                                                           const TW* __restrict__ W,
                                                           TC* __restrict__ C, int M, int N, int K) {
  const int64_t n = (int64_t)blockIdx.x * 64 + threadIdx.x;
  const TW* wrow = W + min(n, (int64_t)N - 1) * K;
  float acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0.f;
  const int k4 = K / 4 * 4;
  int k = 0;
  for (; k < k4; k += 4) {
    const f32x4_fma w = load4_fma(wrow + k);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const f32x4_fma a = load4_fma(A + (int64_t)min(m, M - 1) * K + k);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[m] = fmaf(a[e], w[e], acc[m]);
    }
  }
  for (; k < K; ++k) {
    const float w = to_f32(wrow[k]);
#pragma unroll
    for (int m = 0; m < MR; ++m)
      acc[m] = fmaf(to_f32(A[(int64_t)min(m, M - 1) * K + k]), w, acc[m]);
  }
  if (n >= N) return;
#pragma unroll
  for (int m = 0; m < MR; ++m)
    if (m < M) C[(int64_t)m * N + n] = from_f32<TC>(acc[m]);
}

template <typename TA, typename TW, typename TC>
static void launch_rows(const TA* A, const TW* W, TC* C, int M, int N, int K, hipStream_t stream) {
  const dim3 grid((N + 63) / 64);
  if (M == 1)
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 1>), grid, dim3(64), 0, stream, A, W, C, M, N, K);
  else if (M <= 4)
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 4>), grid, dim3(64), 0, stream, A, W, C, M, N, K);
  else
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 16>), grid, dim3(64), 0, stream, A, W, C, M, N, K);
}

extern "C" int ts_gemm_fma(const void* a, int a_type, const void* w, int w_type, void* c,
                           int c_type, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) TS_FAIL("gemm: K=%d", K);
  // rows of 4 elements must start on 16 (float32) or 8 (bfloat16) bytes for the row kernel
  const bool rows_ok = M <= 16 && K % 4 == 0 && (((uintptr_t)a | (uintptr_t)w) & 15) == 0;
  if (rows_ok) {
    TS_DISPATCH_TYPE(a_type, TA, TS_DISPATCH_TYPE(w_type, TW, TS_DISPATCH_TYPE(c_type, TC,
        launch_rows<TA, TW, TC>((const TA*)a, (const TW*)w, (TC*)c, M, N, K, stream))));
    TS_CHECK_LAUNCH("gemm_fma");
    return 0;
  }
  dim3 grid((N + kTile - 1) / kTile, (M + kTile - 1) / kTile);
  if (grid.y > 65535) TS_FAIL("gemm: M=%d too large for one launch", M);
  TS_DISPATCH_TYPE(a_type, TA, TS_DISPATCH_TYPE(w_type, TW, TS_DISPATCH_TYPE(c_type, TC,
      hipLaunchKernelGGL((gemm_fma_kernel<TA, TW, TC>), grid, dim3(256), 0, stream,
                         (const TA*)a, (const TW*)w, (TC*)c, M, N, K))));
  TS_CHECK_LAUNCH("gemm_fma");
  return 0;
}
