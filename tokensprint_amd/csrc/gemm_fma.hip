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

extern "C" int ts_gemm_fma(const void* a, int a_type, const void* w, int w_type, void* c,
                           int c_type, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) TS_FAIL("gemm: K=%d", K);
  dim3 grid((N + kTile - 1) / kTile, (M + kTile - 1) / kTile);
  if (grid.y > 65535) TS_FAIL("gemm: M=%d too large for one launch", M);
  TS_DISPATCH_TYPE(a_type, TA, TS_DISPATCH_TYPE(w_type, TW, TS_DISPATCH_TYPE(c_type, TC,
      hipLaunchKernelGGL((gemm_fma_kernel<TA, TW, TC>), grid, dim3(256), 0, stream,
                         (const TA*)a, (const TW*)w, (TC*)c, M, N, K))));
  TS_CHECK_LAUNCH("gemm_fma");
  return 0;
}
