// C[M,N] = A[M,K] * W[N,K]^T with float32 fused multiply-adds only: no matrix-core
// instruction and no reduced-precision mode, whatever the operand types.  This is the
// product of the float32 path and of any bfloat16 run whose weights are held in 32-bit.
// Every output element adds its K products in an order fixed by K alone (per lane in
// index order and then across the lanes of a wavefront; in index order with one
// accumulator in the tiled kernel, which serves a K that is no multiple of 4), so its value
// does not depend on which other rows are in the call.
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

// The kernel for every K that is a multiple of 4: a wavefront per four output columns and
// up to 16 rows of A, so that a row of W is read by 64 lanes side by side (a kilobyte a load
// instruction) and a decode step's columns spread over the chip.  Lane l takes elements
// 4 l .. 4 l + 3 of every stretch of 256 of K, adds its products in index order, and the 64
// lanes' sums are added in a fixed butterfly: the order depends on K alone, never on M or
// on which other rows are in the call, so a row's result is the same to the bit however
// the rows are batched (more than 16 rows are further workgroups along y).  The rows of A
// are the same for every wavefront and come out of the caches.
typedef __attribute__((ext_vector_type(4))) float f32x4_fma;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_fma;
__device__ __forceinline__ f32x4_fma load4_fma(const float* p) { return *(const f32x4_fma*)p; }
__device__ __forceinline__ f32x4_fma load4_fma(const bf16_t* p) {
  const bf16x4_fma v = *(const bf16x4_fma*)p;
  return f32x4_fma{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

constexpr int kColumnsPerWave = 4;

template <typename TA, typename TW, typename TC, int MR>
__global__ __launch_bounds__(256) void gemm_fma_rows_kernel(const TA* __restrict__ A,
                                                            const TW* __restrict__ W,
                                                            TC* __restrict__ C, int M, int N, int K) {
  constexpr int CPW = kColumnsPerWave;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t n0 = ((int64_t)blockIdx.x * 4 + wave) * CPW;
  if (n0 >= N) return;
  const int m0 = blockIdx.y * MR;
  A += (int64_t)m0 * K;
  C += (int64_t)m0 * N;
  M -= m0;
  float acc[MR][CPW];
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int c = 0; c < CPW; ++c) acc[m][c] = 0.f;
  // Few rows (a decode step): the rows of W are read once and come from memory; four
  // stretches of them are asked for before the first is used, and each again four ahead, so
  // that a compute unit's few waves keep enough bytes on the way (a decode step's product
  // has one workgroup a unit; stretch after stretch it ran at a tenth of the memory's
  // rate).  The rows of A, the same for every wave, come out of the caches one stretch
  // ahead.  The sums' order is that of the plain loop.
  if constexpr (MR > 8) {
    // many rows (a prompt's portion, workgroups enough to hide the waits): stretch after
    // stretch, a row at a time, so that the sums and not the rows hold the registers
    for (int k = lane * 4; k < K; k += kWave * 4) {
      f32x4_fma w[CPW];
#pragma unroll
      for (int c = 0; c < CPW; ++c) w[c] = load4_fma(W + min(n0 + c, (int64_t)N - 1) * K + k);
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const f32x4_fma a = load4_fma(A + (int64_t)min(m, M - 1) * K + k);
#pragma unroll
        for (int c = 0; c < CPW; ++c)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[m][c] = fmaf(a[e], w[c][e], acc[m][c]);
      }
    }
  } else {
    constexpr int kAhead = 4;
    const int stretches = (K - lane * 4 + kWave * 4 - 1) / (kWave * 4);     // of this lane
    // (a lane without a stretch i reads the row's last four elements and drops them)
    auto w_at = [&](int i, int c) {
      return load4_fma(W + min(n0 + c, (int64_t)N - 1) * K + min(lane * 4 + i * kWave * 4, K - 4));
    };
    auto a_at = [&](int i, int m) {
      return load4_fma(A + (int64_t)min(m, M - 1) * K + min(lane * 4 + i * kWave * 4, K - 4));
    };
    f32x4_fma w[kAhead][CPW], a_next[MR];
#pragma unroll
    for (int p = 0; p < kAhead; ++p)
#pragma unroll
      for (int c = 0; c < CPW; ++c) w[p][c] = w_at(p, c);
#pragma unroll
    for (int m = 0; m < MR; ++m) a_next[m] = a_at(0, m);
    for (int i0 = 0; i0 < stretches; i0 += kAhead) {
#pragma unroll
      for (int p = 0; p < kAhead; ++p) {
        const int i = i0 + p;
        if (i >= stretches) break;
        f32x4_fma a[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) a[m] = a_next[m];
        if (i + 1 < stretches) {
#pragma unroll
          for (int m = 0; m < MR; ++m) a_next[m] = a_at(i + 1, m);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
          for (int c = 0; c < CPW; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[m][c] = fmaf(a[m][e], w[p][c][e], acc[m][c]);
        if (i + kAhead < stretches) {
#pragma unroll
          for (int c = 0; c < CPW; ++c) w[p][c] = w_at(i + kAhead, c);
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      float v = acc[m][c];
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
      if (lane == 0 && m < M && n0 + c < N) C[(int64_t)m * N + n0 + c] = from_f32<TC>(v);
    }
}

template <typename TA, typename TW, typename TC>
static void launch_rows(const TA* A, const TW* W, TC* C, int M, int N, int K, hipStream_t stream) {
  const int columns = (N + 4 * kColumnsPerWave - 1) / (4 * kColumnsPerWave);
  const dim3 grid(columns, M <= 16 ? 1 : (M + 15) / 16);
  if (M == 1)
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 1>), grid, dim3(256), 0, stream, A, W, C, M, N, K);
  else if (M <= 4)
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 4>), grid, dim3(256), 0, stream, A, W, C, M, N, K);
  else if (M <= 8)
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 8>), grid, dim3(256), 0, stream, A, W, C, M, N, K);
  else
    hipLaunchKernelGGL((gemm_fma_rows_kernel<TA, TW, TC, 16>), grid, dim3(256), 0, stream, A, W, C, M, N, K);
}

extern "C" int ts_gemm_fma(const void* a, int a_type, const void* w, int w_type, void* c,
                           int c_type, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) TS_FAIL("gemm: K=%d", K);
  // rows of 4 elements must start on 16 (float32) or 8 (bfloat16) bytes for the row kernel
  // (a property of K and of the buffers, not of M: which kernel serves a weight never
  // depends on the number of rows)
  const bool rows_ok = K % 4 == 0 && (((uintptr_t)a | (uintptr_t)w) & 15) == 0 && (M + 15) / 16 <= 65535;
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
