// C[M,N] = A[M,K] * W[N,K]^T for bfloat16 operands on the matrix cores, float32
// accumulation, for the shapes where streaming W once is the whole cost: M from 1 to a
// few hundred (decode batches, short portions of prompts, the output head).
//
// A wavefront owns a tile of 16 rows of W and up to 64 rows of A.  Both operands go from
// global memory straight into the register layout of v_mfma_f32_16x16x32_bf16; every
// lane reads 64 contiguous bytes of its row per iteration, so a row's four lanes cover
// 256 contiguous bytes.  The K index that a register slot stands for is permuted the
// same way for both operands, which a dot product does not notice.  Waves of a
// workgroup either take different row tiles (large N) or split K and add their partial
// sums in LDS in a fixed order (small N), so a result never depends on timing, and a
// row of C does not depend on which other rows of A are in the call as long as the
// launch shape is chosen from N and K alone.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kIterK = 128;   // K elements a wave consumes per iteration (4 MFMA steps)

template <typename TC> __device__ __forceinline__ void store4(TC* p, f32x4 v, int n_left);
template <> __device__ __forceinline__ void store4<float>(float* p, f32x4 v, int n_left) {
  if (n_left >= 4 && ((uintptr_t)p & 15) == 0) { *(f32x4*)p = v; return; }
  for (int t = 0; t < 4 && t < n_left; ++t) p[t] = v[t];
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4 v, int n_left) {
  if (n_left >= 4 && ((uintptr_t)p & 7) == 0) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
    return;
  }
  for (int t = 0; t < 4 && t < n_left; ++t) p[t] = (bf16_t)v[t];
}

// MT: 16-row tiles of A per wave.  WN x WK = 4 waves: WN along N, WK along K.
// PAIR: W holds two stacked matrices [2][N][K]; C = silu(A W0^T) * (A W1^T).
template <int MT, int WN, int WK, typename TC, bool PAIR>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16_t* __restrict__ A,
                                                          const bf16_t* __restrict__ W,
                                                          TC* __restrict__ C, int M, int N,
                                                          int K) {
  constexpr int NW = PAIR ? 2 : 1;
  __shared__ f32x4 red[WK > 1 ? (WK - 1) * WN * NW * MT * kWave : 1];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int wn = wave % WN, wk = wave / WN;
  const int r = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * WN + wn) * 16;
  const int m_base = blockIdx.y * (MT * 16);
  const bool n_ok = n0 + r < N;
  const bf16_t* wrow = W + (int64_t)min(n0 + r, N - 1) * K;
  const bf16_t* arow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m_base + mt * 16 + r;
    m_ok[mt] = m < M;
    arow[mt] = A + (int64_t)min(m, M - 1) * K;
  }
  f32x4 acc[NW][MT];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[w][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  if (n0 < N) {   // a wave whose tile lies beyond N only takes part in the barrier below
#pragma unroll 2
    for (int kb = wk * kIterK; kb < K; kb += WK * kIterK) {
      bf16x8 wv[NW][4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int k = kb + g * 32 + s * 8;
        const bool ok = n_ok && k < K;
#pragma unroll
        for (int w = 0; w < NW; ++w)
          wv[w][s] = ok ? *(const bf16x8*)(wrow + (int64_t)w * N * K + k) : zero;
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        bf16x8 xv[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int k = kb + g * 32 + s * 8;
          xv[s] = (m_ok[mt] && k < K) ? *(const bf16x8*)(arow[mt] + k) : zero;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int w = 0; w < NW; ++w)
            acc[w][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[w][s], xv[s], acc[w][mt],
                                                                 0, 0, 0);
      }
    }
  }

  if (WK > 1) {   // partial sums of the K splits, added in split order
    if (wk > 0) {
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          red[((((wk - 1) * WN + wn) * NW + w) * MT + mt) * kWave + lane] = acc[w][mt];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int k2 = 1; k2 < WK; ++k2)
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[w][mt] += red[((((k2 - 1) * WN + wn) * NW + w) * MT + mt) * kWave + lane];
  }
  if (n0 >= N) return;

  // lane holds D[n = n0 + g*4 + t][m = tile*16 + r], t = 0..3
  const int n = n0 + g * 4;
  if (n >= N) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m_base + mt * 16 + r;
    if (m >= M) continue;
    f32x4 v = acc[0][mt];
    if (PAIR) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // the two products are rounded to the activation type first, as the unfused
        // path stores them, then silu(gate) * up in float32
        const float gt = (float)(bf16_t)acc[0][mt][t], up = (float)(bf16_t)acc[1][mt][t];
        v[t] = gt / (1.f + expf(-gt)) * up;
      }
    }
    store4<TC>(C + (int64_t)m * N + n, v, N - n);
  }
}

template <int MT, typename TC, bool PAIR>
static void launch_skinny(const bf16_t* A, const bf16_t* W, TC* C, int M, int N, int K,
                          bool split_k, hipStream_t stream) {
  const int m_tiles = (M + MT * 16 - 1) / (MT * 16);
  if (split_k) {
    dim3 grid((N + 15) / 16, m_tiles);
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, 1, 4, TC, PAIR>), grid, dim3(256), 0, stream, A,
                       W, C, M, N, K);
  } else {
    dim3 grid((N + 63) / 64, m_tiles);
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, 4, 1, TC, PAIR>), grid, dim3(256), 0, stream, A,
                       W, C, M, N, K);
  }
}

template <typename TC, bool PAIR>
static int dispatch_skinny(const void* a, const void* w, void* c, int M, int N, int K,
                           hipStream_t stream) {
  // the launch shape follows N and K only, never M, so that a row of C is computed the
  // same way whatever else is in the batch
  const bool split_k = N < 16384 && K >= 512;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  TC* C = (TC*)c;
  if (M <= 16) launch_skinny<1, TC, PAIR>(A, W, C, M, N, K, split_k, stream);
  else if (M <= 32) launch_skinny<2, TC, PAIR>(A, W, C, M, N, K, split_k, stream);
  else launch_skinny<4, TC, PAIR>(A, W, C, M, N, K, split_k, stream);
  return 0;
}

// pair = 1: W is [2, N, K] (gate rows then up rows) and C[M, N] = silu(A Wg^T) * (A Wu^T).
extern "C" int ts_gemm_mfma_bf16(const void* a, const void* w, void* c, int c_type, int M,
                                 int N, int K, int pair, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8) TS_FAIL("gemm_mfma: K=%d must be a positive multiple of 8", K);
  if (((uintptr_t)a | (uintptr_t)w) & 15) TS_FAIL("gemm_mfma: operands must be 16-byte aligned");
  if ((M + 63) / 64 > 65535) TS_FAIL("gemm_mfma: M=%d too large", M);
  if (pair) {
    if (c_type != TS_BF16) TS_FAIL("gemm_mfma: the paired product writes bfloat16");
    dispatch_skinny<bf16_t, true>(a, w, c, M, N, K, stream);
  } else if (c_type == TS_F32) {
    dispatch_skinny<float, false>(a, w, c, M, N, K, stream);
  } else if (c_type == TS_BF16) {
    dispatch_skinny<bf16_t, false>(a, w, c, M, N, K, stream);
  } else {
    TS_FAIL("gemm_mfma: unknown output type %d", c_type);
  }
  TS_CHECK_LAUNCH("gemm_mfma");
  return 0;
}
