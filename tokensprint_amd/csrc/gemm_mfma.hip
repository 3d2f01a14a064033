// C[M,N] = A[M,K] * W[N,K]^T for bfloat16 operands on the matrix cores, float32
// accumulation, for the shapes where streaming W once is the whole cost: the entry
// points of the matrix-core products, and the kernels of the wide layout (a short K), in
// which the four waves of a workgroup take different
// tiles of 16 rows of W and nobody splits K.  The layouts that split K among a
// workgroup's waves are gemm_direct.hip's.
//
// Operands go from global memory into the register layout of v_mfma_f32_16x16x32_bf16;
// every lane reads 64 contiguous bytes of its row per iteration, so a row's four lanes
// cover 256 contiguous bytes.  The K index that a register slot stands for is permuted
// the same way for both operands, which a dot product does not notice.  A result never
// depends on timing, and a row of C does not depend on which other rows of A are in the
// call as long as the launch shape is chosen from N and K alone.
#include "gemm_common.h"

// MT: 16-row tiles of A per wave.  WN x WK = 4 waves: WN along N, WK along K.
// PAIR: W holds two stacked matrices [2][N][K]; C = silu(A W0^T) * (A W1^T).
template <int MT, int WN, int WK, typename TC, bool PAIR>
__global__ __launch_bounds__(WN* WK* kWave) void gemm_skinny_kernel(const bf16_t* __restrict__ A,
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

// ---------------------------------------------------------------------------------
// The same product with the rows of A staged in LDS, shared by the workgroup's waves:
// for more than 16 rows of A (they no longer fit the first-level cache when every wave
// reads them from global memory), and for the fused form in which A is not stored at
// all but is the RMSNorm of a residual stream:
//     x = resid_in + sum of delta slabs          (float32; written to resid_out)
//     A = bf16(x * rsqrt(mean(x^2) + eps) * norm_w)
// Waves: WN along N (16 rows of W each) times WK along K.
struct StagedArgs {
  const bf16_t* A;          // [M, K], or null in the fused form
  const bf16_t* W;          // [N, K] (PAIR: [2, N, K])
  void* C;                  // [M, N]
  const float* resid_in;    // fused form: [M, K]
  const void* delta;        // fused form: [slabs, M, K] bfloat16 or float32, or null
  const float* norm_w;      // [K]
  float* resid_out;         // [M, K], written by workgroup column 0
  int M, N, K;
  int delta_slabs, delta_is_f32;
  int kc;                   // K elements staged per round (multiple of WK*128, or >= K)
  int rstd_offset;          // byte offset in LDS of the fused form's row factors
  float eps;
};

template <int MT, int WN, int WK, typename TC, bool PAIR, bool NORM>
__global__ __launch_bounds__(WN* WK* kWave) void gemm_staged_kernel(StagedArgs a) {
  constexpr int NW = PAIR ? 2 : 1;
  constexpr int NWAVES = WN * WK;
  constexpr int ROWS = MT * 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int M = a.M, N = a.N, K = a.K;
  const int xstride = a.kc + 8;                       // bf16 elements; 16 bytes of padding
  bf16_t* xs = (bf16_t*)smem;                         // [ROWS][xstride]
  f32x4* red = (f32x4*)smem;   // reuses the staging area once the K loop is over
  float* rstd_s = (float*)(smem + a.rstd_offset);   // [rows], fused form only
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int wn = wave % WN, wk = wave / WN;
  const int r = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * WN + wn) * 16;
  const int m_base = blockIdx.y * ROWS;
  const int rows = min(ROWS, M - m_base);
  const bool n_ok = n0 + r < N;
  const bf16_t* wrow = a.W + (int64_t)min(n0 + r, N - 1) * K;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // eight consecutive values of the residual stream (resid_in + delta slabs), float32
  auto stream8 = [&](int m, int k, float* v) {
    const float* rp = a.resid_in + (int64_t)(m_base + m) * K + k;
    const f32x4 r0 = *(const f32x4*)rp, r1 = *(const f32x4*)(rp + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[j] = r0[j]; v[4 + j] = r1[j]; }
    for (int sl = 0; sl < a.delta_slabs; ++sl) {
      const int64_t i = ((int64_t)sl * M + m_base + m) * K + k;
      if (a.delta_is_f32) {
        const float* dp = (const float*)a.delta + i;
        const f32x4 d0 = *(const f32x4*)dp, d1 = *(const f32x4*)(dp + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[j] += d0[j]; v[4 + j] += d1[j]; }
      } else {
        const bf16x8 d = *(const bf16x8*)((const bf16_t*)a.delta + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] += (float)d[j];
      }
    }
  };

  if (NORM) {
    // One pass: each wave takes rows m = wave, wave + NWAVES, ...; it writes the new
    // residual stream (workgroup column 0 only), stages x * norm_w (not yet divided by
    // the row's root mean square) and sums the squares.  The division commutes with the
    // product, so it is applied to the accumulators at the end; nothing waits for the
    // row sums.  The fused form stages all of K at once (kc >= K).
    for (int m = wave; m < rows; m += NWAVES) {
      float ss = 0.f;
      for (int u = lane; u < K / 8; u += kWave) {
        float v[8];
        stream8(m, u * 8, v);
        if (blockIdx.x == 0) {
          float* op = a.resid_out + (int64_t)(m_base + m) * K + u * 8;
          *(f32x4*)op = f32x4{v[0], v[1], v[2], v[3]};
          *(f32x4*)(op + 4) = f32x4{v[4], v[5], v[6], v[7]};
        }
        const f32x4 w0 = *(const f32x4*)(a.norm_w + u * 8), w1 = *(const f32x4*)(a.norm_w + u * 8 + 4);
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ss += v[j] * v[j] + v[4 + j] * v[4 + j];
          o[j] = (bf16_t)(v[j] * w0[j]);
          o[4 + j] = (bf16_t)(v[4 + j] * w1[j]);
        }
        *(bf16x8*)(xs + (size_t)m * xstride + u * 8) = o;
      }
      ss = wave_sum(ss);
      if (lane == 0) rstd_s[m] = rsqrtf(ss / (float)K + a.eps);
    }
  }

  f32x4 acc[NW][MT];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[w][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kc0 = 0; kc0 < K; kc0 += a.kc) {
    const int kc_len = min(a.kc, K - kc0);
    const int units = kc_len / 8;                      // 16-byte units per row
    // weights of this wave's first iteration, asked for before the rows of A are staged
    bf16x8 wv[NW][4];
    auto load_w = [&](int kb) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int k = kb + g * 32 + s * 8;
        const bool ok = n_ok && k < kc0 + kc_len;
#pragma unroll
        for (int w = 0; w < NW; ++w)
          wv[w][s] = ok ? *(const bf16x8*)(wrow + (int64_t)w * N * K + k) : zero;
      }
    };
    load_w(kc0 + wk * kIterK);
    if (!NORM) {
      for (int idx = tid; idx < ROWS * units; idx += NWAVES * kWave) {
        const int m = idx / units, k = kc0 + (idx % units) * 8;
        const bf16x8 v = m < rows ? *(const bf16x8*)(a.A + (int64_t)(m_base + m) * K + k) : zero;
        *(bf16x8*)(xs + (size_t)m * xstride + (k - kc0)) = v;
      }
    }
    __syncthreads();
    if (n0 < N) {
      for (int kb = kc0 + wk * kIterK; kb < kc0 + kc_len; kb += WK * kIterK) {
        bf16x8 cur[NW][4];
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
          for (int s = 0; s < 4; ++s) cur[w][s] = wv[w][s];
        if (kb + WK * kIterK < kc0 + kc_len) load_w(kb + WK * kIterK);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const int k = kb + g * 32 + s * 8;
            // the fused form stages only the rows there are; the rest read as zero
            const bf16x8 xv = (k < kc0 + kc_len && (!NORM || mt * 16 + r < rows))
                ? *(const bf16x8*)(xs + (size_t)(mt * 16 + r) * xstride + (k - kc0)) : zero;
#pragma unroll
            for (int w = 0; w < NW; ++w)
              acc[w][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[w][s], xv, acc[w][mt],
                                                                   0, 0, 0);
          }
        }
      }
    }
    __syncthreads();
  }

  if (WK > 1) {
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
  const int n = n0 + g * 4;
  if (n >= N) return;
  TC* C = (TC*)a.C;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m_base + mt * 16 + r;
    if (m >= M) continue;
    const float rs = NORM ? rstd_s[mt * 16 + r] : 1.f;
    f32x4 v = acc[0][mt];
#pragma unroll
    for (int t = 0; t < 4; ++t) v[t] *= rs;
    if (PAIR) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const float gt = (float)(bf16_t)v[t], up = (float)(bf16_t)(acc[1][mt][t] * rs);
        v[t] = gt / (1.f + expf(-gt)) * up;
      }
    }
    store4<TC>(C + (int64_t)m * N + n, v, N - n);
  }
}

template <int MT, int WN, int WK, typename TC, bool PAIR, bool NORM>
static int launch_staged(StagedArgs a, hipStream_t stream) {
  constexpr int NW = PAIR ? 2 : 1;
  constexpr int ROWS = MT * 16;
  const int round = WK * kIterK;
  // rows of A staged per round: as much of K as 64 KB of LDS hold; the fused form
  // stages all of K for the rows there are
  int kc = ((64 * 1024 / (ROWS * 2) - 8) / round) * round;
  if (kc < round) kc = round;
  if (NORM || kc >= a.K) kc = ((a.K + 7) / 8) * 8;
  a.kc = kc;
  const int staged_rows = NORM ? a.M : ROWS;
  const size_t lds_x = (size_t)staged_rows * (kc + 8) * 2;
  const size_t lds_red = (size_t)(WK - 1) * WN * NW * MT * kWave * 16;
  size_t lds = lds_x > lds_red ? lds_x : lds_red;
  lds = (lds + 15) / 16 * 16;
  a.rstd_offset = (int)lds;
  if (NORM) lds += 64;      // up to 16 row factors
  if (lds > 150 * 1024) TS_FAIL("gemm_staged: %zu bytes of LDS needed", lds);
  auto kernel = gemm_staged_kernel<MT, WN, WK, TC, PAIR, NORM>;
  static bool raised = false;   // per instantiation
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess)
      TS_FAIL("gemm_staged: cannot raise the LDS limit");
    raised = true;
  }
  dim3 grid((a.N + WN * 16 - 1) / (WN * 16), (a.M + ROWS - 1) / ROWS);
  hipLaunchKernelGGL(kernel, grid, dim3(WN * WK * kWave), lds, stream, a);
  return 0;
}

// Only the wide layout (4 waves along N) is served here; the layouts that split K among
// the waves of a workgroup are gemm_direct.hip's.
template <typename TC, bool PAIR, bool NORM>
static int dispatch_staged(const StagedArgs& a, hipStream_t stream) {
  if (NORM || a.M <= 16) return launch_staged<1, 4, 1, TC, PAIR, NORM>(a, stream);
  if (a.M <= 32) return launch_staged<2, 4, 1, TC, PAIR, false>(a, stream);
  return launch_staged<4, 4, 1, TC, PAIR, false>(a, stream);
}

template <int MT, int WN, int WK, typename TC, bool PAIR>
static void launch_skinny(const bf16_t* A, const bf16_t* W, TC* C, int M, int N, int K,
                          hipStream_t stream) {
  dim3 grid((N + WN * 16 - 1) / (WN * 16), (M + MT * 16 - 1) / (MT * 16));
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, WN, WK, TC, PAIR>), grid, dim3(WN * WK * kWave), 0,
                     stream, A, W, C, M, N, K);
}

template <typename TC, bool PAIR>
static int dispatch_skinny(const void* a, const void* w, void* c, int M, int N, int K,
                           hipStream_t stream) {
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  if (M <= 16) {   // few rows: both operands straight from global memory
    launch_skinny<1, 4, 1, TC, PAIR>(A, W, (TC*)c, M, N, K, stream);
    return 0;
  }
  StagedArgs sa = {};
  sa.A = A; sa.W = W; sa.C = c; sa.M = M; sa.N = N; sa.K = K;
  return dispatch_staged<TC, PAIR, false>(sa, stream);
}

// pair = 1: W is [2, N, K] (gate rows then up rows) and C[M, N] = silu(A Wg^T) * (A Wu^T).
extern "C" int ts_gemm_mfma_bf16(const void* a, const void* w, void* c, int c_type, int M,
                                 int N, int K, int pair, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8) TS_FAIL("gemm_mfma: K=%d must be a positive multiple of 8", K);
  if (((uintptr_t)a | (uintptr_t)w) & 15) TS_FAIL("gemm_mfma: operands must be 16-byte aligned");
  if ((M + 63) / 64 > 65535) TS_FAIL("gemm_mfma: M=%d too large", M);
  int rc;
  if (!layout_wide(N, K)) {
    DirectArgs da = {};
    da.A = (const bf16_t*)a; da.W = (const bf16_t*)w; da.C = c; da.M = M; da.N = N; da.K = K;
    rc = gemm_direct_launch(da, c_type, pair != 0, false, stream);
  } else if (pair) {
    if (c_type != TS_BF16) TS_FAIL("gemm_mfma: the paired product writes bfloat16");
    rc = dispatch_skinny<bf16_t, true>(a, w, c, M, N, K, stream);
  } else if (c_type == TS_F32) {
    rc = dispatch_skinny<float, false>(a, w, c, M, N, K, stream);
  } else if (c_type == TS_BF16) {
    rc = dispatch_skinny<bf16_t, false>(a, w, c, M, N, K, stream);
  } else {
    TS_FAIL("gemm_mfma: unknown output type %d", c_type);
  }
  if (rc) return rc;
  TS_CHECK_LAUNCH("gemm_mfma");
  return 0;
}

// Whether the fused form below takes a product of this shape: at most 16 rows; in the
// wide layout rows short enough for its staging buffer; in the others at most 16384
// elements of the residual stream (16 rows of 1024, 4 of 4096) and a weight of at most
// 2^24 elements, because every workgroup reads the stream in float32: with a long K or
// very many workgroups (the output head) that costs more than the norm kernel saved.
extern "C" int ts_norm_gemm_mfma_fits(int M, int N, int K) {
  if (M < 1 || M > 16 || K <= 0 || K % 8) return 0;
  if (layout_wide(N, K)) return (size_t)M * (K + 8) * 2 <= 140 * 1024;
  return (int64_t)M * K <= 16384 && (int64_t)N * K <= (1 << 24);
}

// 0: 4 waves split K, 1: 8 waves split K, 2: wide (4 waves along N).
extern "C" int ts_gemm_mfma_layout(int N, int K) {
  return layout_wide(N, K) ? 2 : layout_deep(N, K) ? 1 : 0;
}

// Fused form for at most 16 rows: C = RMSNorm(resid_in + sum of delta slabs) W^T, and
// resid_out = resid_in + sum of delta slabs.  delta may be null (slabs = 0).
extern "C" int ts_norm_gemm_mfma_bf16(const float* resid_in, const void* delta, int delta_type,
                                      int delta_slabs, const float* norm_w, float eps,
                                      float* resid_out, const void* w, void* c, int c_type,
                                      int M, int N, int K, int pair, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8) TS_FAIL("norm_gemm_mfma: K=%d must be a positive multiple of 8", K);
  if (!ts_norm_gemm_mfma_fits(M, N, K))
    TS_FAIL("norm_gemm_mfma: %d rows of K=%d are more than the fused form takes", M, K);
  if (((uintptr_t)w) & 15) TS_FAIL("norm_gemm_mfma: weights must be 16-byte aligned");
  if (!resid_in || !resid_out || resid_in == resid_out)
    TS_FAIL("norm_gemm_mfma: resid_in and resid_out must be two buffers");
  if (delta_slabs < 0 || (delta_slabs > 0 && !delta)) TS_FAIL("norm_gemm_mfma: delta slabs");
  if (!layout_wide(N, K)) {
    if (delta && (delta_slabs != 1 || delta_type != TS_BF16))
      TS_FAIL("norm_gemm_mfma: this layout takes one bfloat16 delta");
    DirectArgs da = {};
    da.W = (const bf16_t*)w; da.C = c; da.M = M; da.N = N; da.K = K;
    da.resid_in = resid_in; da.delta = (const bf16_t*)delta; da.norm_w = norm_w;
    da.resid_out = resid_out; da.eps = eps;
    if (gemm_direct_launch(da, c_type, pair != 0, true, stream)) return -1;
    TS_CHECK_LAUNCH("norm_gemm_mfma");
    return 0;
  }
  StagedArgs sa = {};
  sa.W = (const bf16_t*)w; sa.C = c; sa.M = M; sa.N = N; sa.K = K;
  sa.resid_in = resid_in; sa.delta = delta; sa.norm_w = norm_w; sa.resid_out = resid_out;
  sa.delta_slabs = delta ? delta_slabs : 0; sa.delta_is_f32 = delta_type == TS_F32;
  sa.eps = eps;
  int rc;
  if (pair) {
    if (c_type != TS_BF16) TS_FAIL("norm_gemm_mfma: the paired product writes bfloat16");
    rc = dispatch_staged<bf16_t, true, true>(sa, stream);
  } else if (c_type == TS_F32) {
    rc = dispatch_staged<float, false, true>(sa, stream);
  } else if (c_type == TS_BF16) {
    rc = dispatch_staged<bf16_t, false, true>(sa, stream);
  } else {
    TS_FAIL("norm_gemm_mfma: unknown output type %d", c_type);
  }
  if (rc) return rc;
  TS_CHECK_LAUNCH("norm_gemm_mfma");
  return 0;
}

// The norm split over two products, for up to 64 rows (see gemm_direct.hip).
//
// ts_gemm_tail_bf16: resid[M, N] += bf16(A[M, K] W[N, K]^T) in place (float32), and for
// the RMSNorm with weight norm_w that follows: prepared[M, N] = bf16(resid * norm_w) and
// sumsq[M][ts_gemm_tail_parts(M, N) rounded up to 4], each row's sum of squares of resid
// over a slice of its columns (16, or fewer where the product is spread over more
// workgroups); what lies beyond a row's slices is not written.
extern "C" int ts_gemm_tail_fits(int M, int N, int K) { return gemm_direct_tail_fits(M, N, K); }
extern "C" int ts_gemm_tail_parts(int M, int N) { return gemm_direct_tail_parts(M, N); }

extern "C" int ts_gemm_tail_bf16(const void* a, const void* w, float* resid, const float* norm_w,
                                 void* prepared, float* sumsq, int M, int N, int K,
                                 hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!gemm_direct_tail_fits(M, N, K))
    TS_FAIL("gemm_tail: M=%d, N=%d, K=%d is not a product the tail form takes", M, N, K);
  if (((uintptr_t)a | (uintptr_t)w | (uintptr_t)resid | (uintptr_t)norm_w) & 15)
    TS_FAIL("gemm_tail: operands must be 16-byte aligned");
  if (((uintptr_t)prepared) & 7) TS_FAIL("gemm_tail: the prepared rows must be 8-byte aligned");
  if (!a || !w || !resid || !norm_w || !prepared || !sumsq) TS_FAIL("gemm_tail: null operand");
  DirectArgs da = {};
  da.A = (const bf16_t*)a; da.W = (const bf16_t*)w; da.M = M; da.N = N; da.K = K;
  da.resid = resid; da.tail_w = norm_w; da.prepared = (bf16_t*)prepared; da.sumsq_out = sumsq;
  if (gemm_direct_launch(da, TS_BF16, false, false, stream)) return -1;
  TS_CHECK_LAUNCH("gemm_tail");
  return 0;
}

// ts_gemm_scaled_bf16: C[M, N] = (prepared[M, K] W[N, K]^T) * rsqrt(sum_j sumsq[m][j] / K + eps)
// for sumsq[M][parts rounded up to 4] (16-byte aligned); pair as in ts_gemm_mfma_bf16.
extern "C" int ts_gemm_scaled_fits(int M, int N, int K, int pair, int parts) {
  return gemm_direct_scaled_fits(M, N, K, pair != 0, parts);
}

extern "C" int ts_gemm_scaled_bf16(const void* prepared, const float* sumsq, int parts, float eps,
                                   const void* w, void* c, int c_type, int M, int N, int K,
                                   int pair, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!gemm_direct_scaled_fits(M, N, K, pair != 0, parts))
    TS_FAIL("gemm_scaled: M=%d, N=%d, K=%d is not a product the scaled form takes", M, N, K);
  if (((uintptr_t)prepared | (uintptr_t)w | (uintptr_t)sumsq) & 15)
    TS_FAIL("gemm_scaled: operands must be 16-byte aligned");
  if (!prepared || !sumsq || !w || !c) TS_FAIL("gemm_scaled: null operand");
  DirectArgs da = {};
  da.A = (const bf16_t*)prepared; da.W = (const bf16_t*)w; da.C = c; da.M = M; da.N = N; da.K = K;
  da.sumsq = sumsq; da.parts = parts; da.eps = eps;
  if (gemm_direct_launch(da, c_type, pair != 0, false, stream)) return -1;
  TS_CHECK_LAUNCH("gemm_scaled");
  return 0;
}
