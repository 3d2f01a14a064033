// Entry points of the LDS-tiled product for many rows (gemm_tiled_kernel.h) in the forms
// that carry a prompt's residual add and RMSNorm: the product that ends a sub-layer adds
// itself into the float32 stream and hands the stream on prepared for the norm, and the
// product behind that norm divides by the rows' root mean square in its epilogue.
#include "gemm_tiled_kernel.h"

extern "C" int ts_gemm_tiled_fits(int M, int N, int K, int pair);

// Slices of a row's sum of squares that ts_gemm_tiled_tail_bf16 writes for N columns.
extern "C" int ts_gemm_tiled_tail_parts(int N) { return N / kSliceColumns; }

// 1 if ts_gemm_tiled_tail_bf16 takes these sizes.
extern "C" int ts_gemm_tiled_tail_fits(int M, int N, int K) {
  return ts_gemm_tiled_fits(M, N, K, 0) && N % kSliceColumns == 0 &&
         (int64_t)M * N * 4 < (1ll << 40);
}

// resid[M, N] += bfloat16(A[M, K] W[N, K]^T) in place (float32); prepared[M, N] =
// bfloat16(resid * norm_w); sumsq[N / 32, M] = the new rows' sums of squares in slices of
// 32 columns.  `tile` as in ts_gemm_tiled_bf16.
extern "C" int ts_gemm_tiled_tail_bf16(const void* a, const void* w, float* resid,
                                       const float* norm_w, void* prepared, float* sumsq, int M,
                                       int N, int K, int tile, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ts_gemm_tiled_tail_fits(M, N, K))
    TS_FAIL("gemm_tiled_tail: M=%d N=%d K=%d not taken (K a multiple of 64 from 256, N of 32)",
            M, N, K);
  if (((uintptr_t)a | (uintptr_t)w | (uintptr_t)resid | (uintptr_t)norm_w | (uintptr_t)prepared) & 15)
    TS_FAIL("gemm_tiled_tail: operands must be 16-byte aligned");
  TiledArgs g{(const bf16_t*)a, (const bf16_t*)w, nullptr, M, N, K, 0, 0, 1};
  g.resid = resid;
  g.norm_w = norm_w;
  g.prepared = (bf16_t*)prepared;
  g.sumsq_out = sumsq;
  return choose_tile<false, bf16_t, kTail>(g, tile, stream);
}

// 1 if ts_gemm_tiled_scaled_bf16 takes these sizes.
extern "C" int ts_gemm_tiled_scaled_fits(int M, int N, int K, int pair, int parts) {
  return ts_gemm_tiled_fits(M, N, K, pair) && parts > 0 && parts <= 4096;
}

// C[M, N] = rsqrt(sum_p sumsq[p, m] / K + eps) * (rows[M, K] W[N, K]^T), or with `pair` the
// same for both halves of W = [Wg; Wu] and C = silu(gate) * up.  `c_type`: bfloat16, or
// float32 without `pair`.
extern "C" int ts_gemm_tiled_scaled_bf16(const void* rows, const float* sumsq, int parts,
                                         float eps, const void* w, void* c, int c_type, int M,
                                         int N, int K, int pair, int tile, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ts_gemm_tiled_scaled_fits(M, N, K, pair, parts))
    TS_FAIL("gemm_tiled_scaled: M=%d N=%d K=%d parts=%d not taken", M, N, K, parts);
  if (((uintptr_t)rows | (uintptr_t)w | (uintptr_t)c) & 15)
    TS_FAIL("gemm_tiled_scaled: operands must be 16-byte aligned");
  TiledArgs g{(const bf16_t*)rows, (const bf16_t*)w, c, M, N, K, 0, 0, 1};
  g.sumsq_in = sumsq;
  g.parts = parts;
  g.eps = eps;
  if (pair) {
    if (c_type != TS_BF16) TS_FAIL("gemm_tiled_scaled: the paired form writes bfloat16");
    return choose_tile<true, bf16_t, kScaled>(g, tile, stream);
  }
  if (c_type == TS_BF16) return choose_tile<false, bf16_t, kScaled>(g, tile, stream);
  if (c_type == TS_F32) return choose_tile<false, float, kScaled>(g, tile, stream);
  TS_FAIL("gemm_tiled_scaled: output type %d", c_type);
}
