// Entry points of the LDS-tiled product for many rows (gemm_tiled_kernel.h): the plain
// form and the gate/up form with the SiLU-multiply in its epilogue.
#include "gemm_tiled_kernel.h"

// 1 if ts_gemm_tiled_bf16 takes these sizes.
extern "C" int ts_gemm_tiled_fits(int M, int N, int K, int pair) {
  const int64_t rows_w = pair ? 2 * (int64_t)N : N;
  return M > 0 && N > 0 && K >= 256 && K % 64 == 0 && N % 16 == 0 &&
         (int64_t)M * K * 2 < (1ll << 32) && rows_w * K * 2 < (1ll << 32);
}

// C[M, N] = A[M, K] W[N, K]^T, or with `pair` C[M, N] = silu(A Wg^T) * (A Wu^T) for
// W = [Wg; Wu] of 2 N rows.  `c_type`: bfloat16 or float32 (float32 not with `pair`).
// `tile`: 0 lets the sizes choose; 1 to 5 name a tile (for measuring; the result is the
// same to the bit).
extern "C" int ts_gemm_tiled_bf16(const void* a, const void* w, void* c, int c_type, int M, int N,
                                  int K, int pair, int tile, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ts_gemm_tiled_fits(M, N, K, pair))
    TS_FAIL("gemm_tiled: M=%d N=%d K=%d not taken (K a multiple of 64 from 256, N of 16, "
            "operands below 4 GiB)", M, N, K);
  if (((uintptr_t)a | (uintptr_t)w | (uintptr_t)c) & 15)
    TS_FAIL("gemm_tiled: operands must be 16-byte aligned");
  TiledArgs g{(const bf16_t*)a, (const bf16_t*)w, c, M, N, K, 0, 0, 1};
  if (pair) {
    if (c_type != TS_BF16) TS_FAIL("gemm_tiled: the paired form writes bfloat16");
    return choose_tile<true, bf16_t>(g, tile, stream);
  }
  if (c_type == TS_BF16) return choose_tile<false, bf16_t>(g, tile, stream);
  if (c_type == TS_F32) return choose_tile<false, float>(g, tile, stream);
  TS_FAIL("gemm_tiled: output type %d", c_type);
}
