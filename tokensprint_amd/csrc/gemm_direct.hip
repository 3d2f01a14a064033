// C[M,N] = A[M,K] * W[N,K]^T, bfloat16 on the matrix cores, for the layouts in which a
// workgroup owns 16 rows of W and its 4 or 8 waves split K: the decode products and the
// short-portion products of up to 64 rows.
//
// Nothing is staged: W and A go from global memory straight into the operand layout of
// v_mfma_f32_16x16x32_bf16, into PD buffers of one step each; a buffer is loaded again as
// soon as it has been multiplied.  A wave so has its whole share of a small product in
// flight at once, and the kernel costs one memory latency, with no barrier before the
// final sum.  A step is S matrix-core products deep (S * 32 elements of K); S = 4
// everywhere except in the fused form with 8 waves, whose float32 operands would not fit
// the registers twice.  A wave holds up to 4 tiles of 16 rows of A; more rows, or too few
// workgroups to cover the chip, go to further workgroups along y, which read W again
// from the second-level cache.
//
// Fused form (at most 16 rows): A is not stored but is the RMSNorm of the residual
// stream, x = resid_in + delta, A = bf16(x * norm_w) * rsqrt(mean(x^2) + eps).  Every
// wave builds its operand from the float32 stream as it arrives and sums the squares of
// its share; the row factor commutes with the product and is applied to the sums at the
// end, so nothing waits for it.  The new stream x goes to resid_out in slices, one per
// workgroup column, read again at the start of the kernel and stored after the K loop:
// a store inside the loop would share the loads' counter and make every wait for an
// operand a wait for everything in flight.
//
// Tail and scaled form (up to 64 rows): the same norm split over two products.  The
// product that ends a sub-layer (TAIL) adds its result to the residual stream in place,
// x = resid + bf16(A W^T), and leaves for the product that follows the rows x * norm_w in
// bfloat16 and, per workgroup column, each row's sum of x^2 over its 16 columns.  That
// product (SCALED) is a plain one over the prepared rows; its waves add the slices of a
// row's sum of squares, in a fixed order, while their operands are on the way, and the
// row factor is applied to the sums at the end.  No workgroup reads the float32 stream
// but the one that updates its own 16 columns of it.
//
// The K split and the order of the final sum are those of the layout rule, so a row's
// result is bit for bit the same for any number of rows and any tile it lands in.
#include "gemm_direct_kernel.h"

// Tiles of 16 rows a workgroup holds: all of them up to `most` when the columns alone
// give the chip's 256 compute units a workgroup each, fewer (more workgroups along y)
// when they do not.  The choice changes which workgroup computes a row, not how.
int gemm_direct_row_tiles(int M, int N, int most) {
  const int tiles_m = (M + 15) / 16, tiles_n = (N + 15) / 16;
  const int want_y = (256 + tiles_n - 1) / tiles_n;
  int mt = tiles_m < most ? tiles_m : most;
  if (want_y > 1) mt = tiles_m / want_y;
  mt = mt < most ? mt : most;
  return mt >= 4 ? 4 : mt >= 2 ? 2 : 1;
}

// Columns per workgroup for a plain or tail product of up to 16 rows: fewer than 16 while
// that gives the chip's 256 compute units more workgroups to share the weight among, and
// never more than 256 of them (the slices of the tail form's sums of squares are one per
// workgroup, and the product that follows holds 256 of them in its lanes).
int gemm_direct_columns(int M, int N) {
  if (M > 16 || (N + 15) / 16 >= 192) return 16;
  return N <= 1024 ? 4 : N <= 2048 ? 8 : 16;
}

// Fused norm in front (at most 16 rows): the operand is built in registers, nothing packed.
template <typename TC, bool PAIR>
static int norm_form(const DirectArgs& a, hipStream_t stream) {
  if (layout_deep(a.N, a.K)) launch<1, 8, TC, PAIR, true, 2, 3>(a, stream);
  else launch<1, 4, TC, PAIR, true, 4, 2>(a, stream);
  return 0;
}

int gemm_direct_norm(const DirectArgs& a, int c_type, bool pair, hipStream_t stream) {
  if (pair) return norm_form<bf16_t, true>(a, stream);
  if (c_type == TS_F32) return norm_form<float, false>(a, stream);
  return norm_form<bf16_t, false>(a, stream);
}

// Steps in flight: as many as the registers hold (a step of one tile is 32 registers, of
// four tiles 80), so that a wave's two or three steps of a decode product all are.
int gemm_direct_pair(const DirectArgs& a, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  const int mt = gemm_direct_row_tiles(a.M, a.N, 2);
  if (mt == 1) {
    TS_DIRECT_ROWS(a.M, {
      if (deep) launch<1, 8, bf16_t, true, false, 4, 4, false, false, 16, AR>(a, stream);
      else launch<1, 4, bf16_t, true, false, 4, 4, false, false, 16, AR>(a, stream);
    })
  } else if (deep) {
    launch<2, 8, bf16_t, true, false, 4, 3>(a, stream);
  } else {
    launch<2, 4, bf16_t, true, false, 4, 3>(a, stream);
  }
  return 0;
}

bool gemm_direct_tail_fits(int M, int N, int K) {
  return M >= 1 && M <= 64 && !layout_wide(N, K) && K > 0 && K % 8 == 0 && N % 4 == 0;
}

// Slices of a row's sum of squares that the tail form of a product with N columns leaves.
int gemm_direct_tail_parts(int M, int N) {
  const int cw = gemm_direct_columns(M, N);
  return (N + cw - 1) / cw;
}

bool gemm_direct_scaled_fits(int M, int N, int K, bool pair, int parts) {
  if (M < 1 || M > 64 || layout_wide(N, K) || K <= 0 || K % 8 || parts < 1) return false;
  const int mt = gemm_direct_row_tiles(M, N, pair ? 2 : 4);
  const int waves = layout_deep(N, K) ? 8 : 4;
  return parts <= (16 / mt) * 4 * waves;     // the slices its lanes hold
}

int gemm_direct_launch(const DirectArgs& a, int c_type, bool pair, bool norm,
                       hipStream_t stream) {
  if (layout_wide(a.N, a.K)) TS_FAIL("gemm_direct: not for the wide layout (N=%d, K=%d)", a.N, a.K);
  if (a.resid && (norm || pair || a.sumsq || c_type != TS_BF16 || !gemm_direct_tail_fits(a.M, a.N, a.K)))
    TS_FAIL("gemm_direct: the tail form does not take this product (M=%d, N=%d, K=%d)", a.M, a.N, a.K);
  if (a.sumsq && (norm || !gemm_direct_scaled_fits(a.M, a.N, a.K, pair, a.parts)))
    TS_FAIL("gemm_direct: the scaled form does not take this product (M=%d, N=%d, K=%d, %d slices)",
            a.M, a.N, a.K, a.parts);
  if (a.K <= 0 || a.K % 8) TS_FAIL("gemm_direct: K=%d must be a positive multiple of 8", a.K);
  if (norm && a.M > 16) TS_FAIL("gemm_direct: the fused form takes at most 16 rows, got %d", a.M);
  if ((a.M + 15) / 16 > 65535) TS_FAIL("gemm_direct: M=%d too large", a.M);
  if (c_type != TS_F32 && c_type != TS_BF16) TS_FAIL("gemm_direct: unknown output type %d", c_type);
  if (pair && c_type != TS_BF16) TS_FAIL("gemm_direct: the paired product writes bfloat16");
  if (norm) return gemm_direct_norm(a, c_type, pair, stream);
  if (a.sumsq) return gemm_direct_scaled(a, c_type, pair, stream);
  if (a.resid) return gemm_direct_tail(a, stream);
  if (pair) return gemm_direct_pair(a, stream);
  return gemm_direct_plain(a, c_type, stream);
}
