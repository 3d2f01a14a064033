// The merged tail form of the product of gemm_direct.hip: the output projection of a
// decode step whose attention was split over the keys.  The attention kernels leave one
// partial result per split; instead of a kernel that merges them into the attention
// output and a product that reads it, the product's workgroups merge the rows they need
// into LDS themselves (each all of them: the partial sums of a few rows are small) and
// go on as the tail form does.  One dependent kernel less per layer, which at one to a
// dozen rows is worth more than the partial sums read 256 times over.
#include "attention_mfma.h"
#include "gemm_direct_kernel.h"

int gemm_direct_merged(const DirectArgs& a, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  const int cw = gemm_direct_columns(a.M, a.N);
  bool ok = true;
  TS_DIRECT_ROWS(a.M, {
    TS_DIRECT_COLUMNS(cw, {
      ok = deep ? launch_merged<8, CW, AR>(a, stream) : launch_merged<4, CW, AR>(a, stream);
    })
  })
  if (!ok) TS_FAIL("gemm_tail_merged: the rows of A (%d bytes) do not fit LDS", a.K * 2 * 16);
  return 0;
}

// Whether ts_gemm_tail_merged_bf16 takes this product: what the tail form takes, one
// tile of rows, whole 8-element pieces inside a head, and the merged rows of A (as
// launch_merged lays them out, padded to the rows a load is packed for) within the 160 KiB
// of LDS a workgroup can have.
extern "C" int ts_gemm_tail_merged_fits(int M, int N, int heads, int hd) {
  const int64_t K = (int64_t)heads * hd;
  if (!(M >= 1 && M <= 16 && heads >= 1 && hd >= 8 && hd % 8 == 0 && K <= 8192)) return 0;
  const int64_t lds = (int64_t)gemm_direct_packed_rows(M) * (K / 8 + 1) * 16;
  return lds <= 160 * 1024 && gemm_direct_tail_fits(M, N, (int)K);
}

// Rows up to which it pays.  Every workgroup merges all rows, and what it reads for that
// grows with the rows while the kernel it saves does not: measured in decode steps of
// the 0.6B shape against a merge kernel of its own, a step is 6.4 % shorter at one row,
// 4.1 % at two, 1.2 % at three, the same at four, 1 to 3 % longer from five to eight.
// Against the decode kernel merging its splits itself (the item's last workgroup to
// finish) it is 3 % ahead at one row, 1 % at two and 2 % behind at three.
extern "C" int ts_gemm_tail_merged_rows() { return 2; }

// ts_gemm_tail_bf16 with A = the attention output of a decode step of M tokens that
// ts_attention_decode left unmerged (`defer_merge`): partial_o [M * nkv * ceil(group / 16),
// splits, 16, hd], partial_ml likewise with (row maximum, row sum), positions [M].
extern "C" int ts_gemm_tail_merged_bf16(const float* partial_o, const float* partial_ml,
                                        const int* positions, int splits, int nq, int nkv, int hd,
                                        int window, const void* w, float* resid,
                                        const float* norm_w, void* prepared, float* sumsq, int M,
                                        int N, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (nkv < 1 || nq % nkv || splits < 1)
    TS_FAIL("gemm_tail_merged: %d heads over %d key/value heads, %d splits", nq, nkv, splits);
  if (!ts_gemm_tail_merged_fits(M, N, nq, hd))
    TS_FAIL("gemm_tail_merged: M=%d, N=%d, %d heads of %d is not a product it takes", M, N, nq, hd);
  if (((uintptr_t)partial_o | (uintptr_t)w | (uintptr_t)resid | (uintptr_t)norm_w) & 15)
    TS_FAIL("gemm_tail_merged: operands must be 16-byte aligned");
  if (((uintptr_t)prepared) & 7) TS_FAIL("gemm_tail_merged: the prepared rows must be 8-byte aligned");
  if (!partial_o || !partial_ml || !positions || !w || !resid || !norm_w || !prepared || !sumsq)
    TS_FAIL("gemm_tail_merged: null operand");
  DirectArgs da = {};
  da.W = (const bf16_t*)w; da.M = M; da.N = N; da.K = nq * hd;
  da.resid = resid; da.tail_w = norm_w; da.prepared = (bf16_t*)prepared; da.sumsq_out = sumsq;
  da.merge_o = partial_o; da.merge_ml = partial_ml; da.merge_pos = positions;
  da.merge_splits = splits; da.merge_nkv = nkv; da.merge_group = nq / nkv; da.merge_hd = hd;
  da.merge_window = window; da.merge_chunk = kChunk;
  if (gemm_direct_merged(da, stream)) return -1;
  TS_CHECK_LAUNCH("gemm_tail_merged");
  return 0;
}
