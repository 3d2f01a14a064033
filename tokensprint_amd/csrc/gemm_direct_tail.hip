// The tail form of the product of gemm_direct.hip: the product that ends a sub-layer adds
// itself into the residual stream and prepares the rows for the norm that follows.
#include "gemm_direct_kernel.h"

int gemm_direct_tail(const DirectArgs& a, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  const int mt = gemm_direct_row_tiles(a.M, a.N, 4);
  if (mt == 1) {
    const int cw = gemm_direct_columns(a.M, a.N);
    TS_DIRECT_ROWS(a.M, {
      TS_DIRECT_COLUMNS(cw, {
        if (deep) launch<1, 8, bf16_t, false, false, 4, 4, false, true, CW, AR>(a, stream);
        else launch<1, 4, bf16_t, false, false, 4, 4, false, true, CW, AR>(a, stream);
      })
    })
  } else if (deep) {
    if (mt == 2) launch<2, 8, bf16_t, false, false, 4, 3, false, true>(a, stream);
    else launch<4, 8, bf16_t, false, false, 4, 2, false, true>(a, stream);
  } else {
    if (mt == 2) launch<2, 4, bf16_t, false, false, 4, 3, false, true>(a, stream);
    else launch<4, 4, bf16_t, false, false, 4, 2, false, true>(a, stream);
  }
  return 0;
}
