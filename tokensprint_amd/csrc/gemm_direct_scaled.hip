// The scaled form of the product of gemm_direct.hip: over rows prepared by a tail form,
// with the row factor of the norm applied to the sums; plain or with the SwiGLU epilogue.
#include "gemm_direct_kernel.h"

template <typename TC, bool PAIR>
static int scaled(const DirectArgs& a, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  const int mt = gemm_direct_row_tiles(a.M, a.N, PAIR ? 2 : 4);
  if (mt == 1) {
    TS_DIRECT_ROWS(a.M, {
      if (deep) launch<1, 8, TC, PAIR, false, 4, 4, true, false, 16, AR>(a, stream);
      else launch<1, 4, TC, PAIR, false, 4, 4, true, false, 16, AR>(a, stream);
    })
  } else if (deep) {
    if (mt == 2) launch<2, 8, TC, PAIR, false, 4, 3, true>(a, stream);
    else if constexpr (!PAIR) launch<4, 8, TC, PAIR, false, 4, 2, true>(a, stream);
  } else {
    if (mt == 2) launch<2, 4, TC, PAIR, false, 4, 3, true>(a, stream);
    else if constexpr (!PAIR) launch<4, 4, TC, PAIR, false, 4, 2, true>(a, stream);
  }
  return 0;
}

int gemm_direct_scaled(const DirectArgs& a, int c_type, bool pair, hipStream_t stream) {
  if (pair) return scaled<bf16_t, true>(a, stream);
  return c_type == TS_F32 ? scaled<float, false>(a, stream) : scaled<bf16_t, false>(a, stream);
}
