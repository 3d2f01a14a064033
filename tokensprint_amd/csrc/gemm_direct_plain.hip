// The plain form of the product of gemm_direct.hip: C = A W^T, bfloat16 or float32 out.
#include "gemm_direct_kernel.h"

template <typename TC>
static int plain(const DirectArgs& a, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  const int mt = gemm_direct_row_tiles(a.M, a.N, 4);
  if (mt == 1) {
    // float32 results are the output head's, which has columns enough
    const int cw = std::is_same<TC, float>::value ? 16 : gemm_direct_columns(a.M, a.N);
    TS_DIRECT_ROWS(a.M, {
      if constexpr (std::is_same<TC, float>::value) {
        if (deep) launch<1, 8, TC, false, false, 4, 4, false, false, 16, AR>(a, stream);
        else launch<1, 4, TC, false, false, 4, 4, false, false, 16, AR>(a, stream);
      } else {
        TS_DIRECT_COLUMNS(cw, {
          if (deep) launch<1, 8, TC, false, false, 4, 4, false, false, CW, AR>(a, stream);
          else launch<1, 4, TC, false, false, 4, 4, false, false, CW, AR>(a, stream);
        })
      }
    })
  } else if (deep) {
    if (mt == 2) launch<2, 8, TC, false, false, 4, 3>(a, stream);
    else launch<4, 8, TC, false, false, 4, 2>(a, stream);
  } else {
    if (mt == 2) launch<2, 4, TC, false, false, 4, 3>(a, stream);
    else launch<4, 4, TC, false, false, 4, 2>(a, stream);
  }
  return 0;
}

int gemm_direct_plain(const DirectArgs& a, int c_type, hipStream_t stream) {
  return c_type == TS_F32 ? plain<float>(a, stream) : plain<bf16_t>(a, stream);
}
