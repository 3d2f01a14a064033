// The scaled form of the product of gemm_direct.hip: over rows prepared by a tail form,
// with the row factor of the norm applied to the sums; plain or with the SwiGLU epilogue.
#include "gemm_direct_kernel.h"

template <typename TC, bool PAIR>
static int scaled(const DirectArgs& a, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  const int mt = gemm_direct_row_tiles(a.M, a.N, PAIR ? 2 : 4);
  if (mt == 1) {
    if constexpr (!PAIR) {
      // Columns: 16 a workgroup fill whole rounds of the chip's 256 compute units or they
      // do not (N = 6,144 is 384 workgroups, a round and a half: the units with two take
      // twice as long, 15.8 us for 50 MB at 8 rows); with 8 a workgroup the last round is
      // fuller, and where that wins a sixth of the chip or more, 8 it is.
      const int tiles = (a.N + 15) / 16;
      auto fill = [](int groups) { return (double)groups / (((groups + 255) / 256) * 256); };
      if (fill(2 * tiles) > fill(tiles) + 0.15) {
        TS_DIRECT_ROWS(a.M, {
          if (deep) launch<1, 8, TC, false, false, 4, 4, true, false, 8, AR>(a, stream);
          else launch<1, 4, TC, false, false, 4, 4, true, false, 8, AR>(a, stream);
        })
        return 0;
      }
    }
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
