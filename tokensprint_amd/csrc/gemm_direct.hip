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
#include <type_traits>
#include "gemm_common.h"

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

template <int MT, int WK, typename TC, bool PAIR, bool NORM, int S, int PD, bool SCALED = false,
          bool TAIL = false>
__global__ __launch_bounds__(WK* kWave) void gemm_direct_kernel(DirectArgs a) {
  static_assert(!NORM || MT == 1, "the fused form holds one tile of rows");
  static_assert(!(NORM && SCALED) && !(TAIL && (NORM || SCALED || PAIR)), "one form at a time");
  // slices of the sums of squares a lane adds per tile (16 registers in all)
  constexpr int kPartLoads = SCALED ? 16 / MT : 1;
  constexpr int kStep = S * 32;          // K elements of one step
  constexpr int kLane = S * 8;           // of which a lane holds this many, contiguous
  constexpr int NW = PAIR ? 2 : 1;
  __shared__ f32x4 red[(WK - 1) * NW * MT * kWave];
  __shared__ float ss_part[(NORM || SCALED) ? WK * MT * 16 : 1];
  const int M = a.M, N = a.N, K = a.K;
  // the wave's index as a scalar: the K loop's control is then scalar too
  const int wk = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int m_base = blockIdx.y * (MT * 16);
  // rows past the end read the last row again; their results are never stored
  const int64_t w_off = (int64_t)min(n0 + r, N - 1) * K + g * kLane;
  const bf16_t* wrow = a.W + w_off;
  int64_t a_off[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) a_off[mt] = (int64_t)min(m_base + mt * 16 + r, M - 1) * K + g * kLane;
  // without a delta the loads read the stream's own memory and the values are dropped:
  // no branch around a load
  const bool has_delta = NORM && a.delta != nullptr;
  const bf16_t* dbase = has_delta ? a.delta : (const bf16_t*)a.resid_in;

  // this workgroup's slice of the new residual stream: 16-byte units [u0, u0 + chunk8) of
  // every row of the y block; a thread's first unit is loaded now, stored after the loop
  const int units_row = K / 8;
  const int chunk8 = NORM ? (units_row + (int)gridDim.x - 1) / (int)gridDim.x : 0;
  const int copy_rows = NORM ? min(MT * 16, M - m_base) : 0;
  const int copy_total = copy_rows * chunk8;
  auto copy_offset = [&](int idx) -> int64_t {   // element offset, or -1 past the row's end
    const int u = (int)blockIdx.x * chunk8 + idx % chunk8;
    return u < units_row ? (int64_t)(m_base + idx / chunk8) * K + u * 8 : -1;
  };
  f32x4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = c0;
  bf16x8 cd = {0, 0, 0, 0, 0, 0, 0, 0};
  int64_t c_off = -1;
  if constexpr (NORM) {
    if ((int)threadIdx.x < copy_total) c_off = copy_offset(threadIdx.x);
    if (c_off >= 0) {
      c0 = *(const f32x4*)(a.resid_in + c_off);
      c1 = *(const f32x4*)(a.resid_in + c_off + 4);
      cd = *(const bf16x8*)(dbase + c_off);
    }
  }

  // tail form: this lane's four columns of the stream and of the next norm's weight,
  // asked for first by every wave (no load hangs on a condition), used by wave 0 last
  const int tail_n = min(n0 + g * 4, max(N - 4, 0));
  f32x4 tail_x[TAIL ? MT : 1], tail_w4 = {0.f, 0.f, 0.f, 0.f};
  if constexpr (TAIL) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      tail_x[mt] = *(const f32x4*)(a.resid + (int64_t)min(m_base + mt * 16 + r, M - 1) * N + tail_n);
    tail_w4 = *(const f32x4*)(a.tail_w + tail_n);
  }
  // scaled form: slice j of a row's sum of squares goes to wave (j / 4) % WK, lane group
  // j % 4; a slice past the last reads the last again and is dropped
  float part[MT][kPartLoads];
  auto load_parts = [&]() {
    if constexpr (SCALED) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < kPartLoads; ++i) {
          const int j = (i * WK + wk) * 4 + g;
          part[mt][i] = a.sumsq[(int64_t)min(j, a.parts - 1) * M + min(m_base + mt * 16 + r, M - 1)];
        }
    }
  };

  f32x4 acc[NW][MT];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[w][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float ss = 0.f;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const f32x4 fzero = {0.f, 0.f, 0.f, 0.f};

  // one K step of operands as they come from memory
  struct Step {
    bf16x8 w[NW][S];
    bf16x8 x[NORM ? 1 : MT][S];     // plain form: rows of A
    f32x4 rs[NORM ? S : 1][2];      // fused form: residual stream, delta, norm weight
    bf16x8 d[NORM ? S : 1];
    f32x4 nw[NORM ? S : 1][2];
  };
  auto load = [&](Step& st, int kb) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
      for (int w = 0; w < NW; ++w) st.w[w][s] = *(const bf16x8*)(wrow + (int64_t)w * N * K + kb + s * 8);
      if constexpr (NORM) {
        const float* rp = a.resid_in + a_off[0] + kb + s * 8;
        st.rs[s][0] = *(const f32x4*)rp;
        st.rs[s][1] = *(const f32x4*)(rp + 4);
        st.d[s] = *(const bf16x8*)(dbase + a_off[0] + kb + s * 8);
        const float* np = a.norm_w + g * kLane + kb + s * 8;
        st.nw[s][0] = *(const f32x4*)np;
        st.nw[s][1] = *(const f32x4*)(np + 4);
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) st.x[mt][s] = *(const bf16x8*)(a.A + a_off[mt] + kb + s * 8);
      }
    }
  };
  // the same for the last, partial step: what lies beyond K reads as zero
  auto load_tail = [&](Step& st, int kb) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const bool ok = kb + g * kLane + s * 8 < K;
#pragma unroll
      for (int w = 0; w < NW; ++w)
        st.w[w][s] = ok ? *(const bf16x8*)(wrow + (int64_t)w * N * K + kb + s * 8) : zero;
      if constexpr (NORM) {
        const float* rp = a.resid_in + a_off[0] + kb + s * 8;
        st.rs[s][0] = ok ? *(const f32x4*)rp : fzero;
        st.rs[s][1] = ok ? *(const f32x4*)(rp + 4) : fzero;
        st.d[s] = ok ? *(const bf16x8*)(dbase + a_off[0] + kb + s * 8) : zero;
        const float* np = a.norm_w + g * kLane + kb + s * 8;
        st.nw[s][0] = ok ? *(const f32x4*)np : fzero;
        st.nw[s][1] = ok ? *(const f32x4*)(np + 4) : fzero;
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          st.x[mt][s] = ok ? *(const bf16x8*)(a.A + a_off[mt] + kb + s * 8) : zero;
      }
    }
  };
  auto multiply = [&](Step& st) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if constexpr (NORM) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[j] = st.rs[s][0][j]; v[4 + j] = st.rs[s][1][j]; }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] += has_delta ? (float)st.d[s][j] : 0.f;
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ss += v[j] * v[j] + v[4 + j] * v[4 + j];
          o[j] = (bf16_t)(v[j] * st.nw[s][0][j]);
          o[4 + j] = (bf16_t)(v[4 + j] * st.nw[s][1][j]);
        }
#pragma unroll
        for (int w = 0; w < NW; ++w)
          acc[w][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.w[w][s], o, acc[w][0], 0, 0, 0);
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int w = 0; w < NW; ++w)
            acc[w][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.w[w][s], st.x[mt][s],
                                                                 acc[w][mt], 0, 0, 0);
      }
    }
  };

  const int kfull = K / kStep * kStep;
  constexpr int stride = WK * kStep;
  const int kb0 = wk * kStep;
  Step st[PD];
  int kb = kb0;
  // (measured: with one workgroup to a compute unit the waits of the plain loop below,
  // which let all of a round's loads land before its products, serve better)
  if (kb0 + (2 * PD - 1) * stride < kfull && gridDim.x * gridDim.y >= 512) {
    // a long K: rounds in which every buffer is loaded again.  No load in them hangs on a
    // condition, so the wait before a product is for that product's operands alone (a
    // load that may or may not have been issued makes the count of those behind it
    // unknown, and the wait one for nearly all of them).
    // (the scheduler must not reorder the steps' loads either: they return in the order
    // issued, and the first step's have to be the oldest)
#pragma unroll
    for (int p = 0; p < PD; ++p) {
      load(st[p], kb0 + p * stride);
      __builtin_amdgcn_sched_barrier(0);
    }
    load_parts();
    __builtin_amdgcn_sched_barrier(0);
    for (; kb + (2 * PD - 1) * stride < kfull; kb += PD * stride) {
#pragma unroll
      for (int p = 0; p < PD; ++p) {
        multiply(st[p]);      // no copy of the step: it would wait for all of it to arrive
        load(st[p], kb + (p + PD) * stride);
      }
    }
  } else {
#pragma unroll
    for (int p = 0; p < PD; ++p)
      if (kb0 + p * stride < kfull) load(st[p], kb0 + p * stride);
    load_parts();
  }
  // the last steps (all of them, for a short K)
  for (; kb < kfull; kb += PD * stride) {
#pragma unroll
    for (int p = 0; p < PD; ++p) {
      const int k = kb + p * stride;
      if (k < kfull) {
        multiply(st[p]);
        if (k + PD * stride < kfull) load(st[p], k + PD * stride);
      }
    }
  }
  // the partial step belongs to the wave whose turn it would be
  if (kfull < K && (kfull / kStep) % WK == wk) {
    load_tail(st[0], kfull);
    multiply(st[0]);
  }

  if constexpr (NORM) {
    auto put = [&](int64_t off, f32x4 x0, f32x4 x1, bf16x8 d) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x0[j] += has_delta ? (float)d[j] : 0.f;
        x1[j] += has_delta ? (float)d[4 + j] : 0.f;
      }
      *(f32x4*)(a.resid_out + off) = x0;
      *(f32x4*)(a.resid_out + off + 4) = x1;
    };
    if (c_off >= 0) put(c_off, c0, c1, cd);
    // few workgroup columns and a long K: more units than threads
    for (int idx = threadIdx.x + blockDim.x; idx < copy_total; idx += blockDim.x) {
      const int64_t off = copy_offset(idx);
      if (off >= 0)
        put(off, *(const f32x4*)(a.resid_in + off), *(const f32x4*)(a.resid_in + off + 4),
            *(const bf16x8*)(dbase + off));
    }
    // squares of row r: the four lanes of the row, then the waves in order
    ss += __shfl_xor(ss, 16, kWave);
    ss += __shfl_xor(ss, 32, kWave);
    if (g == 0) ss_part[wk * 16 + r] = ss;
  }
  if constexpr (SCALED) {
    // the row's squares: this lane's slices in order, the four lane groups, then (below)
    // the waves in order
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float sq = 0.f;
#pragma unroll
      for (int i = 0; i < kPartLoads; ++i) sq += ((i * WK + wk) * 4 + g < a.parts) ? part[mt][i] : 0.f;
      sq += __shfl_xor(sq, 16, kWave);
      sq += __shfl_xor(sq, 32, kWave);
      if (g == 0) ss_part[(wk * MT + mt) * 16 + r] = sq;
    }
  }
  if (WK > 1) {   // partial sums of the K splits, added in split order
    if (wk > 0) {
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          red[(((wk - 1) * NW + w) * MT + mt) * kWave + lane] = acc[w][mt];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int k2 = 1; k2 < WK; ++k2)
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[w][mt] += red[(((k2 - 1) * NW + w) * MT + mt) * kWave + lane];
  }
  float rstd[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    rstd[mt] = 1.f;
    if constexpr (NORM || SCALED) {
      float total = 0.f;
#pragma unroll
      for (int k2 = 0; k2 < WK; ++k2) total += ss_part[(k2 * MT + mt) * 16 + r];
      rstd[mt] = rsqrtf(total / (float)K + a.eps);
    }
  }

  // lane holds D[n = n0 + g*4 + t][m = tile*16 + r], t = 0..3
  const int n = n0 + g * 4;
  if constexpr (TAIL) {
    const bool n_ok = n < N;                 // N is a multiple of 4 here
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = m_base + mt * 16 + r;
      f32x4 x = tail_x[mt];
      float sq = 0.f;
      bf16x4_t h;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // the product rounded to the activation type first, as the unfused path stores it
        x[t] += (float)(bf16_t)acc[0][mt][t];
        sq += x[t] * x[t];
        h[t] = (bf16_t)(x[t] * tail_w4[t]);
      }
      const bool ok = n_ok && m < M;
      if (ok) {
        *(f32x4*)(a.resid + (int64_t)m * N + n) = x;
        *(bf16x4_t*)(a.prepared + (int64_t)m * N + n) = h;
      }
      sq = ok ? sq : 0.f;
      sq += __shfl_xor(sq, 16, kWave);
      sq += __shfl_xor(sq, 32, kWave);
      if (g == 0 && m < M) a.sumsq_out[(int64_t)blockIdx.x * M + m] = sq;
    }
    return;
  }
  if (n >= N) return;
  TC* C = (TC*)a.C;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m_base + mt * 16 + r;
    if (m >= M) continue;
    f32x4 v = acc[0][mt];
    if (NORM || SCALED) {
#pragma unroll
      for (int t = 0; t < 4; ++t) v[t] *= rstd[mt];
    }
    if (PAIR) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // the two products are rounded to the activation type first, as the unfused
        // path stores them, then silu(gate) * up in float32
        const float gt = (float)(bf16_t)v[t], up = (float)(bf16_t)(acc[1][mt][t] * rstd[mt]);
        v[t] = gt / (1.f + expf(-gt)) * up;
      }
    }
    store4<TC>(C + (int64_t)m * N + n, v, N - n);
  }
}

template <int MT, int WK, typename TC, bool PAIR, bool NORM, int S, int PD, bool SCALED = false,
          bool TAIL = false>
static void launch(const DirectArgs& a, hipStream_t stream) {
  dim3 grid((a.N + 15) / 16, (a.M + MT * 16 - 1) / (MT * 16));
  hipLaunchKernelGGL((gemm_direct_kernel<MT, WK, TC, PAIR, NORM, S, PD, SCALED, TAIL>), grid,
                     dim3(WK * kWave), 0, stream, a);
}

// Tiles of 16 rows a workgroup holds: all of them up to `most` when the columns alone
// give the chip's 256 compute units a workgroup each, fewer (more workgroups along y)
// when they do not.  The choice changes which workgroup computes a row, not how.
static int tiles_per_workgroup(int M, int N, int most) {
  const int tiles_m = (M + 15) / 16, tiles_n = (N + 15) / 16;
  const int want_y = (256 + tiles_n - 1) / tiles_n;
  int mt = tiles_m < most ? tiles_m : most;
  if (want_y > 1) mt = tiles_m / want_y;
  mt = mt < most ? mt : most;
  return mt >= 4 ? 4 : mt >= 2 ? 2 : 1;
}

// Steps in flight: as many as the registers hold (a step of one tile is 32 registers, of
// four tiles 80), so that a wave's two or three steps of a decode product all are.
template <typename TC, bool PAIR>
static int dispatch(const DirectArgs& a, bool norm, hipStream_t stream) {
  const bool deep = layout_deep(a.N, a.K);
  if (norm) {
    if (deep) launch<1, 8, TC, PAIR, true, 2, 3>(a, stream);
    else launch<1, 4, TC, PAIR, true, 4, 2>(a, stream);
    return 0;
  }
  const int mt = tiles_per_workgroup(a.M, a.N, PAIR ? 2 : 4);
  if (a.sumsq) {
    if (deep) {
      if (mt == 1) launch<1, 8, TC, PAIR, false, 4, 4, true>(a, stream);
      else if (mt == 2) launch<2, 8, TC, PAIR, false, 4, 3, true>(a, stream);
      else if constexpr (!PAIR) launch<4, 8, TC, PAIR, false, 4, 2, true>(a, stream);
    } else {
      if (mt == 1) launch<1, 4, TC, PAIR, false, 4, 4, true>(a, stream);
      else if (mt == 2) launch<2, 4, TC, PAIR, false, 4, 3, true>(a, stream);
      else if constexpr (!PAIR) launch<4, 4, TC, PAIR, false, 4, 2, true>(a, stream);
    }
    return 0;
  }
  if constexpr (!PAIR && std::is_same<TC, bf16_t>::value) {
    if (a.resid) {
      if (deep) {
        if (mt == 1) launch<1, 8, TC, false, false, 4, 4, false, true>(a, stream);
        else if (mt == 2) launch<2, 8, TC, false, false, 4, 3, false, true>(a, stream);
        else launch<4, 8, TC, false, false, 4, 2, false, true>(a, stream);
      } else {
        if (mt == 1) launch<1, 4, TC, false, false, 4, 4, false, true>(a, stream);
        else if (mt == 2) launch<2, 4, TC, false, false, 4, 3, false, true>(a, stream);
        else launch<4, 4, TC, false, false, 4, 2, false, true>(a, stream);
      }
      return 0;
    }
  }
  if (deep) {
    if (mt == 1) launch<1, 8, TC, PAIR, false, 4, 4>(a, stream);
    else if (mt == 2) launch<2, 8, TC, PAIR, false, 4, 3>(a, stream);
    else if constexpr (!PAIR) launch<4, 8, TC, PAIR, false, 4, 2>(a, stream);
  } else {
    if (mt == 1) launch<1, 4, TC, PAIR, false, 4, 4>(a, stream);
    else if (mt == 2) launch<2, 4, TC, PAIR, false, 4, 3>(a, stream);
    else if constexpr (!PAIR) launch<4, 4, TC, PAIR, false, 4, 2>(a, stream);
  }
  return 0;
}

bool gemm_direct_tail_fits(int M, int N, int K) {
  return M >= 1 && M <= 64 && !layout_wide(N, K) && K > 0 && K % 8 == 0 && N % 4 == 0;
}

bool gemm_direct_scaled_fits(int M, int N, int K, bool pair) {
  if (M < 1 || M > 64 || layout_wide(N, K) || K <= 0 || K % 8) return false;
  const int mt = tiles_per_workgroup(M, N, pair ? 2 : 4);
  const int waves = layout_deep(N, K) ? 8 : 4;
  return (K + 15) / 16 <= (16 / mt) * 4 * waves;     // the slices its lanes hold
}

int gemm_direct_launch(const DirectArgs& a, int c_type, bool pair, bool norm,
                       hipStream_t stream) {
  if (layout_wide(a.N, a.K)) TS_FAIL("gemm_direct: not for the wide layout (N=%d, K=%d)", a.N, a.K);
  if (a.resid && (norm || pair || a.sumsq || c_type != TS_BF16 || !gemm_direct_tail_fits(a.M, a.N, a.K)))
    TS_FAIL("gemm_direct: the tail form does not take this product (M=%d, N=%d, K=%d)", a.M, a.N, a.K);
  if (a.sumsq && (norm || a.parts != (a.K + 15) / 16 || !gemm_direct_scaled_fits(a.M, a.N, a.K, pair)))
    TS_FAIL("gemm_direct: the scaled form does not take this product (M=%d, N=%d, K=%d, %d slices)",
            a.M, a.N, a.K, a.parts);
  if (a.K <= 0 || a.K % 8) TS_FAIL("gemm_direct: K=%d must be a positive multiple of 8", a.K);
  if (norm && a.M > 16) TS_FAIL("gemm_direct: the fused form takes at most 16 rows, got %d", a.M);
  if ((a.M + 15) / 16 > 65535) TS_FAIL("gemm_direct: M=%d too large", a.M);
  if (pair) {
    if (c_type != TS_BF16) TS_FAIL("gemm_direct: the paired product writes bfloat16");
    return dispatch<bf16_t, true>(a, norm, stream);
  }
  if (c_type == TS_F32) return dispatch<float, false>(a, norm, stream);
  if (c_type == TS_BF16) return dispatch<bf16_t, false>(a, norm, stream);
  TS_FAIL("gemm_direct: unknown output type %d", c_type);
}
