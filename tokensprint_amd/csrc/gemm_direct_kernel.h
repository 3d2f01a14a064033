// The kernel of gemm_direct.hip and its launch, for the translation units that hold its
// instantiations (gemm_direct.hip and gemm_direct_*.hip: the forms are many, and they
// compile side by side).
#pragma once
#include <type_traits>
#include "gemm_common.h"


// The lane's 16-byte register moved n lanes down its row of 16 lanes (lane i takes lane
// i + n's; the top n lanes get zeros).
template <int N_>
__device__ __forceinline__ bf16x8 row_down(bf16x8 v) {
  if constexpr (N_ == 0) return v;
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  i32x4 x = __builtin_bit_cast(i32x4, v), y;
#pragma unroll
  for (int i = 0; i < 4; ++i) y[i] = __builtin_amdgcn_update_dpp(0, x[i], 0x100 + N_, 0xf, 0xf, true);
  return __builtin_bit_cast(bf16x8, y);
}

// (n is a constant once the loops around a call are unrolled)
__device__ __forceinline__ bf16x8 row_down_by(bf16x8 v, int n) {
  switch (n) {
    case 4: return row_down<4>(v);
    case 8: return row_down<8>(v);
    case 12: return row_down<12>(v);
    default: return v;
  }
}

template <int MT, int WK, typename TC, bool PAIR, bool NORM, int S, int PD, bool SCALED = false,
          bool TAIL = false, int CW = 16, int AR = 16, bool MERGE = false>
__global__ __launch_bounds__(WK* kWave) void gemm_direct_kernel(DirectArgs a) {
  static_assert(!NORM || MT == 1, "the fused form holds one tile of rows");
  static_assert(!MERGE || (TAIL && MT == 1), "the merged form: a tail product of one tile of rows");
  // Packed operands.  A compute unit takes a wave's 16-byte load in about 28 cycles
  // whatever its lanes ask for, and that rate, not the bytes, bounds these products.  An
  // operand with fewer than 16 rows (AR rows of A that exist, CW rows of W that this
  // workgroup owns) is therefore loaded with its 16 row lanes split into 16/AR (16/CW)
  // sets that fetch the pieces of 16/AR consecutive products, one instruction instead of
  // several, and the piece a product needs is moved down to the first rows' lanes (a DPP
  // move; the other rows of the operand only produce results that nobody stores).
  static_assert((CW == 16 || CW == 8 || CW == 4) && (AR == 16 || AR == 8 || AR == 4), "rows");
  static_assert(CW == 16 || (MT == 1 && !PAIR && !NORM), "narrow tiles: one tile of rows, one weight, A from memory");
  static_assert(AR == 16 || (MT == 1 && !NORM), "packed rows of A: one tile, A from memory");
  constexpr int GW = 16 / CW, GA = 16 / AR;          // pieces per load instruction
  static_assert(S % GW == 0 && S % GA == 0, "a step holds whole instructions");
  static_assert(!(NORM && SCALED) && !(TAIL && (NORM || SCALED || PAIR)), "one form at a time");
  // slices of the sums of squares a lane adds per tile (16 registers in all), four to a load
  constexpr int kPartLoads = SCALED ? 4 / MT : 1;
  constexpr int kStep = S * 32;          // K elements of one step
  // Where a lane's 8-element pieces of a step lie: piece s of lane group g at
  // s * kPiece + g * kGroup elements, so that the four lanes of a row read 64 contiguous
  // bytes with one instruction (a lane with its S pieces side by side had an instruction
  // touch twice as many cache lines: 0.1 to 0.7 us more per product, measured at 8 to 64
  // rows).  A and W take the same places, so the products' pairs are the same.
  constexpr int kGroup = 8, kPiece = 32;
  constexpr int NW = PAIR ? 2 : 1;
  __shared__ f32x4 red[(WK - 1) * NW * MT * kWave];
  __shared__ float ss_part[(NORM || SCALED) ? WK * MT * 16 : 1];
  const int M = a.M, N = a.N, K = a.K;
  // the wave's index as a scalar: the K loop's control is then scalar too
  const int wk = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * CW;
  const int m_base = blockIdx.y * (MT * 16);
  // rows past the end read the last row again; their results are never stored
  const int64_t w_off = (int64_t)min(n0 + r % CW, N - 1) * K + g * kGroup + (r / CW) * kPiece;
  const bf16_t* wrow = a.W + w_off;
  int64_t a_off[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    a_off[mt] = (int64_t)min(m_base + mt * 16 + r % AR, M - 1) * K + g * kGroup + (r / AR) * kPiece;
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
  // scaled form: a row's slices lie side by side (rows of `parts` rounded up to four);
  // four of them, 4 j .. 4 j + 3, go to wave (j / 4) % WK, lane group j % 4 in one load; a
  // four past the last reads the last again and is dropped
  const int part_stride = (a.parts + 3) & ~3;
  f32x4 part[MT][kPartLoads];
  auto load_parts = [&]() {
    if constexpr (SCALED) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < kPartLoads; ++i) {
          const int j = (i * WK + wk) * 4 + g;
          part[mt][i] = *(const f32x4*)(a.sumsq + (int64_t)min(m_base + mt * 16 + r, M - 1) * part_stride +
                                        4 * min(j, part_stride / 4 - 1));
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
    bf16x8 w[NW][S / GW];
    bf16x8 x[NORM ? 1 : MT][S / GA];     // plain form: rows of A
    f32x4 rs[NORM ? S : 1][2];      // fused form: residual stream, delta, norm weight
    bf16x8 d[NORM ? S : 1];
    f32x4 nw[NORM ? S : 1][2];
  };
  // merged form: the rows of A, merged out of the key splits' partial sums into LDS by
  // the whole workgroup before the K loop; a row is K / 8 pieces and one of padding, so
  // that the same piece of the 16 rows lies in 16 different banks
  extern __shared__ __attribute__((aligned(16))) unsigned char merged_rows[];
  const int row_pieces = K / 8 + 1;
  const bf16x8* a_row = (const bf16x8*)merged_rows + min(m_base + r % AR, M - 1) * row_pieces +
                        (g * kGroup + (r / AR) * kPiece) / 8;
  auto load = [&](Step& st, int kb, bool of_w = true, bool of_a = true) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if (s % GW == 0 && of_w) {
#pragma unroll
        for (int w = 0; w < NW; ++w)
          st.w[w][s / GW] = *(const bf16x8*)(wrow + (int64_t)w * N * K + kb + s * kPiece);
      }
      if (!of_a) continue;
      if constexpr (MERGE) {
        if (s % GA == 0) st.x[0][s / GA] = a_row[(kb + s * kPiece) / 8];
      } else if constexpr (NORM) {
        const float* rp = a.resid_in + a_off[0] + kb + s * kPiece;
        st.rs[s][0] = *(const f32x4*)rp;
        st.rs[s][1] = *(const f32x4*)(rp + 4);
        st.d[s] = *(const bf16x8*)(dbase + a_off[0] + kb + s * kPiece);
        const float* np = a.norm_w + g * kGroup + kb + s * kPiece;
        st.nw[s][0] = *(const f32x4*)np;
        st.nw[s][1] = *(const f32x4*)(np + 4);
      } else {
        if (s % GA == 0) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            st.x[mt][s / GA] = *(const bf16x8*)(a.A + a_off[mt] + kb + s * kPiece);
        }
      }
    }
  };
  // the same for the last, partial step: what lies beyond K reads as zero
  auto load_tail = [&](Step& st, int kb) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const bool ok = kb + g * kGroup + s * kPiece < K;
      if (s % GW == 0) {
        const bool ok_w = kb + g * kGroup + (s + r / CW) * kPiece < K;
#pragma unroll
        for (int w = 0; w < NW; ++w)
          st.w[w][s / GW] = ok_w ? *(const bf16x8*)(wrow + (int64_t)w * N * K + kb + s * kPiece) : zero;
      }
      if constexpr (MERGE) {
        if (s % GA == 0)
          st.x[0][s / GA] = kb + g * kGroup + (s + r / AR) * kPiece < K ? a_row[(kb + s * kPiece) / 8] : zero;
      } else if constexpr (NORM) {
        const float* rp = a.resid_in + a_off[0] + kb + s * kPiece;
        st.rs[s][0] = ok ? *(const f32x4*)rp : fzero;
        st.rs[s][1] = ok ? *(const f32x4*)(rp + 4) : fzero;
        st.d[s] = ok ? *(const bf16x8*)(dbase + a_off[0] + kb + s * kPiece) : zero;
        const float* np = a.norm_w + g * kGroup + kb + s * kPiece;
        st.nw[s][0] = ok ? *(const f32x4*)np : fzero;
        st.nw[s][1] = ok ? *(const f32x4*)(np + 4) : fzero;
      } else {
        if (s % GA == 0) {
          const bool ok_a = kb + g * kGroup + (s + r / AR) * kPiece < K;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            st.x[mt][s / GA] = ok_a ? *(const bf16x8*)(a.A + a_off[mt] + kb + s * kPiece) : zero;
        }
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
        for (int mt = 0; mt < MT; ++mt) {
          const bf16x8 x = row_down_by(st.x[mt][s / GA], (s % GA) * AR);
#pragma unroll
          for (int w = 0; w < NW; ++w)
            acc[w][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                row_down_by(st.w[w][s / GW], (s % GW) * CW), x, acc[w][mt], 0, 0, 0);
        }
      }
    }
  };

  const int kfull = K / kStep * kStep;
  constexpr int stride = WK * kStep;
  const int kb0 = wk * kStep;
  Step st[PD];
  int kb = kb0;
  if constexpr (MERGE) {
    // The first steps' rows of W are asked for, then every thread merges pieces of eight
    // elements of A (the arithmetic of attention_merge, split by split in groups of
    // eight, so the rows are bit for bit what that kernel would have stored), then the
    // K loop runs with A out of LDS.
#pragma unroll
    for (int p = 0; p < PD; ++p)
      if (kb0 + p * stride < kfull) load(st[p], kb0 + p * stride, true, false);
    const int hd = a.merge_hd, splits = a.merge_splits, grp = a.merge_group;
    const int head_blocks = (grp + 15) / 16;
    const int pieces = K / 8;
    bf16x8* rows = (bf16x8*)merged_rows;
    // U pieces of a thread at a time, the loads of all of them asked for before the first
    // is used (a piece after the other would cost a trip to memory each), in groups of G
    // splits: few splits (decode steps of several rows) take four pieces of up to four
    // splits, many (one or two rows) a piece of eight splits at a time.
    auto merge_pieces = [&](auto group_size, auto at_a_time) {
      constexpr int G = decltype(group_size)::value, U = decltype(at_a_time)::value;
      constexpr int kThreads = WK * kWave;
      for (int idx0 = threadIdx.x; idx0 < M * pieces; idx0 += U * kThreads) {
        int64_t base[U];
        int used[U], d[U];
        float ms[U][G], ls[U][G];
        f32x4 lo4[U][G], hi4[U][G];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int idx = min(idx0 + u * kThreads, M * pieces - 1);     // past the end: the last again
          const int m = idx / pieces, p8 = idx % pieces;
          const int head = p8 * 8 / hd;
          d[u] = p8 * 8 % hd;
          const int kvh = head / grp, hh = head % grp;
          base[u] = ((int64_t)((m * a.merge_nkv + kvh) * head_blocks + hh / 16) * splits) * 16 + hh % 16;
          const int pos = a.merge_pos[m];
          const int lo = a.merge_window > 0 ? max(0, pos - a.merge_window + 1) : 0;
          const int nchunks = pos / a.merge_chunk - lo / a.merge_chunk + 1;
          const int per = (nchunks - 1 + splits) / splits;
          used[u] = min(splits, (nchunks + per - 1) / per);
          // (the first group is asked for without waiting for the position, which says
          // how many splits hold keys at all; an empty one says so itself)
#pragma unroll
          for (int j = 0; j < G; ++j) {
            const int64_t slot = base[u] + (int64_t)min(j, splits - 1) * 16;
            const bool holds = j < splits;
            ms[u][j] = holds ? a.merge_ml[slot * 2] : -INFINITY;
            ls[u][j] = holds ? a.merge_ml[slot * 2 + 1] : 0.f;
            lo4[u][j] = holds ? *(const f32x4*)(a.merge_o + slot * hd + d[u]) : fzero;
            hi4[u][j] = holds ? *(const f32x4*)(a.merge_o + slot * hd + d[u] + 4) : fzero;
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          float mx = -INFINITY, sum = 0.f, o[8] = {};
          for (int s0 = 0; s0 == 0 || s0 < used[u]; s0 += G) {
            if (s0 > 0) {      // later groups only if they hold keys: every workgroup merges all rows
#pragma unroll
              for (int j = 0; j < G; ++j) {
                const int64_t slot = base[u] + (int64_t)min(s0 + j, splits - 1) * 16;
                const bool holds = s0 + j < used[u];
                ms[u][j] = holds ? a.merge_ml[slot * 2] : -INFINITY;
                ls[u][j] = holds ? a.merge_ml[slot * 2 + 1] : 0.f;
                lo4[u][j] = holds ? *(const f32x4*)(a.merge_o + slot * hd + d[u]) : fzero;
                hi4[u][j] = holds ? *(const f32x4*)(a.merge_o + slot * hd + d[u] + 4) : fzero;
              }
            }
            float mg = mx;
#pragma unroll
            for (int j = 0; j < G; ++j) mg = (s0 + j < splits) ? fmaxf(mg, ms[u][j]) : mg;
            if (mg == -INFINITY) continue;
            const float keep = __builtin_amdgcn_exp2f(mx - mg);
            sum *= keep;
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] *= keep;
#pragma unroll
            for (int j = 0; j < G; ++j) {
              const bool live = s0 + j < splits && ms[u][j] != -INFINITY;
              const float w = live ? __builtin_amdgcn_exp2f(ms[u][j] - mg) : 0.f;
              sum += live ? ls[u][j] * w : 0.f;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                o[i] += live ? lo4[u][j][i] * w : 0.f;
                o[4 + i] += live ? hi4[u][j][i] * w : 0.f;
              }
            }
            mx = mg;
          }
          const float inv = sum > 0.f ? 1.f / sum : 0.f;
          bf16x8 out;
#pragma unroll
          for (int i = 0; i < 8; ++i) out[i] = (bf16_t)(o[i] * inv);
          const int idx = idx0 + u * kThreads;
          if (idx < M * pieces) rows[(idx / pieces) * row_pieces + idx % pieces] = out;
        }
      }
    };
    if (splits <= 4) merge_pieces(std::integral_constant<int, 4>{}, std::integral_constant<int, 4>{});
    else merge_pieces(std::integral_constant<int, 8>{}, std::integral_constant<int, 1>{});
    __syncthreads();
#pragma unroll
    for (int p = 0; p < PD; ++p)
      if (kb0 + p * stride < kfull) load(st[p], kb0 + p * stride, false, true);
  } else
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
      for (int i = 0; i < kPartLoads; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          sq += (((i * WK + wk) * 4 + g) * 4 + e < a.parts) ? part[mt][i][e] : 0.f;
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
    const bool n_ok = n < N && g * 4 < CW;   // N is a multiple of 4 here
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
      if (g == 0 && m < M) a.sumsq_out[(int64_t)m * (((int)gridDim.x + 3) & ~3) + blockIdx.x] = sq;
    }
    return;
  }
  if (n >= N || g * 4 >= CW) return;
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
          bool TAIL = false, int CW = 16, int AR = 16>
static inline void launch(const DirectArgs& a, hipStream_t stream) {
  dim3 grid((a.N + CW - 1) / CW, (a.M + MT * 16 - 1) / (MT * 16));
  hipLaunchKernelGGL((gemm_direct_kernel<MT, WK, TC, PAIR, NORM, S, PD, SCALED, TAIL, CW, AR>),
                     grid, dim3(WK * kWave), 0, stream, a);
}

// The merged tail form: dynamic LDS for the rows of A.  Returns false if the device
// refuses that much.
template <int WK, int CW, int AR>
static inline bool launch_merged(const DirectArgs& a, hipStream_t stream) {
  auto kernel = gemm_direct_kernel<1, WK, bf16_t, false, false, 4, 4, false, true, CW, AR, true>;
  const size_t lds = (size_t)AR * (a.K / 8 + 1) * 16;
  static size_t raised = 48 * 1024;      // per instantiation
  if (lds > raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      return false;
    raised = lds;
  }
  hipLaunchKernelGGL(kernel, dim3((a.N + CW - 1) / CW, 1), dim3(WK * kWave), lds, stream, a);
  return true;
}


// Tiles of 16 rows a workgroup holds, columns it owns and rows of A a load instruction is
// packed for: the rules of gemm_direct.hip.
int gemm_direct_row_tiles(int M, int N, int most);
int gemm_direct_columns(int M, int N);
static inline int gemm_direct_packed_rows(int M) { return M <= 4 ? 4 : M <= 8 ? 8 : 16; }

// The forms' dispatchers, one per translation unit.
int gemm_direct_plain(const DirectArgs& a, int c_type, hipStream_t stream);
int gemm_direct_tail(const DirectArgs& a, hipStream_t stream);
int gemm_direct_merged(const DirectArgs& a, hipStream_t stream);
int gemm_direct_scaled(const DirectArgs& a, int c_type, bool pair, hipStream_t stream);
int gemm_direct_pair(const DirectArgs& a, hipStream_t stream);
int gemm_direct_norm(const DirectArgs& a, int c_type, bool pair, hipStream_t stream);

// launch<...> for one tile of rows with the rows of A packed for M (AR) and, where the
// form allows, CW columns per workgroup: the same kernel, fewer load instructions.
#define TS_DIRECT_ROWS(M, ...)                                  \
  switch (gemm_direct_packed_rows(M)) {                         \
    case 4: { constexpr int AR = 4; __VA_ARGS__; } break;       \
    case 8: { constexpr int AR = 8; __VA_ARGS__; } break;       \
    default: { constexpr int AR = 16; __VA_ARGS__; } break;     \
  }
#define TS_DIRECT_COLUMNS(CWV, ...)                             \
  switch (CWV) {                                                \
    case 4: { constexpr int CW = 4; __VA_ARGS__; } break;       \
    case 8: { constexpr int CW = 8; __VA_ARGS__; } break;       \
    default: { constexpr int CW = 16; __VA_ARGS__; } break;     \
  }
