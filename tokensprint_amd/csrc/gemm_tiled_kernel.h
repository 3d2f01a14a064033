// Matrix products of many rows (portions of prompts): C[M, N] = A[M, K] W[N, K]^T in
// bfloat16 with float32 sums, tiled through LDS for the matrix cores of gfx950.
//
// A workgroup of eight waves (two to a SIMD: one wave alone cannot keep a matrix core
// busy, its instructions issue at two thirds of the core's rate) owns a BM x BN tile of C
// and walks K in steps of 64.  Both
// operands are contiguous along K, which is also how a matrix-core instruction wants
// them (a lane holds eight consecutive k of one row), so a step's slab of A (BM rows of
// 128 bytes) and of W (BN rows) goes from global memory straight into LDS by
// `global_load_lds_dwordx4`, 16 bytes a lane, without passing through registers, several
// steps ahead in a ring of buffers; the waves count their own loads (s_waitcnt vmcnt),
// and one workgroup barrier a step separates the loads' arrival from the reads and the
// reads from the next overwrite.  A row's eight 16-byte pieces are stored in LDS at
// position (piece ^ (row / 2 % 8)), which makes the sixteen rows that a quarter wave reads
// together fall into different banks; since a direct load writes lane l's piece to slot
// l, the permutation is applied on the global side (which piece a lane fetches).
//
// The product is computed as C^T = W A^T (W's rows are the instruction's first operand),
// so a lane ends up with four consecutive columns of one row of C and stores them as one
// piece.  With PAIR, W is [2, N, K] (gate rows, then up rows): a tile holds BN/2 columns
// of each, interleaved per wave, and the epilogue writes silu(gate) * up.
//
// K is summed in index order by one accumulator per element whatever the tile size, so
// the choice of tile changes no bit of the result.
//
// Two further forms put the residual add and the RMSNorm of a prompt's step into the
// products around them, as the weight-streaming kernels do for few rows.  TAIL (the
// product that ends a sub-layer): stream += bfloat16(A W^T) in float32 in place, and the
// stream is handed on as `prepared` = bfloat16(stream * norm weight), not yet divided by
// the row's root mean square, with the rows' sums of squares in slices of 32 columns
// (`sumsq_out` [N / 32, M]; a slice is added up in the same order whatever the tile).
// SCALED (the product behind that norm): A is such prepared rows, and the epilogue
// multiplies row m by rsqrt(sum of its slices / K + eps), which a workgroup works out for
// its BM rows before it sends for its first operands.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gemm_common.h"

namespace {

struct TiledArgs {
  const bf16_t* a;
  const bf16_t* w;
  void* c;
  int M, N, K;          // N: columns of C (with PAIR: of each half of W)
  int tiles_m, tiles_n;
  int groups_n;         // the tile grid is cut into 8 regions, 8 / groups_n by groups_n
  // SCALED: the sums of squares of A's rows [parts, M]
  const float* sumsq_in;
  int parts;
  float eps;
  // TAIL: the float32 stream [M, N] (read and written), the norm's weight [N], what is
  // handed on [M, N], the sums of squares of the new stream's rows [N / 32, M]
  float* resid;
  const float* norm_w;
  bf16_t* prepared;
  float* sumsq_out;
};

constexpr int kPlain = 0, kScaled = 1, kTail = 2;
constexpr int kSliceColumns = 32;   // columns per slice of a row's sum of squares (TAIL)

// One 16-byte piece per lane from global memory (uniform base + per-lane byte offset)
// into LDS at `lds` + 16 * lane.
__device__ __forceinline__ void dma16(const void* base, unsigned offset, unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(offset), "s"(base), "s"(lds)
               : "memory", "m0");
}

template <int N>                                          // N: loads that may still be in flight
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "the load counter has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// Waits until at most the loads of `younger` K steps (of LOADS each; at most MOST steps)
// are in flight.
template <int LOADS, int MOST>
__device__ __forceinline__ void wait_steps(int younger) {
  if constexpr (MOST <= 0) {
    wait_loads<0>();
  } else {
    if (younger >= MOST) wait_loads<LOADS * MOST>();
    else wait_steps<LOADS, MOST - 1>(younger);
  }
}

template <int BM, int BN, int GM, int GN, int STAGES, bool PAIR, typename TO, int FORM = kPlain>
__global__ __launch_bounds__(64 * GM * GN, 1) void gemm_tiled_kernel(TiledArgs g) {
  static_assert(!(FORM == kTail && PAIR), "the product that ends a sub-layer has one weight");
  constexpr int NW = GM * GN;                        // waves: GM along the rows, GN along the columns
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "whole load instructions per operand");
  constexpr int WM = BM / GM, WN = BN / GN;          // a wave's part of the tile
  static_assert(WM % 16 == 0 && WN % (PAIR ? 32 : 16) == 0, "a wave's part in 16 x 16 blocks");
  constexpr int TM = WM / 16, TN = WN / 16;
  static_assert(FORM != kTail || WN % kSliceColumns == 0, "a wave holds whole slices of a row");
  constexpr int LA = BM / (8 * NW), LW = BN / (8 * NW);   // load instructions a wave issues per step
  constexpr int LOADS = LA + LW;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  static_assert(STAGES >= 2 && STAGES <= 8, "a ring of 2 to 8 buffers");
  static_assert(LOADS * (STAGES - 1) < 64, "the load counter has six bits");
  extern __shared__ __attribute__((aligned(1024))) unsigned char tiled_lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, gq = lane >> 4;
  const int wm = wave / GN, wn = wave % GN;

  // Which tile: workgroups go round the 8 XCDs by their index, each XCD has an L2 of its
  // own, so each XCD gets a compact region of the tile grid (its workgroups share rows of
  // A and W), walked row by row.
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int groups_m = 8 / g.groups_n;
  const int region_m = (g.tiles_m + groups_m - 1) / groups_m;
  const int region_n = (g.tiles_n + g.groups_n - 1) / g.groups_n;
  const int tile_m = (xcd / g.groups_n) * region_m + local / region_n;
  const int tile_n = (xcd % g.groups_n) * region_n + local % region_n;
  if (local >= region_m * region_n || tile_m >= g.tiles_m || tile_n >= g.tiles_n) return;
  const int m0 = tile_m * BM;

  // SCALED: the factors of this tile's rows.  Called once the first direct loads are on
  // their way and before the K loop counts loads: these loads are waited for with all
  // those before them, which the first turn needs anyway.  A row's slices are asked for
  // 32 at a time and added in their order.
  float* row_scale = (float*)(tiled_lds + STAGES * ((BM + BN) * 128));
  auto row_scales = [&]() {
    if constexpr (FORM == kScaled) {
      for (int row = threadIdx.x; row < BM; row += 64 * NW) {
        const int m = min(m0 + row, g.M - 1);
        float sq = 0.f;
        for (int p0 = 0; p0 < g.parts; p0 += 32) {
          float part[32];
#pragma unroll
          for (int i = 0; i < 32; ++i)
            part[i] = g.sumsq_in[(int64_t)min(p0 + i, g.parts - 1) * g.M + m];
#pragma unroll
          for (int i = 0; i < 32; ++i) sq += p0 + i < g.parts ? part[i] : 0.f;
        }
        row_scale[row] = rsqrtf(sq / (float)g.K + g.eps);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
  };

  // TAIL with a small part of the tile per wave: the stream's values and the norm's
  // weights are asked for now (before every direct load, so that the waits that count
  // those see them gone first) and wait in registers for the epilogue
  constexpr bool kEarlyStream = FORM == kTail && TM * TN <= 16;
  f32x4 early_x[kEarlyStream ? TN : 1][kEarlyStream ? TM : 1], early_w[kEarlyStream ? TN : 1];
  if constexpr (kEarlyStream) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int n = min(tile_n * BN + wn * WN + tn * 16 + gq * 4, g.N - 4);
      early_w[tn] = *(const f32x4*)(g.norm_w + n);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const int m = min(m0 + wm * WM + tm * 16 + r, g.M - 1);
        early_x[tn][tm] = *(const f32x4*)(g.resid + (int64_t)m * g.N + n);
      }
    }
  }

  // column of W (row of the stacked weight) that LDS row `j` of the W slab holds
  auto w_row = [&](int j) {
    if constexpr (PAIR) {
      const int half = j / WN, in = j % WN;           // which wave column, where in it
      const int col = tile_n * (BN / 2) + half * (WN / 2) + in % (WN / 2);
      return min(col, g.N - 1) + (in >= WN / 2 ? g.N : 0);
    } else {
      return min(tile_n * BN + j, g.N - 1);
    }
  };

  // per-lane byte offsets of this wave's loads: instruction i covers LDS rows
  // (NW i + wave) * 8 .. + 7 of the slab, lane l the piece at slot l % 8 of row l / 8
  unsigned off_a[LA], off_w[LW];
  const unsigned row_bytes = (unsigned)g.K * 2;
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    const int row = (NW * i + wave) * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((row >> 1) & 7);
    off_a[i] = (unsigned)min(m0 + row, g.M - 1) * row_bytes + piece * 16;
  }
#pragma unroll
  for (int i = 0; i < LW; ++i) {
    const int row = (NW * i + wave) * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((row >> 1) & 7);
    off_w[i] = (unsigned)w_row(row) * row_bytes + piece * 16;
  }
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)tiled_lds;

  // load instruction i of this wave for K step kt into ring buffer `stage`
  auto issue_one = [&](int stage, int kt, int i) {
    const unsigned dst = lds0 + stage * STAGE_BYTES + wave * 1024;
    if (i < LA) dma16((const char*)g.a + (int64_t)kt * 128, off_a[i], dst + i * NW * 1024);
    else dma16((const char*)g.w + (int64_t)kt * 128, off_w[i - LA], dst + BM * 128 + (i - LA) * NW * 1024);
  };

  f32x4 acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = f32x4{0.f, 0.f, 0.f, 0.f};

  // a lane's reads: row r of a 16-row block, the piece that holds k = 32 ks + 8 gq ..
  const int swz = (r >> 1) & 7;
  const int read0 = r * 128 + ((gq ^ swz) << 4), read1 = r * 128 + (((4 + gq) ^ swz) << 4);

  struct Frags {
    bf16x8 a[TM], w[TN];
  };
  auto read = [&](Frags& f, int stage, int ks) {
    const unsigned char* slab = tiled_lds + stage * STAGE_BYTES;
    const unsigned char* sa = slab + wm * WM * 128 + (ks ? read1 : read0);
    const unsigned char* sw = slab + (BM + wn * WN) * 128 + (ks ? read1 : read0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) f.w[tn] = *(const bf16x8*)(sw + tn * 2048);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) f.a[tm] = *(const bf16x8*)(sa + tm * 2048);
  };
  // the products of one K step of 32; with `load` the wave's loads for K step `kt` are
  // issued between them, so that neither the matrix cores nor the loads' issue wait
  auto mma = [&](const Frags& f, auto with_loads, int stage, int kt) {
    constexpr bool load = decltype(with_loads)::value;
    constexpr int EVERY = (TN * TM) / LOADS > 0 ? (TN * TM) / LOADS : 1;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.w[tn], f.a[tm], acc[tn][tm], 0, 0, 0);
        const int idx = tn * TM + tm;
        if constexpr (load) {
          if (idx % EVERY == 0 && idx / EVERY < LOADS) issue_one(stage, kt, idx / EVERY);
        }
      }
    if constexpr (load) {
#pragma unroll
      for (int i = (TN * TM + EVERY - 1) / EVERY; i < LOADS; ++i) issue_one(stage, kt, i);
    }
  };

  // The ring: K step kt lives in buffer kt % STAGES.  A turn multiplies step kt's first
  // half while its second half comes out of LDS, then (after the barrier that says step
  // kt + 1 has arrived and step kt has been read by everyone) its second half while the
  // first half of step kt + 1 comes out of LDS and the loads of step kt + STAGES go out
  // into the buffer that step kt has left.
  const int KT = g.K / 64;                              // at least STAGES (the launcher's check)
  if constexpr (TM * TN > 16) {
    // A wave's part is too large to hold two K steps' operands beside its sums: the
    // column operands of a K step of 32 are read first, the row operands one ahead of
    // their products, and a turn is: step kt has arrived and step kt - 1 has been read by
    // everyone (barrier); multiply step kt while the loads of step kt + STAGES - 1 go out
    // into the buffer that step kt - 1 has left.  Two waves share a SIMD and fill each
    // other's waits.
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
#pragma unroll
      for (int i = 0; i < LOADS; ++i) issue_one(s, s, i);
    row_scales();
    for (int kt0 = 0; kt0 < KT; kt0 += STAGES) {
#pragma unroll
      for (int s = 0; s < STAGES; ++s) {
        const int kt = kt0 + s;
        if (kt >= KT) break;
        wait_steps<LOADS, STAGES - 2>(min(STAGES - 2, KT - 1 - kt));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const bool load = kt + STAGES - 1 < KT;
        const unsigned char* slab = tiled_lds + s * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const unsigned char* sa = slab + wm * WM * 128 + (ks ? read1 : read0);
          const unsigned char* sw = slab + (BM + wn * WN) * 128 + (ks ? read1 : read0);
          bf16x8 fw[TN], fa = *(const bf16x8*)sa, fb;
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) fw[tn] = *(const bf16x8*)(sw + tn * 2048);
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) {
            if (tm + 1 < TM) fb = *(const bf16x8*)(sa + (tm + 1) * 2048);
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
              acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[tn], fa, acc[tn][tm], 0, 0, 0);
            fa = fb;
            constexpr int PER = (LOADS + 2 * TM - 1) / (2 * TM);      // loads per row block
            if (load) {
#pragma unroll
              for (int j = 0; j < PER; ++j) {
                const int i = (ks * TM + tm) * PER + j;
                if (i < LOADS) issue_one((s + STAGES - 1) % STAGES, kt + STAGES - 1, i);
              }
            }
          }
        }
      }
    }
  } else {
#pragma unroll
  for (int s = 0; s < STAGES; ++s)
#pragma unroll
    for (int i = 0; i < LOADS; ++i) issue_one(s, s, i);
  row_scales();
  wait_loads<LOADS * (STAGES - 1)>();
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  Frags f0, f1;
  read(f0, 0, 0);
  for (int kt0 = 0; kt0 < KT; kt0 += STAGES) {
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
      const int kt = kt0 + s;
      if (kt < KT) {
        read(f1, s, 1);
        mma(f0, std::false_type{}, 0, 0);
        const bool more = kt + 1 < KT;
        if (more) {
          // step kt + 1 has arrived when at most the younger steps' loads are in flight
          wait_steps<LOADS, STAGES - 2>(min(STAGES - 2, KT - 2 - kt));
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // this wave has read step kt
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
          read(f0, (s + 1) % STAGES, 0);
        }
        if (kt + STAGES < KT) mma(f1, std::true_type{}, s, kt + STAGES);
        else mma(f1, std::false_type{}, 0, 0);
      }
    }
  }
  }

  // acc[tn][tm][e] = C[m0 + wm WM + 16 tm + r][column block tn, column 4 gq + e]
  if constexpr (FORM == kTail) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int m = m0 + wm * WM + tm * 16 + r;
#pragma unroll
      for (int p = 0; p < TN / 2; ++p) {
        // a slice of 32 columns: this lane's four columns of the first block of sixteen in
        // order, those of the second, then the four lanes that share the row
        const int n_slice = tile_n * BN + wn * WN + p * kSliceColumns;
        const bool ok = m < g.M && n_slice < g.N;       // N is a multiple of 32 here
        float sq = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int n = n_slice + h * 16 + gq * 4;
          if (ok) {
            const int64_t at = (int64_t)m * g.N + n;
            f32x4 x, w4;
            if constexpr (kEarlyStream) {
              x = early_x[2 * p + h][tm];
              w4 = early_w[2 * p + h];
            } else {
              x = *(const f32x4*)(g.resid + at);
              w4 = *(const f32x4*)(g.norm_w + n);
            }
            bf16x4_t handed;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              // the product rounded to the activation type first, as the unfused path stores it
              x[e] += (float)(bf16_t)acc[2 * p + h][tm][e];
              sq += x[e] * x[e];
              handed[e] = (bf16_t)(x[e] * w4[e]);
            }
            *(f32x4*)(g.resid + at) = x;
            *(bf16x4_t*)(g.prepared + at) = handed;
          }
        }
        sq += __shfl_xor(sq, 16, 64);
        sq += __shfl_xor(sq, 32, 64);
        if (ok && gq == 0) g.sumsq_out[(int64_t)(n_slice / kSliceColumns) * g.M + m] = sq;
      }
    }
    return;
  }
  TO* c = (TO*)g.c;
  if constexpr (FORM == kScaled) {
    // (the barriers of the K loop lie between the factors' writes and these reads)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const float scale = row_scale[wm * WM + tm * 16 + r];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[tn][tm][e] *= scale;
    }
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int m = m0 + wm * WM + tm * 16 + r;
    if (m >= g.M) continue;
    if constexpr (PAIR) {
#pragma unroll
      for (int tn = 0; tn < TN / 2; ++tn) {
        const int n = tile_n * (BN / 2) + wn * (WN / 2) + tn * 16 + gq * 4;
        if (n >= g.N) continue;
        const f32x4 gate = acc[tn][tm], up = acc[tn + TN / 2][tm];
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // as the separate kernel does it: the product rounded to the activation type first
          const float gv = (float)(TO)gate[e], uv = (float)(TO)up[e];
          // 64 values a lane at the very end of the kernel, the matrix cores idle: the
          // hardware's exp2 and reciprocal (an ulp each) instead of a division's ten steps
          o[e] = gv * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(gv * -1.44269504f)) * uv;
        }
        store4<TO>(c + (int64_t)m * g.N + n, o, g.N - n);
      }
    } else {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const int n = tile_n * BN + wn * WN + tn * 16 + gq * 4;
        if (n >= g.N) continue;
        store4<TO>(c + (int64_t)m * g.N + n, acc[tn][tm], g.N - n);
      }
    }
  }
}

template <int BM, int BN, int GM, int GN, int STAGES, bool PAIR, typename TO, int FORM>
int launch_tiled(TiledArgs g, hipStream_t stream) {
  auto kernel = gemm_tiled_kernel<BM, BN, GM, GN, STAGES, PAIR, TO, FORM>;
  constexpr int lds = STAGES * (BM + BN) * 128 + (FORM == kScaled ? BM * 4 : 0);
  static_assert(lds <= 160 * 1024, "LDS of a compute unit");
  static bool raised[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64)
    TS_FAIL("gemm_tiled: no current device below 64");
  if (!raised[device]) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) !=
        hipSuccess)
      TS_FAIL("gemm_tiled: %d bytes of LDS refused", lds);
    raised[device] = true;
  }
  if (g.K / 64 < STAGES) TS_FAIL("gemm_tiled: K=%d is too short for %d buffers", g.K, STAGES);
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + (PAIR ? BN / 2 : BN) - 1) / (PAIR ? BN / 2 : BN);
  // regions of the tile grid, one per XCD: the cut that brings the fewest bytes of A and W
  // into an L2
  int best = 1;
  int64_t best_cost = -1;
  for (int gn = 1; gn <= 8; gn *= 2) {
    const int gm = 8 / gn;
    const int64_t rm = (g.tiles_m + gm - 1) / gm, rn = (g.tiles_n + gn - 1) / gn;
    const int64_t cost = rm * BM + rn * BN;
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = gn; }
  }
  g.groups_n = best;
  const int gm = 8 / best;
  const int region = ((g.tiles_m + gm - 1) / gm) * ((g.tiles_n + best - 1) / best);
  hipLaunchKernelGGL(kernel, dim3(8 * region), dim3(64 * GM * GN), lds, stream, g);
  TS_CHECK_LAUNCH("gemm_tiled");
  return 0;
}

// The tile that a product of these sizes takes when the caller names none: the one with
// the smallest estimate of rounds x time of a tile, a round being one tile on every
// compute unit.  A tile's time is a fixed part (launch, first loads, epilogue and the
// stores' way to memory; the SiLU of the paired form on top) and a part per K step of 64,
// both measured on an MI355X at 512 to 8,192 rows with the weights of the 0.6B shape
// (N 1,024 to 6,144, K 1,024 to 3,072): a large tile needs fewer bytes from L2 per
// product and its steps are bound by the matrix cores (1.2 us for 256 x 256), a small
// one's by the rate at which a unit takes direct loads (0.28 us for 128 x 64, 2.3 times
// the matrix cores' time), but a tile is one workgroup and a unit without one idles.
struct TileCost {
  int tile, bm, bn;
  float fixed_us, step_us, pair_us;
};
constexpr TileCost kTileCosts[] = {
    {3, 128, 64, 4.4f, 0.275f, 1.f}, {2, 128, 128, 6.3f, 0.39f, 1.5f}, {1, 256, 128, 7.8f, 0.66f, 2.f},
    {5, 256, 192, 8.f, 1.1f, 3.f},   {4, 256, 256, 7.f, 1.19f, 4.f},
};

inline int cheapest_tile(const TiledArgs& g, bool pair) {
  static int units[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 3;
  if (units[device] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0)
      n = 256;
    units[device] = n;
  }
  const int64_t cols = pair ? 2 * (int64_t)g.N : g.N;
  int best = 3;
  float best_us = -1.f;
  for (const TileCost& t : kTileCosts) {
    const int64_t tiles = (int64_t)((g.M + t.bm - 1) / t.bm) * ((cols + t.bn - 1) / t.bn);
    const int64_t rounds = (tiles + units[device] - 1) / units[device];
    const float us = rounds * (t.fixed_us + (pair ? t.pair_us : 0.f) + t.step_us * (g.K / 64));
    if (best_us < 0.f || us < best_us) { best_us = us; best = t.tile; }
  }
  return best;
}

template <bool PAIR, typename TO, int FORM = kPlain>
int choose_tile(const TiledArgs& g, int tile, hipStream_t stream) {
  if (tile == 0) tile = cheapest_tile(g, PAIR);
  switch (tile) {
    case 1: return launch_tiled<256, 128, 4, 2, 3, PAIR, TO, FORM>(g, stream);
    case 2: return launch_tiled<128, 128, 2, 4, 4, PAIR, TO, FORM>(g, stream);
    case 3: return launch_tiled<128, 64, 4, 2, 4, PAIR, TO, FORM>(g, stream);
    case 4: return launch_tiled<256, 256, 2, 4, 2, PAIR, TO, FORM>(g, stream);
    case 5: return launch_tiled<256, 192, 4, 2, 2, PAIR, TO, FORM>(g, stream);
  }
  TS_FAIL("gemm_tiled: no tile %d", tile);
}

}  // namespace
