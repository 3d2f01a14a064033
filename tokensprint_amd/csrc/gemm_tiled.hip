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
};

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

template <int BM, int BN, int GM, int GN, int STAGES, bool PAIR, typename TO>
__global__ __launch_bounds__(64 * GM * GN, 1) void gemm_tiled_kernel(TiledArgs g) {
  constexpr int NW = GM * GN;                        // waves: GM along the rows, GN along the columns
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "whole load instructions per operand");
  constexpr int WM = BM / GM, WN = BN / GN;          // a wave's part of the tile
  static_assert(WM % 16 == 0 && WN % (PAIR ? 32 : 16) == 0, "a wave's part in 16 x 16 blocks");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int LA = BM / (8 * NW), LW = BN / (8 * NW);   // load instructions a wave issues per step
  constexpr int LOADS = LA + LW;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  static_assert(STAGES >= 2 && STAGES <= 4, "the waits below are written for 2 to 4 buffers");
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
    for (int kt0 = 0; kt0 < KT; kt0 += STAGES) {
#pragma unroll
      for (int s = 0; s < STAGES; ++s) {
        const int kt = kt0 + s;
        if (kt >= KT) break;
        const int younger = min(STAGES - 2, KT - 1 - kt);
        if (younger >= 2) wait_loads<LOADS * (STAGES >= 4 ? 2 : 0)>();
        else if (younger == 1) wait_loads<LOADS * (STAGES >= 3 ? 1 : 0)>();
        else wait_loads<0>();
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
          const int younger = min(STAGES - 2, KT - 2 - kt);
          if (younger >= 2) wait_loads<LOADS * (STAGES >= 4 ? 2 : 0)>();
          else if (younger == 1) wait_loads<LOADS * (STAGES >= 3 ? 1 : 0)>();
          else wait_loads<0>();
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
  TO* c = (TO*)g.c;
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
          o[e] = gv / (1.f + __expf(-gv)) * uv;
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

template <int BM, int BN, int GM, int GN, int STAGES, bool PAIR, typename TO>
int launch_tiled(TiledArgs g, hipStream_t stream) {
  auto kernel = gemm_tiled_kernel<BM, BN, GM, GN, STAGES, PAIR, TO>;
  constexpr int lds = STAGES * (BM + BN) * 128;
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

template <bool PAIR, typename TO>
int choose_tile(const TiledArgs& g, int tile, hipStream_t stream) {
  if (tile == 0) {
    // the largest tile that still gives most compute units one: a large tile needs fewer
    // bytes from L2 per product, but a tile is one workgroup and a unit without one idles
    const int64_t cols = PAIR ? 2 * (int64_t)g.N : g.N;
    auto tiles = [&](int bm, int bn) { return (int64_t)((g.M + bm - 1) / bm) * ((cols + bn - 1) / bn); };
    const int64_t enough = 160;
    if (tiles(256, 256) >= enough) tile = 4;
    else if (tiles(256, 128) >= enough) tile = 1;
    else if (tiles(128, 128) >= enough) tile = 2;
    else tile = 3;
  }
  switch (tile) {
    case 1: return launch_tiled<256, 128, 4, 2, 3, PAIR, TO>(g, stream);
    case 2: return launch_tiled<128, 128, 2, 4, 4, PAIR, TO>(g, stream);
    case 3: return launch_tiled<128, 64, 4, 2, 4, PAIR, TO>(g, stream);
    case 4: return launch_tiled<256, 256, 2, 4, 2, PAIR, TO>(g, stream);
  }
  TS_FAIL("gemm_tiled: no tile %d", tile);
}

}  // namespace

// 1 if ts_gemm_tiled_bf16 takes these sizes.
extern "C" int ts_gemm_tiled_fits(int M, int N, int K, int pair) {
  const int64_t rows_w = pair ? 2 * (int64_t)N : N;
  return M > 0 && N > 0 && K >= 256 && K % 64 == 0 && N % 16 == 0 &&
         (int64_t)M * K * 2 < (1ll << 32) && rows_w * K * 2 < (1ll << 32);
}

// C[M, N] = A[M, K] W[N, K]^T, or with `pair` C[M, N] = silu(A Wg^T) * (A Wu^T) for
// W = [Wg; Wu] of 2 N rows.  `c_type`: bfloat16 or float32 (float32 not with `pair`).
// `tile`: 0 lets the sizes choose; 1 to 4 name a tile (for measuring; the result is the
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
