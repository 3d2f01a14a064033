// The inner work of the matrix-core attention kernels: operand loads for a block of 32
// keys and the update of one 16-row query tile with that block.
//
// Layouts (v_mfma_f32_16x16x32_bf16, lane = 16*g + r):
//   K operand   lane (r, g) holds K[key blk*16 + r][g*8*KS + s*8 + j]        (A of S^T = K Q^T)
//   Q operand   lane (r, g) holds Q[row r][g*8*KS + s*8 + j]                 (B)
//   S^T result  lane (r, g) holds S^T[key blk*16 + g*4 + t][row r]
//   V operand   lane (r, g) holds V^T[d = db*16 + r][keys blk0: g*4..+3, blk1: g*4..+3]
//               (one 8-element register group per 16 head elements)
//   P operand   lane (r, g) holds its own 8 probabilities, in that key order
// so a lane's scores are, in place, its part of the second product's B operand, and the
// softmax statistics of a query row live in the four lanes r, r+16, r+32, r+48.
//
// PAGE16: the page size is a power of two from 16 up, so a block of 16 keys lies in one page and
// its page id is the same for the whole wave: the ids come out of a register strip of
// the block table by readlane, addresses are scalar plus a lane offset, and all loads
// of a block are independent of each other.  Otherwise every lane looks its page up
// (small test page sizes; slow but the same arithmetic).
#pragma once
#include "attention_mfma.h"

template <int HD>
struct KvBlock {
  static constexpr int KS = (HD + 31) / 32;
  static constexpr int DB = HD / 16;
  bf16x8 k[2][KS];
  bf16x8 v[DB];        // [0..3]: keys of the first 16-key block, [4..7]: of the second
};

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// Reductions over the four lanes r, r+16, r+32, r+48 that share a query row, with the
// gfx950 row-swap instructions (no LDS round trip): v_permlane16_swap exchanges odd rows
// of 16 lanes of one operand with even rows of the other, v_permlane32_swap the upper 32
// lanes of one with the lower 32 of the other; fed the same value twice they return the
// value of each half (pair of rows) in both halves.
//
// max2: the larger of two by the NaN-propagating maximum (v_maximum3_f32, which also
// takes three operands, so two calls in a row are one instruction).  fmaxf would first
// quiet a signalling NaN in each operand, an instruction per operand and call, which
// scores (finite products, or -inf from the mask) do not need.
__device__ __forceinline__ float max2(float a, float b) {
  return __builtin_elementwise_maximum(a, b);
}
__device__ __forceinline__ float col4_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float col4_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Page ids of the coming 32-key block, fetched one block ahead through the scalar cache
// (read-only, wave-uniform addresses), so that neither a wait for vector loads nor an
// address dependency stands between a block's loads.
typedef const int __attribute__((address_space(4))) * ConstTable;

struct PageCursor {
  ConstTable table;   // block table row of the entry
  int page_size;      // with PAGE16 a power of two >= 16
  int last_key;
  int next0, next1;   // page ids of the two 16-key blocks of the next call (two
                      // scalars: an array indexed at run time would live in memory)
  __device__ __forceinline__ int fetch(int k0) const {          // k0 is wave-uniform
    return k0 <= last_key ? table[k0 >> (__builtin_ctz(page_size))] : -1;
  }
  __device__ __forceinline__ void start(int kb) {
    next0 = fetch(kb);
    next1 = fetch(kb + 16);
  }
};

// Loads the K and V operands of keys [kb, kb + 32).  With PAGE16 calls must come in
// steps of `stride` keys from the cursor's start (the cursor holds this call's pages and
// then fetches those of kb + stride).
template <int HD, bool PAGE16>
__device__ __forceinline__ void load_kv_block(KvBlock<HD>& b, const AttentionArgs& a,
                                              const int* table, PageCursor& cur, int kvh,
                                              int kb, int stride, int r, int g) {
  constexpr int KS = KvBlock<HD>::KS, DB = KvBlock<HD>::DB;
  const bf16_t* kp = (const bf16_t*)a.k_pages;
  const bf16_t* vp = (const bf16_t*)a.v_pages;
  const int P = a.page_size;
  const int last_key = cur.last_key;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16x4 zero4 = {0, 0, 0, 0};
  bf16x4 vh[2][DB];
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    const int k0 = kb + blk * 16;                        // first key of the 16-key block
    if (PAGE16) {
      const int page = blk ? cur.next1 : cur.next0;      // scalar
      if (page >= 0) {
        const int off = k0 & (P - 1);
        const bf16_t* krow = kp + (((int64_t)page * a.nkv + kvh) * P + off + r) * HD;
        const bf16_t* vcol = vp + ((int64_t)page * a.nkv + kvh) * HD * P + off + g * 4;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const int e = g * 8 * KS + s * 8;
          b.k[blk][s] = (KS * 32 == HD || e < HD) ? *(const bf16x8*)(krow + e) : zero8;
        }
#pragma unroll
        for (int db = 0; db < DB; ++db)
          vh[blk][db] = *(const bf16x4*)(vcol + (int64_t)(db * 16 + r) * P);
      } else {
#pragma unroll
        for (int s = 0; s < KS; ++s) b.k[blk][s] = zero8;
#pragma unroll
        for (int db = 0; db < DB; ++db) vh[blk][db] = zero4;
      }
    } else {
      const int key = k0 + r;
      const int kpage = key <= last_key ? table[key / P] : -1;
      const bf16_t* krow = kp + (((int64_t)max(kpage, 0) * a.nkv + kvh) * P + key % P) * HD;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int e = g * 8 * KS + s * 8;
        b.k[blk][s] = (kpage >= 0 && e < HD) ? *(const bf16x8*)(krow + e) : zero8;
      }
      const int key4 = k0 + g * 4;
      const int vpage = key4 <= last_key ? table[key4 / P] : -1;
      const bf16_t* vcol = vp + ((int64_t)max(vpage, 0) * a.nkv + kvh) * HD * P + key4 % P;
#pragma unroll
      for (int db = 0; db < DB; ++db)
        vh[blk][db] = vpage >= 0 ? *(const bf16x4*)(vcol + (int64_t)(db * 16 + r) * P) : zero4;
    }
  }
#pragma unroll
  for (int db = 0; db < DB; ++db)
    b.v[db] = __builtin_shufflevector(vh[0][db], vh[1][db], 0, 1, 2, 3, 4, 5, 6, 7);
  if (PAGE16) cur.start(kb + stride);
}

// The same block with its keys assigned to the rows of the two score products so that lane
// (r, g) holds the scores of keys g * 8 .. g * 8 + 7 of the block (row i of product b is
// key (i / 4) * 8 + b * 4 + i % 4; tile_update's PERM): the lane's share of V^T[d] is then
// one 16-byte run of a page's row instead of two 8-byte ones, and a block costs a third
// fewer load instructions, which is what a compute unit's rate of taking them makes a
// short walk cost.  Page sizes that are powers of two from 16 up; calls in steps of
// `stride` keys from the cursor's start.
template <int HD>
__device__ __forceinline__ void load_kv_block_wide(KvBlock<HD>& b, const AttentionArgs& a,
                                                   PageCursor& cur, int kvh, int kb, int stride,
                                                   int r, int g) {
  constexpr int KS = KvBlock<HD>::KS, DB = KvBlock<HD>::DB;
  static_assert(HD % 32 == 0, "whole 32-element slices");
  const bf16_t* kp = (const bf16_t*)a.k_pages;
  const bf16_t* vp = (const bf16_t*)a.v_pages;
  const int P = a.page_size;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int page0 = cur.next0, page1 = cur.next1;          // of the block's two 16-key halves
  const int in0 = kb & (P - 1), in1 = (kb + 16) & (P - 1);
  // scalar: where the halves' key rows and value columns of this head begin
  const int64_t h0 = ((int64_t)max(page0, 0) * a.nkv + kvh) * P, h1 = ((int64_t)max(page1, 0) * a.nkv + kvh) * P;
  const bf16_t* k0 = kp + (h0 + in0) * HD;
  const bf16_t* k1 = kp + (h1 + in1) * HD;
  const bf16_t* v0 = vp + h0 * HD + in0;
  const bf16_t* v1 = vp + h1 * HD + in1;
  const bool k_second = r >= 8, v_second = g >= 2;         // which half this lane's keys lie in
  // keys: rows (r / 4) * 8 + r % 4 (product 0) and four further (product 1) of the block,
  // i.e. row (r % 8 / 4) * 8 + r % 4 [+ 4] of the lane's half
  const bf16_t* krow = (k_second ? k1 : k0) + (((r % 8) / 4) * 8 + r % 4) * HD + g * 8 * KS;
  const bf16_t* vcol = (v_second ? v1 : v0) + (int64_t)r * P + (g % 2) * 8;
#pragma unroll
  for (int blk = 0; blk < 2; ++blk)
#pragma unroll
    for (int s = 0; s < KS; ++s) b.k[blk][s] = *(const bf16x8*)(krow + blk * 4 * HD + s * 8);
#pragma unroll
  for (int db = 0; db < DB; ++db) b.v[db] = *(const bf16x8*)(vcol + (int64_t)db * 16 * P);
  if (page0 < 0 || page1 < 0) {      // scalar: only where the context ends or a window has let go
    const bool k_ok = (k_second ? page1 : page0) >= 0, v_ok = (v_second ? page1 : page0) >= 0;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int s = 0; s < KS; ++s) b.k[blk][s] = k_ok ? b.k[blk][s] : zero8;
#pragma unroll
    for (int db = 0; db < DB; ++db) b.v[db] = v_ok ? b.v[db] : zero8;
  }
  cur.start(kb + stride);
}

// One query tile's running state.
template <int HD>
struct TileState {
  static constexpr int KS = (HD + 31) / 32;
  static constexpr int DB = HD / 16;
  bf16x8 q[KS];
  f32x4 o[DB];
  float m, l;         // l: this lane's share of the row's sum of weights (row_sum adds the four)
  int pos, lo;        // this lane's row: position and first visible key (pos = -1: no row)
};

// The sum of weights of a lane's query row: the shares of the four lanes that hold the row.
template <int HD>
__device__ __forceinline__ float row_sum(const TileState<HD>& t) { return col4_sum(t.l); }

template <int HD>
__device__ __forceinline__ void load_query(TileState<HD>& t, const bf16_t* qrow, bool row_ok,
                                           int g) {
  constexpr int KS = TileState<HD>::KS;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int e = g * 8 * KS + s * 8;
    t.q[s] = (row_ok && e < HD) ? *(const bf16x8*)(qrow + e) : zero8;
  }
#pragma unroll
  for (int db = 0; db < TileState<HD>::DB; ++db) t.o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  t.m = -INFINITY;
  t.l = 0.f;
}

// Scores of the block for one tile, masked softmax update, and O^T += V^T P^T.
// `interior` (wave-uniform): every key of the block is visible to every row of the tile,
// so the mask is skipped: by a branch around it, the rest is one stretch of code either
// way.  scale_log2 = softmax scale * log2(e); m is kept in that unit.  A row that has
// seen no key yet has m = -inf; the exponentials take a finite stand-in for it, which
// makes all of them 0 without a special case.
//
// LAZY: the sums so far are rescaled only if some row of the tile met a new largest score
// (a wave-uniform branch).  Far into a long context most blocks bring none.  For kernels
// whose loads of the next block are in flight across this call the branch costs more
// than it saves (the waits at its join are for all of them).
//
// PERM: the keys of the block are assigned to the rows of the two score products so that
// lane (r, g) holds the scores of keys g * 8 .. g * 8 + 7 (row i of product b is key
// (i / 4) * 8 + b * 4 + i % 4) instead of keys g * 4 .. + 3 of each 16-key half.
template <int HD, bool LAZY = false, bool PERM = false>
__device__ __forceinline__ void tile_update(TileState<HD>& t, const KvBlock<HD>& b, int kb,
                                            float scale_log2, bool interior, int g) {
  constexpr int KS = TileState<HD>::KS, DB = TileState<HD>::DB;
  f32x4 st[2];
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    st[blk] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
      st[blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.k[blk][s], t.q[s], st[blk], 0, 0, 0);
  }
  if (!interior) {
    asm volatile("" ::: "memory");   // keeps this a branch: blended in, it costs every block
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = PERM ? kb + g * 8 + blk * 4 + i : kb + blk * 16 + g * 4 + i;
        st[blk][i] = (key <= t.pos && key >= t.lo) ? st[blk][i] : -INFINITY;
      }
  }
  const float mx = max2(max2(max2(max2(st[0][0], st[0][1]), st[0][2]),
                             max2(max2(st[0][3], st[1][0]), st[1][1])),
                        max2(st[1][2], st[1][3]));
  // the scale is positive: the largest score stays the largest
  const float m_new = max2(t.m, col4_max(mx) * scale_log2);
  const float m_use = max2(m_new, -1e30f);
  const float corr = __builtin_amdgcn_exp2f(t.m - m_use);
  float ps;
  bf16x8 pv;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[i / 4][i % 4], scale_log2, -m_use));
    ps = i ? ps + p : p;
    pv[i] = (bf16_t)p;
  }
  // the correction is the same in the four lanes of a row, so each lane keeps the sum of
  // its own keys and the four are added once, at the end
  t.l = t.l * corr + ps;
  t.m = m_new;
  if (!LAZY || __builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) t.o[db][i] *= corr;
  }
#pragma unroll
  for (int db = 0; db < DB; ++db)
    t.o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.v[db], pv, t.o[db], 0, 0, 0);
}

template <int HD>
__device__ __forceinline__ void store_tile(const TileState<HD>& t, float sum, bf16_t* out,
                                           int g) {
  const float inv = sum > 0.f ? 1.f / sum : 0.f;
#pragma unroll
  for (int db = 0; db < TileState<HD>::DB; ++db) {
    bf16x4 ov = {(bf16_t)(t.o[db][0] * inv), (bf16_t)(t.o[db][1] * inv),
                 (bf16_t)(t.o[db][2] * inv), (bf16_t)(t.o[db][3] * inv)};
    *(bf16x4*)(out + db * 16 + g * 4) = ov;
  }
}
