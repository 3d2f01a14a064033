// Paged causal attention on the matrix cores for bfloat16: decode tokens and portions
// of prompts in one launch, any head grouping, head sizes in steps of 16 up to 256.
//
// One wavefront owns a tile of 16 query rows: up to 16 query heads of one key/value
// head for 16/rows_per_token consecutive tokens of one batch entry (a decode token
// gives one token per tile).  Everything is computed transposed,
//     S^T = K Q^T          (v_mfma_f32_16x16x32_bf16, reduction over the head size)
//     O^T = V^T P^T        (reduction over 32 keys)
// so that a lane holds one query's scores for 8 of the 32 keys: these 8 numbers are,
// in place, the B operand of the second product, and the softmax statistics of a query
// live in the four lanes that share its column.  K rows (contiguous along the head
// size) and V columns (contiguous along positions, the cache stores values transposed
// inside a page) are both read from global memory in operand layout: no LDS, no
// transposes.  The key range of a tile is cut into chunks of kChunk keys at fixed
// positions; a launch either lets a wave walk all its chunks or spreads them over
// `num_splits` waves whose partial results a second kernel merges.
#include "attention_core.h"

// COOP = false: a wavefront per item walks its keys alone.
// COOP = true: a workgroup per item; its four waves take every fourth 32-key block and
// merge in LDS (few tiles: decode), so a short context costs one round of loads.
template <int HD, bool COOP, bool PAGE16>
__global__ __launch_bounds__(256, HD <= 128 ? 2 : 1) void attention_mfma_kernel(AttentionMfmaArgs args) {
  constexpr int DB = HD / 16;
  const AttentionArgs& a = args.base;
  const int wave = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int items = args.num_tiles * a.nkv * args.head_blocks;
  const int item = COOP ? blockIdx.x : blockIdx.x * 4 + wave;
  if (item >= items) return;
  const int tile = item / (a.nkv * args.head_blocks);
  const int kvh = (item / args.head_blocks) % a.nkv;
  const int hb = item % args.head_blocks;
  const int split = blockIdx.y;
  // without a tile list every entry brings one token (a decode step): tile = entry = token
  const int entry = args.tiles ? uniform(args.tiles[tile * 3]) : tile,
            tok0 = args.tiles ? uniform(args.tiles[tile * 3 + 1]) : tile,
            ntok = args.tiles ? uniform(args.tiles[tile * 3 + 2]) : 1;
  const int* table = a.table + (int64_t)entry * a.table_width;

  // my query row: column r of S^T
  const int ti = r / args.rows_per_token;
  const int hh = hb * 16 + r % args.rows_per_token;          // head inside the group
  const bool row_ok = ti < ntok && hh < group;
  const int token = tok0 + min(ti, ntok - 1);
  const int head = kvh * group + min(hh, group - 1);

  // key range of the tile and my share of its chunks
  const int pos_first = uniform(a.positions[tok0]);           // positions are consecutive
  const int pos_last = pos_first + ntok - 1;
  const int lo_tile = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;
  const int c_first = lo_tile / kChunk, c_last = pos_last / kChunk;
  const int per = (c_last - c_first + args.num_splits) / args.num_splits;   // ceil(n / splits)
  const int c0 = c_first + split * per, c1 = min(c0 + per, c_last + 1);
  if (c0 > c_last) {   // more splits than chunks: a neutral partial, no data touched
    if (g == 0 && (!COOP || wave == 0)) {
      const int64_t slot = ((int64_t)item * args.num_splits + split) * 16 + r;
      args.partial_ml[slot * 2] = -INFINITY;
      args.partial_ml[slot * 2 + 1] = 0.f;
    }
    return;
  }

  TileState<HD> t;
  t.pos = row_ok ? pos_first + ti : -1;
  t.lo = (a.window > 0) ? max(0, t.pos - a.window + 1) : 0;
  load_query<HD>(t, (const bf16_t*)a.q + ((int64_t)token * a.nq + head) * HD, row_ok, g);
  const float scale_log2 = a.scale * 1.44269504088896341f;
  const int lo_last = (a.window > 0) ? max(0, pos_last - a.window + 1) : 0;

  constexpr int kStride = COOP ? 128 : 32;
  const int key_begin = max(c0 * kChunk, lo_tile & ~31) + (COOP ? wave * 32 : 0);
  const int key_end = min(c1 * kChunk, pos_last + 1);
  PageCursor cur{(ConstTable)table, a.page_size, pos_last, -1, -1};
  if (PAGE16) cur.start(key_begin);

  KvBlock<HD> A, B;
  // head sizes in whole 32-element slices on power-of-two pages take the blocks with
  // 16-byte value loads (the keys of a block permuted over the score products' rows)
  constexpr bool kWide = PAGE16 && HD % 32 == 0;
  auto load_block = [&](KvBlock<HD>& b, int kb) {
    if constexpr (kWide) load_kv_block_wide<HD>(b, a, cur, kvh, kb, kStride, r, g);
    else load_kv_block<HD, PAGE16>(b, a, table, cur, kvh, kb, kStride, r, g);
  };
  if (key_begin < key_end) load_block(A, key_begin);
  for (int kb = key_begin; kb < key_end; kb += 2 * kStride) {
    if (kb + kStride < key_end) load_block(B, kb + kStride);
    tile_update<HD, false, kWide>(t, A, kb, scale_log2, kb + 31 <= pos_first && kb >= lo_last, g);
    if (kb + kStride >= key_end) break;
    if (kb + 2 * kStride < key_end) load_block(A, kb + 2 * kStride);
    tile_update<HD, false, kWide>(t, B, kb + kStride, scale_log2,
                                  kb + kStride + 31 <= pos_first && kb + kStride >= lo_last, g);
  }
  f32x4 (&o)[DB] = t.o;
  float m = t.m, l = row_sum<HD>(t);

  if (COOP) {   // the four waves' partial results, merged by wave 0 in wave order
    __shared__ float s_ml[3][kWave][2];
    __shared__ f32x4 s_o[3][DB][kWave];
    if (wave > 0) {
      s_ml[wave - 1][lane][0] = m;
      s_ml[wave - 1][lane][1] = l;
#pragma unroll
      for (int db = 0; db < DB; ++db) s_o[wave - 1][db][lane] = o[db];
    }
    __syncthreads();
    if (wave > 0) return;
    float M = m;
#pragma unroll
    for (int w = 0; w < 3; ++w) M = fmaxf(M, s_ml[w][lane][0]);
    if (M != -INFINITY) {
      const float w0 = __builtin_amdgcn_exp2f(m - M);
      l *= w0;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][i] *= w0;
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        const float mw = s_ml[w][lane][0];
        if (mw == -INFINITY) continue;
        const float ww = __builtin_amdgcn_exp2f(mw - M);
        l += s_ml[w][lane][1] * ww;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const f32x4 ow = s_o[w][db][lane];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[db][i] += ow[i] * ww;
        }
      }
      m = M;
    }
  }

  // lane (r, g) holds O^T[d = db*16 + g*4 + i][row r]
  if (args.num_splits == 1) {
    if (!row_ok) return;
    store_tile<HD>(t, l, (bf16_t*)a.out + ((int64_t)token * a.nq + head) * HD, g);
  } else {
    const int64_t slot = ((int64_t)item * args.num_splits + split) * 16 + r;
    if (row_ok) {
      float* po = args.partial_o + slot * HD;
#pragma unroll
      for (int db = 0; db < DB; ++db) *(f32x4*)(po + db * 16 + g * 4) = o[db];
    }
    if (g == 0) {
      args.partial_ml[slot * 2] = m;      // in units of log2: scores were scaled by log2(e)
      args.partial_ml[slot * 2 + 1] = l;
    }
  }
}

// Merge the splits of every tile: out = sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M),
// splits taken in order.  One workgroup per item, thread (row, column group).  A split
// without keys has left m = -inf and is skipped.  Splits are taken eight at a time: the
// loads of the eight, statistics and values, are all asked for before the first is used,
// none under a condition, and the first eight do not wait for the position either (it
// says how many splits hold keys at all, which ends the loop early when a short context
// has been given many splits), so a merge of up to eight splits costs one trip to memory.
template <int HD>
__global__ __launch_bounds__(256) void attention_merge_kernel(AttentionMfmaArgs args) {
  constexpr int kGroup = 8, DC = HD / 16;
  const AttentionArgs& a = args.base;
  const int item = blockIdx.x;
  const int tile = item / (a.nkv * args.head_blocks);
  const int kvh = (item / args.head_blocks) % a.nkv;
  const int hb = item % args.head_blocks;
  const int tok0 = args.tiles ? args.tiles[tile * 3 + 1] : tile,
            ntok = args.tiles ? args.tiles[tile * 3 + 2] : 1;
  const int group = a.nq / a.nkv;
  const int r = threadIdx.x / 16, dc = threadIdx.x % 16;
  const int ti = r / args.rows_per_token, hh = hb * 16 + r % args.rows_per_token;
  if (ti >= ntok || hh >= group) return;
  const int S = args.num_splits;
  const int64_t base = (int64_t)item * S * 16 + r;
  // splits beyond the tile's chunks hold nothing: same arithmetic as the first kernel
  const int pos_first = a.positions[tok0], pos_last = pos_first + ntok - 1;
  float M = -INFINITY, L = 0.f;
  float acc[DC] = {};
  int used = S;                              // known after the first group's loads
  for (int s0 = 0; s0 < used; s0 += kGroup) {
    float ms[kGroup], ls[kGroup], part[kGroup][DC];
#pragma unroll
    for (int j = 0; j < kGroup; ++j) {
      const int64_t slot = base + (int64_t)min(s0 + j, S - 1) * 16;   // past the end: the last again
      ms[j] = args.partial_ml[slot * 2];
      ls[j] = args.partial_ml[slot * 2 + 1];
#pragma unroll
      for (int i = 0; i < DC; ++i) part[j][i] = args.partial_o[slot * HD + i * 16 + dc];
    }
    if (s0 == 0) {
      const int lo_tile = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;
      const int nchunks = pos_last / kChunk - lo_tile / kChunk + 1;
      const int per = (nchunks - 1 + S) / S;
      used = min(S, (nchunks + per - 1) / per);
    }
    float Mg = M;
#pragma unroll
    for (int j = 0; j < kGroup; ++j) Mg = (s0 + j < S) ? fmaxf(Mg, ms[j]) : Mg;
    if (Mg == -INFINITY) continue;            // nothing but empty splits so far
    const float keep = __builtin_amdgcn_exp2f(M - Mg);     // M = -inf gives 0
    L *= keep;
#pragma unroll
    for (int i = 0; i < DC; ++i) acc[i] *= keep;
#pragma unroll
    for (int j = 0; j < kGroup; ++j) {
      // an empty split wrote no values: what is there is dropped, not multiplied by 0
      const bool live = s0 + j < S && ms[j] != -INFINITY;
      const float w = live ? __builtin_amdgcn_exp2f(ms[j] - Mg) : 0.f;
      L += live ? ls[j] * w : 0.f;
#pragma unroll
      for (int i = 0; i < DC; ++i) acc[i] += live ? part[j][i] * w : 0.f;
    }
    M = Mg;
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  bf16_t* out = (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + kvh * group + hh) * HD;
#pragma unroll
  for (int i = 0; i < DC; ++i) out[i * 16 + dc] = (bf16_t)(acc[i] * inv);
}

int ts_check_attention_args(const AttentionArgs& a, const char* who);

template <int HD>
static int launch_mfma(const AttentionMfmaArgs& args, hipStream_t stream) {
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  const int P = args.base.page_size;
  const bool page16 = P >= 16 && (P & (P - 1)) == 0;
  const dim3 coop_grid(items, args.num_splits), walk_grid((items + 3) / 4, args.num_splits);
  if (args.cooperative && page16)
    hipLaunchKernelGGL((attention_mfma_kernel<HD, true, true>), coop_grid, dim3(256), 0, stream, args);
  else if (args.cooperative)
    hipLaunchKernelGGL((attention_mfma_kernel<HD, true, false>), coop_grid, dim3(256), 0, stream, args);
  else if (page16)
    hipLaunchKernelGGL((attention_mfma_kernel<HD, false, true>), walk_grid, dim3(256), 0, stream, args);
  else
    hipLaunchKernelGGL((attention_mfma_kernel<HD, false, false>), walk_grid, dim3(256), 0, stream, args);
  if (args.num_splits > 1)
    hipLaunchKernelGGL(attention_merge_kernel<HD>, dim3(items), dim3(256), 0, stream, args);
  return 0;
}

// The merge alone, for the decode kernel's splits.
int launch_attention_merge(const AttentionMfmaArgs& args, hipStream_t stream) {
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  switch (args.base.hd) {
#define TS_CASE(HD) case HD: hipLaunchKernelGGL(attention_merge_kernel<HD>, dim3(items), dim3(256), 0, stream, args); break;
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_merge: head_dim=%d not built", args.base.hd);
  }
  return 0;
}

// The merge of a decode step's key splits that ts_attention_decode was told to leave.
extern "C" int ts_attention_merge(const AttentionMfmaArgs* p, hipStream_t stream) {
  const AttentionMfmaArgs& args = *p;
  if (args.num_tiles <= 0 || args.num_splits <= 1) return 0;
  if (!args.partial_o || !args.partial_ml) TS_FAIL("attention_merge: no partial results");
  if (launch_attention_merge(args, stream)) return -1;
  TS_CHECK_LAUNCH("attention_merge");
  return 0;
}

extern "C" int ts_attention_mfma_chunk() { return kChunk; }

int ts_check_attention_mfma_args(const AttentionMfmaArgs& args, const char* who) {
  const AttentionArgs& a = args.base;
  if (ts_check_attention_args(a, who)) return -1;
  if (a.hd % 16) TS_FAIL("%s: head_dim=%d must be a multiple of 16", who, a.hd);
  if (a.page_size % 4) TS_FAIL("%s: page_size=%d must be a multiple of 4", who, a.page_size);
  const int group = a.nq / a.nkv;
  if (args.rows_per_token != (group < 16 ? group : 16) ||
      args.head_blocks != (group + 15) / 16)
    TS_FAIL("%s: rows_per_token/head_blocks do not fit a group of %d", who, group);
  if (!args.tiles && args.num_tiles != a.num_entries)
    TS_FAIL("%s: without a tile list there is one tile per entry", who);
  if (((uintptr_t)a.q | (uintptr_t)a.out | (uintptr_t)a.k_pages | (uintptr_t)a.v_pages) & 15)
    TS_FAIL("%s: tensors must be 16-byte aligned", who);
  return 0;
}

extern "C" int ts_attention_mfma(const AttentionMfmaArgs* p, hipStream_t stream) {
  AttentionMfmaArgs args = *p;
  const AttentionArgs& a = args.base;
  if (a.num_tokens <= 0 || args.num_tiles <= 0) return 0;
  if (ts_check_attention_mfma_args(args, "attention_mfma")) return -1;
  if (args.num_splits < 1 || args.num_splits > 65535) TS_FAIL("attention_mfma: num_splits=%d", args.num_splits);
  if (args.num_splits > 1 && (!args.partial_o || !args.partial_ml))
    TS_FAIL("attention_mfma: splits need partial buffers");
  switch (a.hd) {
#define TS_CASE(HD) case HD: launch_mfma<HD>(args, stream); break;
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_mfma: head_dim=%d not built", a.hd);
  }
  TS_CHECK_LAUNCH("attention_mfma");
  return 0;
}
