// Paged causal attention on the matrix cores for long portions of prompts (bfloat16).
//
// A wavefront works on TPW consecutive 16-row query tiles of one batch entry and walks
// their common key range alone, 32 keys at a time, with the next block's keys and values
// in flight while the current block is worked on.  Every K and V block it loads serves
// TPW tiles; the four waves of a workgroup take neighbouring tiles, so most of their
// loads meet in the first-level cache.  A tile skips blocks beyond its causal range or
// before its window, and skips the mask where every key of a block is visible.
#include "attention_core.h"

template <int HD, int TPW, bool PAGE16>
__global__ __launch_bounds__(256) void attention_prefill_kernel(AttentionMfmaArgs args) {
  const AttentionArgs& a = args.base;
  const int wave = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  // Workgroups are handed to the eight XCDs in turn, and each XCD has an L2 of its own:
  // workgroup b works on head (b mod heads), so a head's keys and values stay in one L2.
  // Its four waves take neighbouring query tiles, the longest key ranges first.
  const int heads = a.nkv * args.head_blocks;
  const int head_slot = blockIdx.x % heads;
  const int tile_rank = (blockIdx.x / heads) * 4 + wave;
  if (tile_rank >= args.num_tiles) return;
  const int tile = args.num_tiles - 1 - tile_rank;
  const int kvh = head_slot / args.head_blocks;
  const int hb = head_slot % args.head_blocks;
  const int entry = uniform(args.tiles[tile * 3]), tok0 = uniform(args.tiles[tile * 3 + 1]),
            ntok = uniform(args.tiles[tile * 3 + 2]);
  const int* table = a.table + (int64_t)entry * a.table_width;
  const int tq = 16 / args.rows_per_token;                   // tokens per 16-row tile

  const int ti = r / args.rows_per_token;
  const int hh = hb * 16 + r % args.rows_per_token;
  const int head = kvh * group + min(hh, group - 1);
  const int pos_first = uniform(a.positions[tok0]);          // positions are consecutive
  const int pos_last = pos_first + ntok - 1;
  const int lo_all = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;
  const float scale_log2 = a.scale * 1.44269504088896341f;

  TileState<HD> ts[TPW];
  int tile_first[TPW], tile_last[TPW], tile_lo[TPW], tile_lo_last[TPW];   // wave-uniform
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int t = j * tq + ti;
    const bool row_ok = t < ntok && hh < group;
    ts[j].pos = row_ok ? pos_first + t : -1;
    ts[j].lo = (a.window > 0) ? max(0, ts[j].pos - a.window + 1) : 0;
    tile_first[j] = pos_first + j * tq;
    tile_last[j] = j * tq < ntok ? pos_first + min(ntok, (j + 1) * tq) - 1 : -1;
    tile_lo[j] = (a.window > 0) ? max(0, tile_first[j] - a.window + 1) : 0;
    tile_lo_last[j] = (a.window > 0) ? max(0, tile_last[j] - a.window + 1) : 0;
    load_query<HD>(ts[j], (const bf16_t*)a.q +
                   ((int64_t)(tok0 + min(t, ntok - 1)) * a.nq + head) * HD, row_ok, g);
  }

  const int key_begin = lo_all & ~31;
  PageCursor cur{(ConstTable)table, a.page_size, pos_last, {-1, -1}};
  if (PAGE16) cur.start(key_begin);

  auto work = [&](const KvBlock<HD>& b, int kb) {
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      if (kb > tile_last[j] || kb + 31 < tile_lo[j]) continue;        // scalar conditions
      const bool interior = kb + 31 <= tile_first[j] && kb >= tile_lo_last[j];
      tile_update<HD>(ts[j], b, kb, scale_log2, interior, g);
    }
  };

  KvBlock<HD> A, B;
  load_kv_block<HD, PAGE16>(A, a, table, cur, kvh, key_begin, 32, r, g);
  for (int kb = key_begin; kb <= pos_last; kb += 64) {
    if (kb + 32 <= pos_last)
      load_kv_block<HD, PAGE16>(B, a, table, cur, kvh, kb + 32, 32, r, g);
    work(A, kb);
    if (kb + 32 > pos_last) break;
    if (kb + 64 <= pos_last)
      load_kv_block<HD, PAGE16>(A, a, table, cur, kvh, kb + 64, 32, r, g);
    work(B, kb + 32);
  }

#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    if (ts[j].pos < 0) continue;
    store_tile<HD>(ts[j], (bf16_t*)a.out + ((int64_t)(tok0 + j * tq + ti) * a.nq + head) * HD, g);
  }
}

// Query tiles per wavefront: as many as the register file holds accumulators for.
constexpr int tiles_per_wave(int hd) { return hd <= 64 ? 4 : (hd <= 128 ? 2 : 1); }

extern "C" int ts_attention_prefill_tiles(int head_dim) { return tiles_per_wave(head_dim); }

template <int HD, bool PAGE16>
static int launch_prefill(const AttentionMfmaArgs& args, hipStream_t stream) {
  if (args.tiles_per_wave != tiles_per_wave(HD))
    TS_FAIL("attention_prefill: tiles_per_wave=%d, head size %d takes %d", args.tiles_per_wave,
            HD, tiles_per_wave(HD));
  dim3 grid(((args.num_tiles + 3) / 4) * args.base.nkv * args.head_blocks);
  hipLaunchKernelGGL((attention_prefill_kernel<HD, tiles_per_wave(HD), PAGE16>), grid, dim3(256),
                     0, stream, args);
  return 0;
}

int ts_check_attention_mfma_args(const AttentionMfmaArgs& args, const char* who);

// `tiles` lists wave items (entry, first flat token, tokens) of at most
// tiles_per_wave * (16 / rows_per_token) consecutive tokens each.
extern "C" int ts_attention_prefill(const AttentionMfmaArgs* p, hipStream_t stream) {
  AttentionMfmaArgs args = *p;
  const AttentionArgs& a = args.base;
  if (a.num_tokens <= 0 || args.num_tiles <= 0) return 0;
  if (ts_check_attention_mfma_args(args, "attention_prefill")) return -1;
  const bool page16 = a.page_size % 16 == 0;
  int rc = 0;
  switch (a.hd) {
#define TS_CASE(HD)                                                               \
  case HD:                                                                        \
    rc = page16 ? launch_prefill<HD, true>(args, stream) : launch_prefill<HD, false>(args, stream); \
    break;
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_prefill: head_dim=%d not built", a.hd);
  }
  if (rc) return rc;
  TS_CHECK_LAUNCH("attention_prefill");
  return 0;
}
