// Paged causal attention on the matrix cores for long portions of prompts (bfloat16).
//
// The tile list comes sorted by the length of the key range, longest first.
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
  const int tile = tile_rank;                                // the list is sorted: longest first
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
    // (16 rows need not be a whole number of tokens: a row past the tile's tokens would
    // be the next tile's token with this tile's key range, stored over the right result)
    const bool row_ok = ti < tq && t < ntok && hh < group;
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
  PageCursor cur{(ConstTable)table, a.page_size, pos_last, -1, -1};
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
    const float sum = row_sum<HD>(ts[j]);        // by all lanes: it crosses lanes
    if (ts[j].pos < 0) continue;
    store_tile<HD>(ts[j], sum,
                   (bf16_t*)a.out + ((int64_t)(tok0 + j * tq + ti) * a.nq + head) * HD, g);
  }
}

// ---------------------------------------------------------------------------------
// The same walk with the workgroup's four waves sharing every K and V block through LDS
// (page sizes that are powers of two from 16 up).  The waves take four consecutive query tiles of
// one entry and one key/value head; per block of 32 keys each wave fetches a quarter of
// the operand registers from global memory and stores them to LDS in operand layout,
// double-buffered: the fetch of the next block is in flight while a block is worked on,
// and one barrier per block separates the two.  A block is read from L2 once per workgroup
// instead of once per wave, and operands come out of LDS just before their product, so
// few registers are held and several workgroups share a CU.
template <int HD>
__global__ __launch_bounds__(256, HD <= 128 ? 4 : 1) void attention_prefill_lds_kernel(
    AttentionMfmaArgs args) {
  constexpr int KS = (HD + 31) / 32, DB = HD / 16;
  constexpr int KQ = (2 * KS + 3) / 4, VQ = (2 * DB + 3) / 4;    // operand slots per wave
  __shared__ bf16x8 k_lds[2][2 * KS][kWave];
  __shared__ bf16x8 v_lds[2][DB][kWave];     // low half: first 16-key block, high: second
  const AttentionArgs& a = args.base;
  const int wave = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int heads = a.nkv * args.head_blocks;
  const int head_slot = blockIdx.x % heads;                   // one head per XCD's L2
  // All workgroups of a prompt of a few thousand tokens are resident at once, two or
  // three to a compute unit, in launch order: the first half of the launch takes the
  // items with the longest key ranges, longest first, the second half the shortest,
  // shortest first, so a unit's workgroups add up to about the same work.
  const int rank = blockIdx.x / heads, half = (args.num_tiles + 1) / 2;
  const int item = rank < half ? rank : args.num_tiles - 1 - (rank - half);   // sorted: longest first
  const int kvh = head_slot / args.head_blocks;
  const int hb = head_slot % args.head_blocks;
  const int entry = uniform(args.tiles[item * 3]), tok0 = uniform(args.tiles[item * 3 + 1]),
            ntok = uniform(args.tiles[item * 3 + 2]);
  const int* table = a.table + (int64_t)entry * a.table_width;
  const int P = a.page_size;
  const int tq = 16 / args.rows_per_token;

  // this wave's tile: tokens [wave*tq, wave*tq + tq) of the item
  const int ti = wave * tq + r / args.rows_per_token;
  const int hh = hb * 16 + r % args.rows_per_token;
  const int head = kvh * group + min(hh, group - 1);
  // (16 rows need not be a whole number of tokens: a row past the tile's tokens would be
  // the next wave's token with this wave's key range, stored over the right result)
  const bool row_ok = r / args.rows_per_token < tq && ti < ntok && hh < group;
  const int pos_first = uniform(a.positions[tok0]);
  const int pos_last = pos_first + ntok - 1;
  const int lo_all = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;
  const float scale_log2 = a.scale * 1.44269504088896341f;

  TileState<HD> t;
  t.pos = row_ok ? pos_first + ti : -1;
  t.lo = (a.window > 0) ? max(0, t.pos - a.window + 1) : 0;
  const int tile_first = pos_first + wave * tq;
  const int tile_last = wave * tq < ntok ? pos_first + min(ntok, (wave + 1) * tq) - 1 : -1;
  const int tile_lo = (a.window > 0) ? max(0, tile_first - a.window + 1) : 0;
  const int tile_lo_last = (a.window > 0) ? max(0, tile_last - a.window + 1) : 0;
  load_query<HD>(t, (const bf16_t*)a.q + ((int64_t)(tok0 + min(ti, ntok - 1)) * a.nq + head) * HD,
                 row_ok, g);

  const bf16_t* kp = (const bf16_t*)a.k_pages;
  const bf16_t* vp = (const bf16_t*)a.v_pages;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16x4 zero4 = {0, 0, 0, 0};
  PageCursor cur{(ConstTable)table, P, pos_last, -1, -1};
  const int key_begin = lo_all & ~31;
  cur.start(key_begin);

  // This wave's quarter of a block's operands: global -> registers.  The loads are
  // issued unconditionally (a missing page reads page 0 and is zeroed when stored to
  // LDS), so nothing but the barrier stands between them and the work on the block.
  constexpr bool kEven = (2 * KS) % 4 == 0, vEven = (2 * DB) % 4 == 0;
  // Values, wide form (head sizes in steps of 64): a block's values are DB * 16 head
  // elements times 32 keys, 64 bytes a row of the transposed page: a lane fetches 8 keys
  // of one row in a 16-byte load (lane % 4 = which 8 keys, lane / 4 and the instruction =
  // which row) instead of 4 keys in an 8-byte one, half the load instructions, and the two
  // groups of 4 keys go to their lanes' slots in LDS, every lane of a store to a bank of
  // its own.
  constexpr bool kWideV = DB % 4 == 0;
  // kAhead blocks are on their way from memory while one is worked on.  More than one
  // was measured and does not pay: the registers they take cost a resident wave, and it
  // is the number of resident waves (four per SIMD up to head size 128) that hides the
  // waits of this kernel, those for memory among them.
  constexpr int kAhead = 1;
  struct Fetched {
    bf16x8 k[KQ];
    bf16x4 v[VQ];
    bf16x8 vw[kWideV ? DB / 4 : 1];             // wide form: 8 keys of one head element each
    bool kvalid[KQ], vvalid[VQ];                // wave-uniform but for the head size's tail
    bool vwvalid;                               // wide form: this lane's half of the block
  };
  Fetched ring[kAhead];
  // address = head base + page * page stride (scalar) + position in page (scalar)
  //           + this lane's offset inside the slot (fixed for the whole walk)
  const int64_t k_page_stride = (int64_t)a.nkv * P * HD, v_page_stride = k_page_stride;
  const bf16_t* k_head = kp + (int64_t)kvh * P * HD;
  const bf16_t* v_head = vp + (int64_t)kvh * HD * P;
  // in bytes and unsigned: added to a scalar base as a 32-bit offset, without 64-bit
  // lane arithmetic (a page of one head is far below 4 GiB)
  unsigned k_lane[KQ], v_lane[VQ];
  int k_blk[KQ], v_blk[VQ];
  bool k_dim_ok[KQ];
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int q = kEven ? wave + 4 * i : min(wave + 4 * i, 2 * KS - 1);
    const int s0 = q % KS;
    k_blk[i] = q / KS;
    k_dim_ok[i] = KS * 32 == HD || g * 8 * KS + s0 * 8 < HD;
    k_lane[i] = 2u * (r * HD + min(g * 8 * KS + s0 * 8, HD - 8));
  }
  const int vw_q = lane % 4;                          // keys vw_q * 8 .. + 7 of the block
  unsigned vw_lane[kWideV ? DB / 4 : 1];
  if constexpr (kWideV) {
#pragma unroll
    for (int i = 0; i < DB / 4; ++i)
      vw_lane[i] = 2u * ((((i * 4 + wave) * 16 + lane / 4) * P) + (vw_q % 2) * 8);
  }
#pragma unroll
  for (int i = 0; i < VQ; ++i) {
    const int q = vEven ? wave + 4 * i : min(wave + 4 * i, 2 * DB - 1);
    v_blk[i] = q / DB;
    v_lane[i] = 2u * (((q % DB) * 16 + r) * P + g * 4);
  }
  // the offset as the load sees it: opaque, so that it stays a 32-bit register beside the
  // scalar base instead of being widened once, outside the loop, into a register pair
  auto lane_offset = [](unsigned off) {
    asm volatile("" : "+v"(off));
    return off;
  };
  auto fetch = [&](Fetched& f, int kb) {
    const int in_page = kb & (P - 1);             // a block of 16 keys never straddles a page
    const int page0 = cur.next0, page1 = cur.next1;
    const bf16_t* kb0 = k_head + (int64_t)max(page0, 0) * k_page_stride + in_page * HD;
    const bf16_t* kb1 = k_head + (int64_t)max(page1, 0) * k_page_stride +
                        ((in_page + 16) & (P - 1)) * HD;
    const bf16_t* vb0 = v_head + (int64_t)max(page0, 0) * v_page_stride + in_page;
    const bf16_t* vb1 = v_head + (int64_t)max(page1, 0) * v_page_stride + ((in_page + 16) & (P - 1));
#pragma unroll
    for (int i = 0; i < KQ; ++i) {
      f.kvalid[i] = (k_blk[i] ? page1 : page0) >= 0 && k_dim_ok[i];
      f.k[i] = *(const bf16x8*)((const char*)(k_blk[i] ? kb1 : kb0) + lane_offset(k_lane[i]));
    }
    if constexpr (kWideV) {
      const bool second = vw_q >= 2;             // the block's second 16 keys
      f.vwvalid = (second ? page1 : page0) >= 0;
      const char* vb = (const char*)(second ? vb1 : vb0);
#pragma unroll
      for (int i = 0; i < DB / 4; ++i) f.vw[i] = *(const bf16x8*)(vb + vw_lane[i]);
    } else {
#pragma unroll
      for (int i = 0; i < VQ; ++i) {
        f.vvalid[i] = (v_blk[i] ? page1 : page0) >= 0;
        f.v[i] = *(const bf16x4*)((const char*)(v_blk[i] ? vb1 : vb0) + lane_offset(v_lane[i]));
      }
    }
    cur.start(kb + 32);
  };
  // registers -> LDS, operand layout.  (Blanking under a branch, taken only by the last
  // block of a context, was measured: slower than the selects it saves.)
  auto stash = [&](const Fetched& f, int buf) {
#pragma unroll
    for (int i = 0; i < KQ; ++i)
      if (kEven || wave + 4 * i < 2 * KS)
        k_lds[buf][wave + 4 * i][lane] = f.kvalid[i] ? f.k[i] : zero8;
    if constexpr (kWideV) {
      // keys vw_q*8 .. +3 belong to lane group (vw_q % 2) * 2, the next four to the group
      // after it, in the half of the slot that the 16-key half of the block has
#pragma unroll
      for (int i = 0; i < DB / 4; ++i) {
        const bf16x8 x = f.vwvalid ? f.vw[i] : zero8;
        const bf16x4 lo = {x[0], x[1], x[2], x[3]}, hi = {x[4], x[5], x[6], x[7]};
        bf16x4* slot = (bf16x4*)&v_lds[buf][i * 4 + wave][(vw_q % 2) * 32 + lane / 4];
        slot[vw_q / 2] = lo;
        slot[32 + vw_q / 2] = hi;                 // 16 lanes further: the next lane group
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < VQ; ++i)
      if (vEven || wave + 4 * i < 2 * DB)
        ((bf16x4*)&v_lds[buf][(wave + 4 * i) % DB][lane])[(wave + 4 * i) / DB] =
            f.vvalid[i] ? f.v[i] : zero4;
  };

#pragma unroll
  for (int p = 0; p < kAhead; ++p)
    if (key_begin + 32 * p <= pos_last) fetch(ring[p], key_begin + 32 * p);
  stash(ring[0], 0);
  __syncthreads();
  int buf = 0;
  // ring slot p holds block kb0 + 32 p, already in LDS when its turn comes, and is
  // fetched into again at once for the block kAhead further on
  for (int kb0 = key_begin; kb0 <= pos_last; kb0 += 32 * kAhead) {
#pragma unroll
    for (int p = 0; p < kAhead; ++p) {
      const int kb = kb0 + 32 * p;
      if (kb > pos_last) break;
      if (kb + 32 * kAhead <= pos_last) fetch(ring[p], kb + 32 * kAhead);
      if (kb <= tile_last && kb + 31 >= tile_lo) {
        KvBlock<HD> b;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int s0 = 0; s0 < KS; ++s0) b.k[blk][s0] = k_lds[buf][blk * KS + s0][lane];
#pragma unroll
        for (int db = 0; db < DB; ++db) b.v[db] = v_lds[buf][db][lane];
        tile_update<HD, true>(t, b, kb, scale_log2, kb + 31 <= tile_first && kb >= tile_lo_last, g);
      }
      if (kb + 32 <= pos_last) stash(ring[(p + 1) % kAhead], buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
  }
  const float sum = row_sum<HD>(t);                // by all lanes: it crosses lanes
  if (row_ok)
    store_tile<HD>(t, sum, (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + head) * HD, g);
}


// ---------------------------------------------------------------------------------
// The walk of the kernel above with the blocks brought into LDS by the memory system
// itself (head sizes 64 and 128, page sizes that are powers of two from 16 up).
//
// global_load_lds writes a wave's 64 x 16 bytes to consecutive LDS addresses, whatever
// global addresses the lanes name: each lane names the 16 bytes that its own operand
// register will hold, so the block lies in LDS in operand layout without passing through
// registers, nothing is selected or stored by the waves, and the loads of a block are
// issued two blocks ahead into a ring of three buffers at no cost in registers.  (Measured
// on the kernel above: bringing a block in through registers, one block ahead, is a
// third to two fifths of its time.)
//
// For the values to be 16 bytes per lane the keys of a block are assigned to the rows of
// the two score products so that a lane's eight scores belong to eight consecutive keys:
// row i of product b is key (i / 4) * 8 + b * 4 + i % 4 of the block.  Lane (r, g) then
// holds the scores of keys g * 8 .. g * 8 + 7 and needs V^T[d][those keys], one 16-byte
// run of a page's row.
//
// A page that is not there (beyond the context, or given back by a window) is read from
// page 0 instead: its scores are masked, their weights are exactly zero, and what the
// cache holds is finite.
// 64 x 16 bytes from the lanes' global addresses to LDS at `dst` + 16 * lane, without
// registers in between.  Written as an instruction rather than through the compiler's
// builtin: the compiler, knowing such a load writes LDS, makes LDS reads wait for every
// one of them in flight (it cannot always tell the buffers apart), which is the opposite
// of sending for blocks ahead of time.  The kernel counts these loads itself (s_waitcnt
// vmcnt) and separates them from the reads by a barrier; "memory" tells the compiler that
// LDS has changed.
__device__ __forceinline__ void lds_dma16(const void* src, void* dst) {
  const unsigned lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)dst;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(src), "s"(lds)
               : "memory", "m0");
}

// H = 2: a second set of four waves takes the same four tiles and every second block of
// their keys (the first set the others), with a ring of its own, and the two partial
// results of a tile are merged through LDS at the end: twice the waves for a prompt with
// too few tiles to give every SIMD several.
//
// `paired`: a workgroup takes the item at its rank from the front of the sorted list and
// then the one at the same rank from the back, so every workgroup walks about the same
// number of blocks wherever it lands.  Unpaired, the first half of the launch takes the
// long items, longest first, and the second half the short ones, shortest first.
template <int HD, int H>
__global__ __launch_bounds__(256 * H, H == 1 ? 3 : 2) void attention_prefill_async_kernel(
    AttentionMfmaArgs args, int paired) {
  constexpr int KS = HD / 32, DB = HD / 16;
  constexpr int KQ = 2 * KS / 4, VQ = DB / 4;               // slots a wave brings in per block
  static_assert(HD % 64 == 0, "head sizes in steps of 64");
  // a ring buffer: the key slots of a block, then its value slots; three per set of waves
  constexpr int kSlots = 2 * KS + DB;
  extern __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[];
  typedef bf16x8 (*Slots)[kWave];
  const AttentionArgs& a = args.base;
  const int wave_all = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wave = wave_all % 4;             // which of the item's four tiles
  const int set = H == 1 ? 0 : wave_all / 4; // which of every H key blocks
  const Slots ring = (Slots)prefill_lds + set * 3 * kSlots;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int heads = a.nkv * args.head_blocks;
  const int head_slot = blockIdx.x % heads;                   // one head per XCD's L2
  const int rank = blockIdx.x / heads;
  const int kvh = head_slot / args.head_blocks;
  const int hb = head_slot % args.head_blocks;
  const int P = a.page_size;
  const int tq = 16 / args.rows_per_token;
  const float scale_log2 = a.scale * 1.44269504088896341f;

  // Where this lane's 16 bytes of each slot lie, relative to the start of the half of the
  // block (16 keys) they belong to.  Keys: slot q = b * KS + s0 is product b, elements
  // g*8*KS + s0*8 .. + 7 of the key in row r.  Values: slot db is head elements
  // db*16 .. + 15, this lane's row r of them, keys g*8 .. + 7 of the block.
  const int64_t page_stride = (int64_t)a.nkv * P * HD;         // elements, keys and values alike
  const bf16_t* k_head = (const bf16_t*)a.k_pages + (int64_t)kvh * P * HD;
  const bf16_t* v_head = (const bf16_t*)a.v_pages + (int64_t)kvh * HD * P;
  const bool k_second = r >= 8;          // this lane's keys lie in the block's second 16
  const bool v_second = g >= 2;
  unsigned k_off[KQ], v_off[VQ];         // bytes
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int q = wave + 4 * i, b = q / KS, s0 = q % KS;
    const int key16 = ((r / 4) * 8 + b * 4 + r % 4) % 16;    // inside its half
    k_off[i] = 2u * (key16 * HD + g * 8 * KS + s0 * 8);
  }
#pragma unroll
  for (int i = 0; i < VQ; ++i)
    v_off[i] = 2u * (((wave + 4 * i) * 16 + r) * P + (g % 2) * 8);
  constexpr int kLoads = KQ + VQ;        // vector memory loads a wave has in flight per block

  for (int part = 0; part < 2; ++part) {
    int item;
    if (paired) {
      item = part == 0 ? rank : args.num_tiles - 1 - rank;
      if (part == 1 && item <= rank) break;
    } else {
      if (part == 1) break;
      const int front = (args.num_tiles + 1) / 2;
      item = rank < front ? rank : args.num_tiles - 1 - (rank - front);
    }
    const int entry = uniform(args.tiles[item * 3]), tok0 = uniform(args.tiles[item * 3 + 1]),
              ntok = uniform(args.tiles[item * 3 + 2]);
    const int* table = a.table + (int64_t)entry * a.table_width;

    const int ti = wave * tq + r / args.rows_per_token;
    const int hh = hb * 16 + r % args.rows_per_token;
    const int head = kvh * group + min(hh, group - 1);
    const bool row_ok = r / args.rows_per_token < tq && ti < ntok && hh < group;
    const int pos_first = uniform(a.positions[tok0]);
    const int pos_last = pos_first + ntok - 1;
    const int lo_all = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;

    TileState<HD> t;
    t.pos = row_ok ? pos_first + ti : -1;
    t.lo = (a.window > 0) ? max(0, t.pos - a.window + 1) : 0;
    const int tile_first = pos_first + wave * tq;
    const int tile_last = wave * tq < ntok ? pos_first + min(ntok, (wave + 1) * tq) - 1 : -1;
    const int tile_lo = (a.window > 0) ? max(0, tile_first - a.window + 1) : 0;
    const int tile_lo_last = (a.window > 0) ? max(0, tile_last - a.window + 1) : 0;
    load_query<HD>(t, (const bf16_t*)a.q + ((int64_t)(tok0 + min(ti, ntok - 1)) * a.nq + head) * HD,
                   row_ok, g);

    // The item's blocks of 32 keys, numbered from its first; this set of waves takes
    // blocks set, set + H, ...: `mine` of them, numbered j here.  Every set makes the same
    // number of turns (a barrier each), the last of them idle for a set with one block less.
    const int key_begin = lo_all & ~31;
    const int nblocks = ((pos_last - key_begin) >> 5) + 1;
    const int turns = (nblocks + H - 1) / H;
    const int mine = (nblocks - set + H - 1) / H;
    const int kb_first = key_begin + 32 * set;
    PageCursor cur{(ConstTable)table, P, pos_last, -1, -1};
    cur.start(kb_first);
    // issue the loads of this set's block j into ring buffer `to`; calls come in order of
    // j, as the cursor needs
    auto issue = [&](int j, int to) {
      const int kb = kb_first + 32 * H * j;
      const int in0 = kb & (P - 1), in1 = (kb + 16) & (P - 1);
      const int64_t p0 = (int64_t)max(cur.next0, 0) * page_stride, p1 = (int64_t)max(cur.next1, 0) * page_stride;
      const bf16_t* kb0 = k_head + p0 + in0 * HD;
      const bf16_t* kb1 = k_head + p1 + in1 * HD;
      const bf16_t* vb0 = v_head + p0 + in0;
      const bf16_t* vb1 = v_head + p1 + in1;
      const char* kbase = (const char*)(k_second ? kb1 : kb0);
      const char* vbase = (const char*)(v_second ? vb1 : vb0);
      const Slots kdst = ring + to * kSlots, vdst = kdst + 2 * KS;
#pragma unroll
      for (int i = 0; i < KQ; ++i) lds_dma16(kbase + k_off[i], &kdst[wave + 4 * i][0]);
#pragma unroll
      for (int i = 0; i < VQ; ++i) lds_dma16(vbase + v_off[i], &vdst[wave + 4 * i][0]);
      cur.start(kb + 32 * H);
    };

    // One turn: block j is worked on out of ring buffer `from` while block j + 2 is sent
    // for into buffer `to`, which block j - 1 was read from.
    auto turn = [&](int j, int from, int to) {
      const int kb = kb_first + 32 * H * j;
      // this wave's share of block j has arrived: at most block j + 1's loads are in flight
      if (j + 1 < mine) __builtin_amdgcn_s_waitcnt(0x0F70 | kLoads);
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      // Every wave's share of block j is in LDS, and every wave is through with block
      // j - 1.  The bare barrier: __syncthreads would first wait for every load in flight,
      // the younger block's among them.  The empty statements keep the compiler from
      // moving LDS reads across it.
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      // Only now may block j - 1's buffer be written: a wave that has nothing to do with a
      // block (outside its tile's window, or past its tile's last row) runs ahead of the
      // others by a whole turn, and loads sent for before the barrier could land while a
      // slower wave still reads that buffer.
      if (j + 2 < mine) issue(j + 2, to);
      if (j < mine && kb <= tile_last && kb + 31 >= tile_lo) {
        const Slots kcur = ring + from * kSlots, vcur = kcur + 2 * KS;
        KvBlock<HD> b;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int s0 = 0; s0 < KS; ++s0) b.k[blk][s0] = kcur[blk * KS + s0][lane];
#pragma unroll
        for (int db = 0; db < DB; ++db) b.v[db] = vcur[db][lane];
        tile_update<HD, true, true>(t, b, kb, scale_log2, kb + 31 <= tile_first && kb >= tile_lo_last, g);
      }
    };

    // The query rows are waited for here, once (the empty statement uses them), and not at
    // their first use inside the loop, where the wait would be for every block in flight
    // as well; with them gone the vector memory counter counts the blocks' loads alone.
#pragma unroll
    for (int s0 = 0; s0 < KS; ++s0) asm volatile("" : "+v"(t.q[s0]));
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (mine > 0) issue(0, 0);
    if (mine > 1) issue(1, 1);
    // written out three times so that every turn's ring buffers are constants
    for (int j = 0; j < turns; j += 3) {
      turn(j, 0, 2);
      if (j + 1 < turns) turn(j + 1, 1, 0);
      if (j + 2 < turns) turn(j + 2, 2, 1);
    }

    if constexpr (H == 2) {
      // The second set hands its partial result over in LDS, in the rings' space: values
      // [tile][element][lane], then the row statistics.
      float* lds_o = (float*)prefill_lds;
      float* lds_ml = lds_o + 4 * DB * 4 * kWave;
      static_assert(H * 3 * kSlots * kWave * 16 >= (4 * DB * 4 + 4 * 2) * kWave * 4, "merge area");
      __syncthreads();                             // the rings have been read for the last time
      if (set == 1) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) lds_o[((wave * DB + db) * 4 + i) * kWave + lane] = t.o[db][i];
        lds_ml[(wave * 2) * kWave + lane] = t.m;
        lds_ml[(wave * 2 + 1) * kWave + lane] = t.l;
      }
      __syncthreads();
      if (set == 0) {
        const float m1 = lds_ml[(wave * 2) * kWave + lane], l1 = lds_ml[(wave * 2 + 1) * kWave + lane];
        // m is in units of log2; a set that saw no key of this row has m = -inf and weight 0
        const float m_use = max2(max2(t.m, m1), -1e30f);
        const float w0 = __builtin_amdgcn_exp2f(t.m - m_use), w1 = __builtin_amdgcn_exp2f(m1 - m_use);
        t.l = t.l * w0 + l1 * w1;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float o1 = lds_o[((wave * DB + db) * 4 + i) * kWave + lane];
            t.o[db][i] = t.o[db][i] * w0 + (w1 == 0.f ? 0.f : o1 * w1);
          }
        const float sum = row_sum<HD>(t);          // by all lanes: it crosses lanes
        if (row_ok)
          store_tile<HD>(t, sum, (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + head) * HD, g);
      }
    } else {
      const float sum = row_sum<HD>(t);            // by all lanes: it crosses lanes
      if (row_ok)
        store_tile<HD>(t, sum, (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + head) * HD, g);
    }
    __syncthreads();       // before the next item's blocks are sent for into these buffers
  }
}

// Query tiles per wavefront: as many as the register file holds accumulators for.
constexpr int tiles_per_wave(int hd) { return hd <= 32 ? 4 : (hd <= 64 ? 2 : 1); }

// Tokens one work item covers, in 16-row tiles: four (one per wave) for the LDS kernel.
extern "C" int ts_attention_prefill_tiles(int head_dim, int page_size) {
  return page_size >= 16 && (page_size & (page_size - 1)) == 0 ? 4 : tiles_per_wave(head_dim);
}

static int compute_units() {
  static int cus = 0;       // of the device current when first asked; a host's GPUs are alike
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  return cus;
}

template <int HD, int H>
static int launch_prefill_async(const AttentionMfmaArgs& args, int paired, hipStream_t stream) {
  const int heads = args.base.nkv * args.head_blocks;
  const dim3 grid((paired ? (args.num_tiles + 1) / 2 : args.num_tiles) * heads);
  const size_t lds = (size_t)H * 3 * (2 * (HD / 32) + HD / 16) * kWave * 16;
  auto kernel = attention_prefill_async_kernel<HD, H>;
  static bool raised = false;     // per instantiation
  if (!raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      TS_FAIL("attention_prefill: cannot raise the LDS limit to %zu bytes", lds);
    raised = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(256 * H), lds, stream, args, paired);
  return 0;
}

template <int HD>
static int launch_prefill_lds(const AttentionMfmaArgs& args, hipStream_t stream) {
  if (args.tiles_per_wave != 4) TS_FAIL("attention_prefill: the LDS kernel takes items of 4 tiles");
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  if constexpr (HD % 64 == 0 && HD <= 128) {
    // Up to two items a compute unit: two sets of waves per item, and the items paired (a
    // long one and a short one per workgroup) once there are more items than units, so
    // that one round of workgroups of equal length fills the chip.  More: one set, three
    // workgroups a unit, longest first.  (Measured at 16 query and 8 key/value heads of
    // 128: 1,024 tokens 21.5 us with two sets unpaired, 25.3 paired; 1,536 tokens 34.0
    // paired, 35.7 unpaired; 2,048 tokens 42.6 paired, 48.8 with one set; 2,560 tokens 63.9
    // with one set, 92.7 with two sets paired, which then need a second round.)
    const int units = compute_units();
    if (items <= 2 * units) return launch_prefill_async<HD, 2>(args, items > units, stream);
    return launch_prefill_async<HD, 1>(args, 0, stream);
  } else {
    hipLaunchKernelGGL((attention_prefill_lds_kernel<HD>), dim3(items), dim3(256), 0, stream, args);
  }
  return 0;
}

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
  if (!args.tiles) TS_FAIL("attention_prefill: no tile list");
  const bool page16 = a.page_size >= 16 && (a.page_size & (a.page_size - 1)) == 0;
  int rc = 0;
  switch (a.hd) {
#define TS_CASE(HD)                                                               \
  case HD:                                                                        \
    rc = page16 ? launch_prefill_lds<HD>(args, stream) : launch_prefill<HD, false>(args, stream); \
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
