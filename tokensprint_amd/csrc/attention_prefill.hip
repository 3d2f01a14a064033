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

// ---------------------------------------------------------------------------------
// The walk of the kernel above, 64 keys a turn (two sub-blocks of 32 keys, each laid out in
// LDS as that kernel lays out a block), with what a turn costs beside its products cut
// down: one barrier, one wait and one softmax update (row maximum, rescale, row sum) per 64
// keys instead of two; four independent chains of score products instead of two; and the
// addresses of a turn's loads formed in a few vector instructions instead of some ninety
// scalar ones: a lane's address is a 64-bit constant of its own (head, row, slice of the
// row) plus its page's id times the page stride, one multiply-add per load, the page ids
// of the turn's four 16-key halves fetched through the scalar cache a turn ahead.
//
// A ring of two buffers of 64 keys per set of waves: a turn's loads are sent for right
// after the barrier that says every wave is through with the buffer they go into (the
// buffer of the turn before), and are waited for at the start of the next turn.
//
// TILES waves share an item's key blocks (an item is TILES consecutive 16-row tiles); H
// sets of them split the item's turns (set s takes turns s, s + H, ...) and merge through
// LDS at the end.  `paired` as above.
// Scores of a 64-key turn for one tile, masked softmax update over all 64, and
// O^T += V^T P^T for both sub-blocks.  `buf` holds the turn's two sub-blocks (keys, then
// values, in operand layout).  `between` runs once all the key operands have been asked
// for (the kernel sends for the next turn's blocks there, while LDS answers).
//
// The operands of a stretch of products are asked for together, before the first of them,
// and the scheduler is told to leave the stretches in that order: the compiler, left
// alone, asks for an operand only a few instructions before its product, and with two to
// four waves a SIMD nothing else hides the time LDS takes to answer.  DEEP (kernels that
// keep two waves a SIMD and so have registers to spare): a stretch is the whole turn, all
// sixteen key operands before the first score product and all sixteen value operands
// before the softmax arithmetic.  Otherwise (four waves a SIMD, 128 registers each) the
// order is the compiler's.
template <int HD, bool DEEP, typename Between>
__device__ __forceinline__ void tile_update64(TileState<HD>& t, bf16x8 (*buf)[kWave], int lane, int kb,
                                              float scale_log2, bool interior, int g,
                                              Between between) {
  constexpr int KS = HD / 32, DB = HD / 16, kSlots = 2 * KS + DB;
  f32x4 st[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) st[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if constexpr (DEEP) {
    bf16x8 k[4][KS];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int s = 0; s < KS; ++s) k[j][s] = buf[(j / 2) * kSlots + (j % 2) * KS + s][lane];
    __builtin_amdgcn_sched_barrier(0);
    between();
    __builtin_amdgcn_sched_barrier(0);
    // four chains side by side: a product never waits for the one before it
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        st[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k[j][s], t.q[s], st[j], 0, 0, 0);
  } else {
    between();
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int s = 0; s < KS; ++s)
        st[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[(j / 2) * kSlots + (j % 2) * KS + s][lane],
                                                        t.q[s], st[j], 0, 0, 0);
  }
  bf16x8 v[2][DB];
  if constexpr (DEEP) {
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int db = 0; db < DB; ++db) v[sb][db] = buf[sb * kSlots + 2 * KS + db][lane];
    __builtin_amdgcn_sched_barrier(0);
  }
  if (!interior) {
    asm volatile("" ::: "memory");   // keeps this a branch
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb + (j / 2) * 32 + g * 8 + (j % 2) * 4 + i;
        st[j][i] = (key <= t.pos && key >= t.lo) ? st[j][i] : -INFINITY;
      }
  }
  float mx = max2(max2(st[0][0], st[0][1]), max2(st[0][2], st[0][3]));
#pragma unroll
  for (int j = 1; j < 4; ++j)
    mx = max2(max2(mx, max2(st[j][0], st[j][1])), max2(st[j][2], st[j][3]));
  const float m_new = max2(t.m, col4_max(mx) * scale_log2);
  const float m_use = max2(m_new, -1e30f);
  const float corr = __builtin_amdgcn_exp2f(t.m - m_use);
  float ps = 0.f;
  bf16x8 pv[2];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[j][i], scale_log2, -m_use));
      ps += p;
      pv[j / 2][(j % 2) * 4 + i] = (bf16_t)p;
    }
  t.l = t.l * corr + ps;
  t.m = m_new;
  if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) t.o[db][i] *= corr;
  }
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x8 operand = DEEP ? v[sb][db] : buf[sb * kSlots + 2 * KS + db][lane];
      t.o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(operand, pv[sb], t.o[db], 0, 0, 0);
    }
  }
}


template <int HD, int H, int TILES, int NBUF, bool P16>
__device__ __forceinline__ void attention_prefill_wide(const AttentionMfmaArgs& args, int paired) {
  constexpr int KS = HD / 32, DB = HD / 16;
  constexpr int kSlots = 2 * KS + DB;        // of a sub-block of 32 keys
  constexpr int L = kSlots / TILES;          // loads a wave sends for per sub-block
  static_assert(HD % 64 == 0 && kSlots % TILES == 0, "head sizes in steps of 64");
  constexpr int kBuf = 2 * kSlots;           // slots of a ring buffer: 64 keys
  constexpr int kAhead = NBUF - 1;           // turns whose blocks are on their way
  extern __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[];
  typedef bf16x8 (*Slots)[kWave];
  const AttentionArgs& a = args.base;
  const int wave_all = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wave = wave_all % TILES;             // which of the item's tiles
  const int set = H == 1 ? 0 : wave_all / TILES; // which of every H turns
  const Slots ring = (Slots)prefill_lds + set * NBUF * kBuf;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int heads = a.nkv * args.head_blocks;
  const int head_slot = blockIdx.x % heads;                   // one head per XCD's L2
  const int rank = blockIdx.x / heads;
  const int kvh = head_slot / args.head_blocks;
  const int hb = head_slot % args.head_blocks;
  const int P = a.page_size, lp = __builtin_ctz(P);
  const int tq = 16 / args.rows_per_token;
  const float scale_log2 = a.scale * 1.44269504088896341f;

  // What this lane names in each of its loads of a sub-block: a 64-bit address that lacks
  // only the page (page id times the page stride, the same for keys and values) and, with
  // pages above 16 keys, the 16-key half's place inside its page.  Slot q of a sub-block is
  // a key slot (product q / KS, elements g*8*KS + (q % KS)*8 .. + 7 of the key in row r)
  // below 2 KS, else the value slot of head elements (q - 2 KS)*16 .. + 15 (this lane's row
  // r of them, keys g*8 .. + 7).  A lane's keys lie in the sub-block's second half from row
  // 8 (keys) or from lane group 2 (values).
  const unsigned page_stride = 2u * (unsigned)a.nkv * P * HD;   // bytes
  const char* k_head = (const char*)a.k_pages + (int64_t)kvh * P * HD * 2;
  const char* v_head = (const char*)a.v_pages + (int64_t)kvh * HD * P * 2;
  const char* cbase[L];
  bool second[L];
  unsigned in_bytes[L];                      // bytes per key of the place inside a page
#pragma unroll
  for (int i = 0; i < L; ++i) {
    const int q = wave + TILES * i;
    if (q < 2 * KS) {
      const int b = q / KS, s0 = q % KS;
      const int key16 = ((r / 4) * 8 + b * 4 + r % 4) % 16;
      cbase[i] = k_head + 2 * (key16 * HD + g * 8 * KS + s0 * 8);
      second[i] = r >= 8;
      in_bytes[i] = 2u * HD;
    } else {
      cbase[i] = v_head + 2 * (((q - 2 * KS) * 16 + r) * P + (g % 2) * 8);
      second[i] = g >= 2;
      in_bytes[i] = 2u;
    }
  }

  // The workgroup's items (one, or with `paired` the one at its rank from the front of the
  // sorted list and the one at the same rank from the back), their first positions and this
  // lane's query rows: all asked for now, so that the second item begins without the chain
  // of trips to memory that the first one waits through.
  int item_of[2], entry_of[2], tok0_of[2], ntok_of[2], pos_of[2];
  bool has[2] = {true, false};
  if (paired) {
    item_of[0] = rank;
    item_of[1] = args.num_tiles - 1 - rank;
    has[1] = item_of[1] > rank;
  } else {
    const int front = (args.num_tiles + 1) / 2;
    item_of[0] = rank < front ? rank : args.num_tiles - 1 - (rank - front);
    item_of[1] = item_of[0];
  }
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    entry_of[p] = args.tiles[item_of[p] * 3];
    tok0_of[p] = args.tiles[item_of[p] * 3 + 1];
    ntok_of[p] = args.tiles[item_of[p] * 3 + 2];
  }
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    entry_of[p] = uniform(entry_of[p]); tok0_of[p] = uniform(tok0_of[p]); ntok_of[p] = uniform(ntok_of[p]);
    pos_of[p] = a.positions[tok0_of[p]];
  }
  const int hh = hb * 16 + r % args.rows_per_token;
  const int head = kvh * group + min(hh, group - 1);
  const int ti = wave * tq + r / args.rows_per_token;
  bf16x8 q_of[2][KS];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    pos_of[p] = uniform(pos_of[p]);
    const bool row_ok = r / args.rows_per_token < tq && ti < ntok_of[p] && hh < group;
    const bf16_t* qrow = (const bf16_t*)a.q +
                         ((int64_t)(tok0_of[p] + min(ti, ntok_of[p] - 1)) * a.nq + head) * HD;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int s0 = 0; s0 < KS; ++s0)
      q_of[p][s0] = row_ok && p == 0 ? *(const bf16x8*)(qrow + g * 8 * KS + s0 * 8) : zero8;
  }

#pragma unroll
  for (int part = 0; part < 2; ++part) {
    if (!has[part]) break;
    const int entry = entry_of[part], tok0 = tok0_of[part], ntok = ntok_of[part];
    const ConstTable table = (ConstTable)(a.table + (int64_t)entry * a.table_width);
    const bool row_ok = r / args.rows_per_token < tq && ti < ntok && hh < group;
    const int pos_first = pos_of[part];
    const int pos_last = pos_first + ntok - 1;
    const int lo_all = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;

    TileState<HD> t;
    t.pos = row_ok ? pos_first + ti : -1;
    t.lo = (a.window > 0) ? max(0, t.pos - a.window + 1) : 0;
    const int tile_first = pos_first + wave * tq;
    const int tile_last = wave * tq < ntok ? pos_first + min(ntok, (wave + 1) * tq) - 1 : -1;
    const int tile_lo = (a.window > 0) ? max(0, tile_first - a.window + 1) : 0;
    const int tile_lo_last = (a.window > 0) ? max(0, tile_last - a.window + 1) : 0;
    if (part == 0) {
#pragma unroll
      for (int s0 = 0; s0 < KS; ++s0) t.q[s0] = q_of[0][s0];
    } else {
      const bf16_t* qrow = (const bf16_t*)a.q + ((int64_t)(tok0 + min(ti, ntok - 1)) * a.nq + head) * HD;
      const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int s0 = 0; s0 < KS; ++s0)
        t.q[s0] = row_ok ? *(const bf16x8*)(qrow + g * 8 * KS + s0 * 8) : zero8;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) t.o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    t.m = -INFINITY;
    t.l = 0.f;

    // The item's turns of 64 keys, numbered from its first; this set takes turns set,
    // set + H, ...: `mine` of them, numbered j here.  Every set passes the same number of
    // barriers.
    const int key_begin = lo_all & ~63;
    const int nturns = ((pos_last - key_begin) >> 6) + 1;
    const int rounds = (nturns + H - 1) / H;
    const int mine = (nturns - set + H - 1) / H;
    const int kb_first = key_begin + 64 * set;
    const int last_page = pos_last >> lp;              // the last page the item may name
    // page ids of the four 16-key halves of the turn that will be sent for next (a page
    // beyond the item's last is the last again: its keys are masked; a page that a window
    // has let go reads page 0, masked as well).  Raw here: what is done with them waits for
    // the scalar loads, so it is done where they are used, a turn later.
    int nx[4];
    typedef int Ids4 __attribute__((ext_vector_type(4), aligned(4)));
    auto fetch_ids = [&](int kb) {
      const int i0 = kb >> lp;
      if (P16 && i0 + 3 <= last_page) {        // four consecutive pages: one scalar load
        const Ids4 ids = *(const Ids4 __attribute__((address_space(4)))*)(table + i0);
        nx[0] = ids[0]; nx[1] = ids[1]; nx[2] = ids[2]; nx[3] = ids[3];
      } else {
#pragma unroll
        for (int h = 0; h < 4; ++h) nx[h] = table[min((kb + 16 * h) >> lp, last_page)];
      }
    };
    fetch_ids(kb_first);

    auto issue = [&](int j, int to) {
      const int kb = kb_first + 64 * H * j;
      const Slots dst = ring + to * kBuf;
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
        const unsigned pa = max(nx[2 * sb], 0), pb = max(nx[2 * sb + 1], 0);
        const unsigned ia = (kb + 32 * sb) & (P - 1), ib = (kb + 32 * sb + 16) & (P - 1);
#pragma unroll
        for (int i = 0; i < L; ++i) {
          const unsigned page = second[i] ? pb : pa;
          const char* src = cbase[i] + (uint64_t)page * page_stride;
          if (!P16) src += (uint64_t)(second[i] ? ib : ia) * in_bytes[i];
          lds_dma16(src, &dst[sb * kSlots + wave + TILES * i][0]);
        }
      }
      fetch_ids(kb + 64 * H);
    };

    auto turn = [&](int j, int from, int to) {
      const int kb = kb_first + 64 * H * j;
      // this wave's share of turn j has arrived: at most the turn after it is in flight
      if (kAhead == 2 && j + 1 < mine) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * L));
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();      // every wave's share has, and every wave is through with turn j - 1
      asm volatile("" ::: "memory");
      // (the blocks of the turn `kAhead` on are sent for, into the buffer of the turn before
      // this one, after this turn's key operands have been asked for, so that LDS answers
      // meanwhile)
      auto send = [&]() { if (j + kAhead < mine) issue(j + kAhead, to); };
      if (j < mine && kb <= tile_last && kb + 63 >= tile_lo)
        tile_update64<HD, true>(t, ring + from * kBuf, lane, kb, scale_log2,
                                kb + 63 <= tile_first && kb >= tile_lo_last, g, send);
      else
        send();
    };

    // The query rows (both items') are waited for here, once (the empty statement uses
    // them), and not at their first use inside the loop, where the wait would be for every
    // block in flight as well; with them gone the vector memory counter counts the blocks'
    // loads alone.
#pragma unroll
    for (int s0 = 0; s0 < KS; ++s0) asm volatile("" : "+v"(t.q[s0]));
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (mine > 0) issue(0, 0);
    if (kAhead == 2 && mine > 1) issue(1, 1);
    // written out once per ring buffer so that every turn's buffers are constants
    if constexpr (NBUF == 2) {
      for (int j = 0; j < rounds; j += 2) {
        turn(j, 0, 1);
        if (j + 1 < rounds) turn(j + 1, 1, 0);
      }
    } else {
      for (int j = 0; j < rounds; j += 3) {
        turn(j, 0, 2);
        if (j + 1 < rounds) turn(j + 1, 1, 0);
        if (j + 2 < rounds) turn(j + 2, 2, 1);
      }
    }

    if constexpr (H == 2) {
      // The second set hands its partial result over in LDS, in the rings' space: values
      // [tile][element][lane], then the row statistics.
      float* lds_o = (float*)prefill_lds;
      float* lds_ml = lds_o + TILES * DB * 4 * kWave;
      static_assert(H * NBUF * kBuf * kWave * 16 >= (TILES * DB * 4 + TILES * 2) * kWave * 4, "merge area");
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
        const float sum = row_sum<HD>(t);
        if (row_ok)
          store_tile<HD>(t, sum, (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + head) * HD, g);
      }
    } else {
      const float sum = row_sum<HD>(t);
      if (row_ok)
        store_tile<HD>(t, sum, (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + head) * HD, g);
    }
    __syncthreads();       // before the next item's blocks are sent for into these buffers
  }
}

// Two waves a SIMD in every form, so a wave may take half the register file.  Four tiles
// an item: one workgroup of two sets beside rings of two buffers (128 KB).  Eight tiles:
// one workgroup of eight waves a unit beside a ring of three buffers (96 KB), two turns'
// blocks on their way, every block it brings in serving eight tiles.
template <int HD, bool P16>
__global__ __launch_bounds__(kWave * 8) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attention_prefill_wide_kernel4(AttentionMfmaArgs args, int paired) {
  attention_prefill_wide<HD, 2, 4, 2, P16>(args, paired);
}
template <int HD, bool P16>
__global__ __launch_bounds__(kWave * 8) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attention_prefill_wide_kernel8(AttentionMfmaArgs args, int paired) {
  attention_prefill_wide<HD, 1, 8, 3, P16>(args, paired);
}

// Query tiles per wavefront: as many as the register file holds accumulators for.
constexpr int tiles_per_wave(int hd) { return hd <= 32 ? 4 : (hd <= 64 ? 2 : 1); }

static int compute_units();
// Which kernel takes the long portions of head sizes 64 and 128.  2 (the default): turns of
// 64 keys for few items (two sets of waves per item) and for many (eight tiles an item),
// turns of 32 keys between; 1: for few items only; 0: turns of 32 keys everywhere; 3: eight
// tiles an item whatever the number of items (so that tests reach that kernel at small sizes).
static int g_prefill_variant = 2;
extern "C" void ts_attention_prefill_variant(int v) { g_prefill_variant = v; }

// Tokens one work item covers, in 16-row tiles, for a step of `tiles16` such tiles over
// `heads` key/value heads (x blocks of 16 query heads): one tile per wave of the kernels
// that share key blocks through LDS, i.e. four, or eight where four would give more than
// two items a compute unit (then eight waves share every block they bring in, and twice
// the waves fit beside the same rings); the register-only kernel's own count otherwise.
extern "C" int ts_attention_prefill_tiles(int head_dim, int page_size, int tiles16, int heads) {
  if (!(page_size >= 16 && (page_size & (page_size - 1)) == 0)) return tiles_per_wave(head_dim);
  const bool wide = g_prefill_variant >= 2 && head_dim % 64 == 0 && head_dim <= 128;
  const int64_t items4 = (int64_t)((tiles16 + 3) / 4) * heads;
  return wide && (g_prefill_variant == 3 || items4 >= 6 * compute_units()) ? 8 : 4;
}

int compute_units() {
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

// TILES 4: two sets of four waves per item (`paired` as above).  TILES 8: eight waves.
template <int HD, int TILES>
static int launch_prefill_wide(const AttentionMfmaArgs& args, int paired, hipStream_t stream) {
  const int heads = args.base.nkv * args.head_blocks;
  const dim3 grid((paired ? (args.num_tiles + 1) / 2 : args.num_tiles) * heads);
  const size_t lds = (size_t)(TILES == 8 ? 3 : 4) * 2 * (2 * (HD / 32) + HD / 16) * kWave * 16;
  const bool p16 = args.base.page_size == 16;
  void (*kernel)(AttentionMfmaArgs, int);
  if constexpr (TILES == 8)
    kernel = p16 ? attention_prefill_wide_kernel8<HD, true> : attention_prefill_wide_kernel8<HD, false>;
  else
    kernel = p16 ? attention_prefill_wide_kernel4<HD, true> : attention_prefill_wide_kernel4<HD, false>;
  static bool raised[2] = {false, false};     // per instantiation
  if (!raised[p16]) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      TS_FAIL("attention_prefill: cannot raise the LDS limit to %zu bytes", lds);
    raised[p16] = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kWave * 8), lds, stream, args, paired);
  return 0;
}

template <int HD>
static int launch_prefill_lds(const AttentionMfmaArgs& args, hipStream_t stream) {
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  if constexpr (HD % 64 == 0 && HD <= 128) {
    if (args.tiles_per_wave == 8) {
      if (g_prefill_variant < 1) TS_FAIL("attention_prefill: items of 8 tiles need the 64-key kernel");
      return launch_prefill_wide<HD, 8>(args, 0, stream);
    }
  }
  if (args.tiles_per_wave != 4) TS_FAIL("attention_prefill: the LDS kernel takes items of 4 tiles");
  if constexpr (HD % 64 == 0 && HD <= 128) {
    // Up to two items a compute unit: two sets of waves per item, and the items paired (a
    // long one and a short one per workgroup) once there are more items than units, so
    // that one round of workgroups of equal length fills the chip.  More: one set, three
    // workgroups a unit, longest first.  (Measured at 16 query and 8 key/value heads of
    // 128: 1,024 tokens 21.5 us with two sets unpaired, 25.3 paired; 1,536 tokens 34.0
    // paired, 35.7 unpaired; 2,048 tokens 42.6 paired, 48.8 with one set; 2,560 tokens 63.9
    // with one set, 92.7 with two sets paired, which then need a second round.)
    const int units = compute_units();
    if (g_prefill_variant >= 1 && items <= 2 * units)
      return launch_prefill_wide<HD, 4>(args, items > units, stream);
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
