// Paged attention for a decode step (one new token per batch entry) on the matrix cores,
// bfloat16, page sizes that are powers of two from 16 up.
//
// One workgroup owns a tile: the query heads of one key/value head of one entry (up to
// 16 rows) and, with `num_splits` > 1, one share of the entry's 128-key chunks.  Its NW
// waves take every NW-th block of 32 keys with the loads and arithmetic of
// attention_core.h and merge in LDS, so up to a few thousand keys cost one launch and no
// partial results in memory; longer contexts are split over workgroups and merged by
// attention_merge, or by the workgroup of the item that finishes last (below).
//
// Fused form (FUSED): what lies between the q/k/v projection and attention happens here
// as well, so a decode layer needs no kernel for it.  Every wave reads its query rows
// from the projection's output, applies the per-head RMSNorm and the rotation in float32
// in the registers of the operand layout (a head's four lanes hold a quarter of it each;
// the rotation's partner of element d, d +- hd/2, is in the lane 32 further), and rounds
// to bfloat16 as the unfused kernel stores it.  The last wave of a workgroup does this
// for the others instead of walking (they have their first key block in flight and no
// registers to spare) and hands the rows over in LDS.  In the first split's workgroup it
// also prepares the new key, writes key and value to their cache slot and gives them to
// the merge as one more partial sum (score q.k, weight 1, value v) instead of anyone
// reading them back; the keys walked from the cache end one before the new position.
// (A wave of its own also because a store in flight makes every later wait for a load a
// wait for all of them: loads and stores share one counter.)
#include "attention_core.h"

struct AttentionDecodeArgs {
  AttentionMfmaArgs m;      // tiles = null, num_tiles = entries = tokens
  const bf16_t* qkv;        // fused: [T, (nq + 2 * kv_in_row) * hd]; else null
  const float* q_weight;    // [hd] or null: no norm
  const float* k_weight;
  const float* cos;         // [max_pos, hd / 2] or null: no rotation
  const float* sin;
  float eps;
  int kv_in_row;            // nkv: the row brings k and v, written to the cache here; 0: q only
  int defer_merge;          // 1: with more than one split, leave the partial results unmerged
                            // (ts_gemm_tail_merged_bf16 or ts_attention_merge takes them)
  unsigned* arrivals;       // [items] zeros, or null.  Given (and the merge not deferred), the
                            // workgroup of an item that finishes last merges the splits itself
                            // and leaves the item's count at zero: no merge kernel
};

int launch_attention_merge(const AttentionMfmaArgs& args, hipStream_t stream);

template <int HD> constexpr int decode_waves() { return HD <= 128 ? 8 : 4; }

// Norm and rotation of one head vector held in the query operand layout: `v` has the
// lane's HD/4 elements [g*HD/4 + s*8 + j] as they come from the projection and gets them
// back normed, rotated and rounded to bfloat16.  The elements are widened to float32 twice
// (for the sum of squares, then slice by slice) rather than kept widened: registers are
// short here, next to the first key block in flight.  `w` and `cs` are the lane's slices
// of the norm weight and of the position's cos and sin, loaded by the caller together
// with everything else the kernel starts with.
template <int HD>
__device__ __forceinline__ void prepare_head(bf16x8 (&v)[HD / 32], bool live, bool weight,
                                             const f32x4 (&w)[HD / 32][2], float eps,
                                             const f32x4 (&cs)[HD / 32][4], bool rotate, int g) {
  constexpr int KS = HD / 32;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  float rstd = 1.f;
  if (weight) {
    float ss = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)v[s][j] * (float)v[s][j];
    ss = col4_sum(live ? ss : 0.f);
    rstd = rsqrtf(ss / (float)HD + eps);
  }
  const bool first = g < 2;            // elements below hd/2
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = (float)v[s][j];
    if (weight) {
#pragma unroll
      for (int j = 0; j < 4; ++j) { x[j] *= rstd * w[s][0][j]; x[4 + j] *= rstd * w[s][1][j]; }
    }
    if (rotate) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // the partner's element, from the lane 32 further: a row-swap instruction, fed
        // the same value twice, returns each half's value in both halves
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x[j]), __float_as_uint(x[j]),
                                                         false, false);
        const float other = __uint_as_float(first ? sw[1] : sw[0]);
        const float c = cs[s][j / 4][j % 4], sn = cs[s][2 + j / 4][j % 4];
        x[j] = first ? x[j] * c - other * sn : x[j] * c + other * sn;
      }
    }
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (bf16_t)x[j];
    v[s] = live ? o : zero8;
  }
}

// A float32 to memory, and back, at device scope without ordering: such accesses pass the
// caches that another XCD does not share.
__device__ __forceinline__ void store_past_caches(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_past_caches(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The merge of attention_merge_kernel (same order, same arithmetic per element, so the same
// bits) by the THREADS threads of one workgroup, over the `used` first splits of one item:
// slot (first_slot + split * 16 + row) holds a row's statistics and HD partial sums.  A
// thread takes two elements at a time and asks for all of a group of eight splits before it
// uses the first.
template <int HD, int THREADS>
__device__ __forceinline__ void merge_splits_here(const float* partial_o, const float* partial_ml,
                                                  int64_t first_slot, int used, int rows, bf16_t* out) {
  constexpr int kGroup = 8, E = 2;
  const int count = rows * HD;
  for (int e0 = threadIdx.x; e0 < count; e0 += E * THREADS) {
    int row[E], d[E];
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const int e = min(e0 + k * THREADS, count - 1);    // past the end: the last again, not stored
      row[k] = e / HD;
      d[k] = e % HD;
    }
    float M[E], L[E], acc[E];
#pragma unroll
    for (int k = 0; k < E; ++k) { M[k] = -INFINITY; L[k] = 0.f; acc[k] = 0.f; }
    for (int s0 = 0; s0 < used; s0 += kGroup) {
      float ms[E][kGroup], ls[E][kGroup], part[E][kGroup];
#pragma unroll
      for (int j = 0; j < kGroup; ++j)
#pragma unroll
        for (int k = 0; k < E; ++k) {
          const int64_t slot = first_slot + (int64_t)min(s0 + j, used - 1) * 16 + row[k];
          ms[k][j] = load_past_caches(partial_ml + slot * 2);
          ls[k][j] = load_past_caches(partial_ml + slot * 2 + 1);
          part[k][j] = load_past_caches(partial_o + slot * HD + d[k]);
        }
#pragma unroll
      for (int k = 0; k < E; ++k) {
        float Mg = M[k];
#pragma unroll
        for (int j = 0; j < kGroup; ++j) Mg = (s0 + j < used) ? fmaxf(Mg, ms[k][j]) : Mg;
        if (Mg == -INFINITY) continue;
        const float keep = __builtin_amdgcn_exp2f(M[k] - Mg);
        L[k] *= keep;
        acc[k] *= keep;
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
          const bool live = s0 + j < used && ms[k][j] != -INFINITY;
          const float w = live ? __builtin_amdgcn_exp2f(ms[k][j] - Mg) : 0.f;
          L[k] += live ? ls[k][j] * w : 0.f;
          acc[k] += live ? part[k][j] * w : 0.f;
        }
        M[k] = Mg;
      }
    }
#pragma unroll
    for (int k = 0; k < E; ++k) {
      if (e0 + k * THREADS >= count) break;
      const float inv = L[k] > 0.f ? 1.f / L[k] : 0.f;
      out[(int64_t)row[k] * HD + d[k]] = (bf16_t)(acc[k] * inv);
    }
  }
}

template <int HD, bool FUSED>
__global__ __launch_bounds__(decode_waves<HD>() * kWave) void attention_decode_kernel(
    AttentionDecodeArgs args) {
  constexpr int NW = decode_waves<HD>();
  constexpr int DB = HD / 16, KS = (HD + 31) / 32;
  const AttentionMfmaArgs& ma = args.m;
  const AttentionArgs& a = ma.base;
  const int wave = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int item = blockIdx.x, split = blockIdx.y;
  const int entry = item / (a.nkv * ma.head_blocks);
  const int kvh = (item / ma.head_blocks) % a.nkv;
  const int hb = item % ma.head_blocks;
  const int token = entry;
  const int* table = a.table + (int64_t)entry * a.table_width;

  const int hh = hb * 16 + r;                                 // head inside the group
  const bool row_ok = r < ma.rows_per_token && hh < group;
  const int head = kvh * group + min(hh, group - 1);
  // Fused form: the last wave does not walk; it prepares the query rows for the others.
  // In the first split the wave before it does not walk either: it takes the new key,
  // side by side with the last wave's work on the queries.  What those two need from
  // memory is asked for first of all, before anything else is worked out: the head
  // vector and the norm weight at once, cos and sin as soon as the position is here.
  const bool new_key = FUSED && args.kv_in_row > 0;           // the step's own key is not in the cache yet
  const bool adds_new = new_key && split == 0;                // this workgroup brings the new key in
  const bool prep_wave = FUSED && wave == NW - 1;
  const bool key_wave = adds_new && wave == NW - 2;
  const bool walker = !prep_wave && !key_wave;
  const int pos_lane = a.positions[token];
  bf16x8 kq[KS];            // the head vector such a wave prepares: query rows, or the new key
  f32x4 cs[KS][4];          // cos (2 x 4) and sin (2 x 4) of the lane's elements
  f32x4 pw[KS][2];          // norm weight
  const float* prep_weight = nullptr;
  if constexpr (FUSED) {
    if (!walker) {
      prep_weight = prep_wave ? args.q_weight : args.k_weight;
      const bf16_t* src = args.qkv + (int64_t)token * ((a.nq + 2 * args.kv_in_row) * HD) +
                          (int64_t)(prep_wave ? head : a.nq + kvh) * HD + g * (HD / 4);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        kq[s] = *(const bf16x8*)(src + s * 8);
        if (prep_weight) {
          pw[s][0] = *(const f32x4*)(prep_weight + g * (HD / 4) + s * 8);
          pw[s][1] = *(const f32x4*)(prep_weight + g * (HD / 4) + s * 8 + 4);
        }
      }
    }
  }
  const int pos = uniform(pos_lane);
  if constexpr (FUSED) {
    if (!walker && args.cos != nullptr) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int64_t i = (int64_t)pos * (HD / 2) + (g & 1) * (HD / 4) + s * 8;
        cs[s][0] = *(const f32x4*)(args.cos + i);
        cs[s][1] = *(const f32x4*)(args.cos + i + 4);
        cs[s][2] = *(const f32x4*)(args.sin + i);
        cs[s][3] = *(const f32x4*)(args.sin + i + 4);
      }
    }
  }
  const int last = new_key ? pos - 1 : pos;                   // last key walked from the cache
  const int lo = (a.window > 0) ? max(0, pos - a.window + 1) : 0;
  // chunks of this split: the arithmetic of attention_merge (from pos, not from last)
  const int c_first = lo / kChunk, c_last = pos / kChunk;
  const int per = (c_last - c_first + ma.num_splits) / ma.num_splits;
  const int c0 = c_first + split * per, c1 = min(c0 + per, c_last + 1);
  if (c0 > c_last) {   // more splits than chunks: a neutral partial, no data touched
    if (g == 0 && wave == 0) {
      const int64_t slot = ((int64_t)item * ma.num_splits + split) * 16 + r;
      ma.partial_ml[slot * 2] = -INFINITY;
      ma.partial_ml[slot * 2 + 1] = 0.f;
    }
    return;
  }

  const int walkers = FUSED ? NW - 1 - (adds_new ? 1 : 0) : NW;

  TileState<HD> t;
  t.pos = row_ok ? last : -1;
  t.lo = lo;
  const float scale_log2 = a.scale * 1.44269504088896341f;
  const int stride = walkers * 32;
  const int key_begin = max(c0 * kChunk, lo & ~31) + wave * 32;
  const int key_end = (prep_wave || key_wave) ? 0 : min(c1 * kChunk, last + 1);
  PageCursor cur{(ConstTable)table, a.page_size, last, -1, -1};
  KvBlock<HD> A, B;
  // head sizes in whole 32-element slices take the blocks with 16-byte value loads
  constexpr bool kWide = HD % 32 == 0;
  auto load_block = [&](KvBlock<HD>& b, int kb) {
    if constexpr (kWide) load_kv_block_wide<HD>(b, a, cur, kvh, kb, stride, r, g);
    else load_kv_block<HD, true>(b, a, table, cur, kvh, kb, stride, r, g);
  };

  if constexpr (FUSED) {
    // The last wave prepares the query rows for all of them (through LDS): the others
    // have their first key block in flight meanwhile and no registers to spare for the
    // cos, sin and norm weight slices.
    __shared__ bf16x8 s_q[KS][kWave];
    const int row_width = (a.nq + 2 * args.kv_in_row) * HD;
    const bf16_t* row = args.qkv + (int64_t)token * row_width;
    const bool rotate = args.cos != nullptr;
    if (walker) {
      cur.start(key_begin);
      if (key_begin < key_end) load_block(A, key_begin);
    }
    if (!walker) {
      prepare_head<HD>(kq, prep_wave ? row_ok : true, prep_weight != nullptr, pw, args.eps, cs, rotate, g);
      if (prep_wave) {
#pragma unroll
        for (int s = 0; s < KS; ++s) s_q[s][lane] = kq[s];
      }
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < KS; ++s) t.q[s] = s_q[s][lane];
#pragma unroll
    for (int db = 0; db < DB; ++db) t.o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    t.m = -INFINITY;
    t.l = 0.f;

    if (key_wave) {
      const bf16_t* vrow = row + (int64_t)(a.nq + args.kv_in_row + kvh) * HD;
      float dot = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int j = 0; j < 8; ++j) dot += (float)t.q[s][j] * (float)kq[s][j];
      // this wave's partial: one key with weight 1
      t.m = col4_sum(dot) * scale_log2;
      t.l = g == 0 ? 1.f : 0.f;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x4 v = *(const bf16x4*)(vrow + db * 16 + g * 4);
        t.o[db] = f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
      }
      if (hb == 0) {   // into the cache slot of position pos, once per key/value head
        const int P = a.page_size;
        const int page = uniform(table[pos >> __builtin_ctz(P)]);
        const int off = pos & (P - 1);
        if (page >= 0) {
          bf16_t* kdst = (bf16_t*)a.k_pages + (((int64_t)page * a.nkv + kvh) * P + off) * HD;
          if (r == 0) {
#pragma unroll
            for (int s = 0; s < KS; ++s) *(bf16x8*)(kdst + g * (HD / 4) + s * 8) = kq[s];
          }
          bf16_t* vdst = (bf16_t*)a.v_pages + ((int64_t)page * a.nkv + kvh) * HD * P + off;
          if (r < DB) {
            const bf16x4 v = *(const bf16x4*)(vrow + r * 16 + g * 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) vdst[(int64_t)(r * 16 + g * 4 + i) * P] = v[i];
          }
        }
        // vmcnt(0): no store is in flight where this path joins the walkers' (this wave
        // has nothing else to do meanwhile)
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
    }
  } else {
    cur.start(key_begin);
    if (key_begin < key_end) load_block(A, key_begin);
    load_query<HD>(t, (const bf16_t*)a.q + ((int64_t)token * a.nq + head) * HD, row_ok, g);
  }

  for (int kb = key_begin; kb < key_end; kb += 2 * stride) {
    if (kb + stride < key_end)
      load_block(B, kb + stride);
    tile_update<HD, false, kWide>(t, A, kb, scale_log2, kb + 31 <= last && kb >= lo, g);
    if (kb + stride >= key_end) break;
    if (kb + 2 * stride < key_end)
      load_block(A, kb + 2 * stride);
    tile_update<HD, false, kWide>(t, B, kb + stride, scale_log2, kb + stride + 31 <= last && kb + stride >= lo, g);
  }
  f32x4 (&o)[DB] = t.o;
  float m = t.m, l = row_sum<HD>(t);

  // The waves' partial results (the new key's among them) all go to LDS, and every wave
  // merges, in wave order, its share of the head's blocks of 16 elements and stores that
  // share: the merge is as wide as the workgroup instead of one wave's long tail.
  extern __shared__ __attribute__((aligned(16))) unsigned char merge_lds[];
  float (*s_ml)[kWave][2] = (float (*)[kWave][2])merge_lds;                        // [NW]
  f32x4 (*s_o)[DB][kWave] = (f32x4 (*)[DB][kWave])(merge_lds + NW * kWave * 2 * 4);  // [NW]
  s_ml[wave][lane][0] = m;
  s_ml[wave][lane][1] = l;
#pragma unroll
  for (int db = 0; db < DB; ++db) s_o[wave][db][lane] = o[db];
  __syncthreads();
  constexpr int kShare = (DB + NW - 1) / NW;         // blocks of 16 elements per wave
  // Merge by the last to finish: the partial results go out past the caches (their readers
  // may sit on another XCD, behind another L2), each wave waits until its own have been
  // taken, the workgroup counts itself in at the item's counter, and the one that finds
  // all the others there reads every split's result back the same way and merges them in
  // the order and arithmetic of attention_merge.  Nothing here needs the caches written
  // back or dropped, which is what release and acquire at device scope would cost.
  const bool fold = ma.num_splits > 1 && !args.defer_merge && args.arrivals != nullptr;
  const bool has_share = wave * kShare < DB;
  if (!has_share && !fold) return;
  const int64_t slot = ((int64_t)item * ma.num_splits + split) * 16 + r;
  if (has_share) {
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, s_ml[w][lane][0]);
    float ww[NW];
    l = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = s_ml[w][lane][0];
      // a wave that saw no key has m = -inf (and so has everyone if M is): weight 0
      ww[w] = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - M);
      l += s_ml[w][lane][1] * ww[w];
    }
    m = M;
    // lane (r, g) holds O^T[d = db*16 + g*4 + i][row r]
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int k = 0; k < kShare; ++k) {
      const int db = wave * kShare + k;
      if (db >= DB) break;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const f32x4 ow = s_o[w][db][lane];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += ww[w] == 0.f ? 0.f : ow[i] * ww[w];   // never 0 * garbage
      }
      if (!row_ok) continue;
      if (ma.num_splits == 1) {
        bf16x4 ov = {(bf16_t)(acc[0] * inv), (bf16_t)(acc[1] * inv), (bf16_t)(acc[2] * inv),
                     (bf16_t)(acc[3] * inv)};
        *(bf16x4*)((bf16_t*)a.out + ((int64_t)token * a.nq + head) * HD + db * 16 + g * 4) = ov;
      } else if (fold) {
#pragma unroll
        for (int i = 0; i < 4; ++i) store_past_caches(ma.partial_o + slot * HD + db * 16 + g * 4 + i, acc[i]);
      } else {
        *(f32x4*)(ma.partial_o + slot * HD + db * 16 + g * 4) = acc;
      }
    }
    if (ma.num_splits > 1 && wave == 0 && g == 0) {
      if (fold) {
        store_past_caches(ma.partial_ml + slot * 2, m);
        store_past_caches(ma.partial_ml + slot * 2 + 1, l);
      } else {
        ma.partial_ml[slot * 2] = m;
        ma.partial_ml[slot * 2 + 1] = l;
      }
    }
  }
  if (!fold) return;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);                     // this wave's stores have been taken
  __shared__ unsigned s_before;
  __syncthreads();
  if (threadIdx.x == 0)
    s_before = __hip_atomic_fetch_add(args.arrivals + item, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  // splits that hold chunks: the arithmetic of attention_merge; the others have returned
  const int nchunks = c_last - c_first + 1;
  const int used = min(ma.num_splits, (nchunks + per - 1) / per);
  if ((int)s_before + 1 != used) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (threadIdx.x == 0)
    __hip_atomic_store(args.arrivals + item, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int rows = min(ma.rows_per_token, group - hb * 16);
  bf16_t* out = (bf16_t*)a.out + ((int64_t)token * a.nq + kvh * group + hb * 16) * HD;
  merge_splits_here<HD, NW * kWave>(ma.partial_o, ma.partial_ml, (int64_t)item * ma.num_splits * 16,
                                    used, rows, out);
}

int ts_check_attention_mfma_args(const AttentionMfmaArgs& args, const char* who);

template <int HD>
static int launch_decode(const AttentionDecodeArgs& args, hipStream_t stream) {
  const AttentionMfmaArgs& m = args.m;
  const int items = m.num_tiles * m.base.nkv * m.head_blocks;
  const dim3 grid(items, m.num_splits), block(decode_waves<HD>() * kWave);
  // the merge area: per wave its row statistics and HD/16 blocks of partial sums
  const size_t lds = (size_t)decode_waves<HD>() * (kWave * 2 * 4 + (HD / 16) * kWave * 16);
  if (args.qkv) {
    if constexpr (HD % 32 == 0) {
      auto kernel = attention_decode_kernel<HD, true>;
      static bool raised = false;     // per head size
      if (lds > 48 * 1024 && !raised) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
          TS_FAIL("attention_decode: cannot raise the LDS limit to %zu bytes", lds);
        raised = true;
      }
      hipLaunchKernelGGL(kernel, grid, block, lds, stream, args);
    } else {
      TS_FAIL("attention_decode: the fused form needs a head size that is a multiple of 32");
    }
  } else {
    auto kernel = attention_decode_kernel<HD, false>;
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
      if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds) != hipSuccess)
        TS_FAIL("attention_decode: cannot raise the LDS limit to %zu bytes", lds);
      raised = true;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, args);
  }
  if (m.num_splits > 1 && !args.defer_merge && !args.arrivals) return launch_attention_merge(m, stream);
  return 0;
}

// 1 if ts_attention_decode takes this head size and page size (fused: its fused form).
extern "C" int ts_attention_decode_fits(int hd, int page_size, int fused) {
  if (hd < 16 || hd > 256 || hd % 16 || (fused && hd % 32)) return 0;
  return page_size >= 16 && (page_size & (page_size - 1)) == 0;
}

extern "C" int ts_attention_decode(const AttentionDecodeArgs* p, hipStream_t stream) {
  AttentionDecodeArgs args = *p;
  const AttentionMfmaArgs& m = args.m;
  const AttentionArgs& a = m.base;
  if (a.num_tokens <= 0) return 0;
  if (ts_check_attention_mfma_args(m, "attention_decode")) return -1;
  if (m.tiles || m.num_tiles != a.num_tokens || a.num_tokens != a.num_entries)
    TS_FAIL("attention_decode: one token per entry and no tile list (tokens %d, entries %d)",
            a.num_tokens, a.num_entries);
  if (!ts_attention_decode_fits(a.hd, a.page_size, args.qkv != nullptr))
    TS_FAIL("attention_decode: head_dim=%d, page_size=%d not served", a.hd, a.page_size);
  if (m.num_splits < 1 || m.num_splits > 65535) TS_FAIL("attention_decode: num_splits=%d", m.num_splits);
  if (m.num_splits > 1 && (!m.partial_o || !m.partial_ml))
    TS_FAIL("attention_decode: splits need partial buffers");
  if (args.qkv) {
    if ((uintptr_t)args.qkv & 15) TS_FAIL("attention_decode: qkv must be 16-byte aligned");
    if ((args.cos == nullptr) != (args.sin == nullptr)) TS_FAIL("attention_decode: cos and sin go together");
    if (args.kv_in_row != 0 && args.kv_in_row != a.nkv)
      TS_FAIL("attention_decode: the row brings %d key heads, the cache has %d", args.kv_in_row, a.nkv);
  } else if (!a.q) {
    TS_FAIL("attention_decode: neither q nor qkv");
  }
  int rc = 0;
  switch (a.hd) {
#define TS_CASE(HD) case HD: rc = launch_decode<HD>(args, stream); break;
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_decode: head_dim=%d not built", a.hd);
  }
  if (rc) return rc;
  TS_CHECK_LAUNCH("attention_decode");
  return 0;
}
