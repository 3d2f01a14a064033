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
#include "attention.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kChunk = 128;    // keys per chunk; chunk c covers keys [c*kChunk, (c+1)*kChunk)

struct AttentionMfmaArgs {
  AttentionArgs base;
  const int* tiles;      // [num_tiles, 3]: batch entry, first flat token, tokens in tile
  float* partial_o;      // [items, num_splits, 16, hd]   (num_splits > 1)
  float* partial_ml;     // [items, num_splits, 16, 2]
  int num_tiles;
  int rows_per_token;    // query heads of a tile per token: min(group, 16)
  int head_blocks;       // ceil(group / 16)
  int num_splits;
  int cooperative;       // 1: a workgroup per item (few tiles), 0: a wavefront per item
};

// COOP = false: a wavefront per item walks its keys alone (many tiles: prompts).
// COOP = true: a workgroup per item; its four waves take every fourth 32-key block and
// merge in LDS (few tiles: decode), so a short context costs one round of loads.
template <int HD, bool COOP>
__global__ __launch_bounds__(256) void attention_mfma_kernel(AttentionMfmaArgs args) {
  constexpr int KS = (HD + 31) / 32;   // k-steps of the first product over the head size
  constexpr int DB = HD / 16;          // 16-row blocks of O^T
  const AttentionArgs& a = args.base;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int items = args.num_tiles * a.nkv * args.head_blocks;
  const int item = COOP ? blockIdx.x : blockIdx.x * 4 + wave;
  if (item >= items) return;
  const int tile = item / (a.nkv * args.head_blocks);
  const int kvh = (item / args.head_blocks) % a.nkv;
  const int hb = item % args.head_blocks;
  const int split = blockIdx.y;
  const int entry = args.tiles[tile * 3], tok0 = args.tiles[tile * 3 + 1],
            ntok = args.tiles[tile * 3 + 2];
  const int P = a.page_size;
  const int* table = a.table + (int64_t)entry * a.table_width;

  // my query row: column r of S^T
  const int ti = r / args.rows_per_token;
  const int hh = hb * 16 + r % args.rows_per_token;          // head inside the group
  const bool row_ok = ti < ntok && hh < group;
  const int token = tok0 + min(ti, ntok - 1);
  const int head = kvh * group + min(hh, group - 1);
  const int pos_r = row_ok ? a.positions[token] : -1;
  const int lo_r = (a.window > 0) ? max(0, pos_r - a.window + 1) : 0;

  // key range of the tile and my share of its chunks
  const int pos_first = a.positions[tok0], pos_last = a.positions[tok0 + ntok - 1];
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

  // Q^T operand: lane (r, g) holds Q[row r][g*8*KS + s*8 + j]
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16x4 zero4 = {0, 0, 0, 0};
  bf16x8 qv[KS];
  {
    const bf16_t* q = (const bf16_t*)a.q + ((int64_t)token * a.nq + head) * HD;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int e = g * 8 * KS + s * 8;
      qv[s] = (row_ok && e < HD) ? *(const bf16x8*)(q + e) : zero8;
    }
  }

  f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const bf16_t* kp = (const bf16_t*)a.k_pages;
  const bf16_t* vp = (const bf16_t*)a.v_pages;

  const int key_begin = max(c0 * kChunk, lo_tile & ~31) + (COOP ? wave * 32 : 0);
  const int key_end = min(c1 * kChunk, pos_last + 1);
  constexpr int kStride = COOP ? 128 : 32;

  // K operand of a 32-key block: lane (r, g) holds K[key blk*16 + r][g*8*KS + s*8 + j]
  bf16x8 kv[2][KS];
  auto load_k = [&](int kb) {
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int key = kb + blk * 16 + r;
      const int page = key <= pos_last ? table[key / P] : -1;
      const bf16_t* krow = kp + (((int64_t)max(page, 0) * a.nkv + kvh) * P + key % P) * HD;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int e = g * 8 * KS + s * 8;
        kv[blk][s] = (page >= 0 && e < HD) ? *(const bf16x8*)(krow + e) : zero8;
      }
    }
  };
  if (key_begin < key_end) load_k(key_begin);

  for (int kb = key_begin; kb < key_end; kb += kStride) {
    // ---- V^T operand of this block, asked for before the scores are worked out.
    //      Slot (g, j) of the reduction stands for key kb + g*4 + j (j < 4) or
    //      kb + 16 + g*4 + j - 4, in both operands of the second product.
    bf16x4 vv[2][DB];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int key4 = kb + blk * 16 + g * 4;
      const int page = key4 <= pos_last ? table[key4 / P] : -1;
      const bf16_t* vcol = vp + ((int64_t)max(page, 0) * a.nkv + kvh) * HD * P + key4 % P;
#pragma unroll
      for (int db = 0; db < DB; ++db)
        vv[blk][db] = page >= 0 ? *(const bf16x4*)(vcol + (int64_t)(db * 16 + r) * P) : zero4;
    }
    // ---- S^T for 32 keys: two blocks of 16
    f32x4 st[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      st[blk] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s)
        st[blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv[blk][s], qv[s], st[blk], 0, 0, 0);
    }
    // ---- keys of the next block, in flight during the softmax and the second product
    if (kb + kStride < key_end) load_k(kb + kStride);
    // ---- mask, running maximum and sum of my query (column r; lanes r, r+16, r+32, r+48)
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int key = kb + blk * 16 + g * 4 + t;
        const bool vis = row_ok && key <= pos_r && key >= lo_r;
        const float s = vis ? st[blk][t] * a.scale : -INFINITY;
        sv[blk * 4 + t] = s;
        mx = fmaxf(mx, s);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m, mx);
    const bool any = m_new != -INFINITY;
    const float corr = any ? __expf(m - m_new) : 1.f;
    float ps = 0.f;
    bf16x8 pv;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = any ? __expf(sv[i] - m_new) : 0.f;
      ps += p;
      pv[i] = (bf16_t)p;
    }
    ps += __shfl_xor(ps, 16, kWave);
    ps += __shfl_xor(ps, 32, kWave);
    l = l * corr + ps;
    m = m_new;
    // ---- O^T += V^T P^T
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x4 v0 = vv[0][db], v1 = vv[1][db];
      const bf16x8 vfull = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
      f32x4 acc = o[db];
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[t] *= corr;
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfull, pv, acc, 0, 0, 0);
    }
  }

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
      const float w0 = __expf(m - M);
      l *= w0;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int t = 0; t < 4; ++t) o[db][t] *= w0;
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        const float mw = s_ml[w][lane][0];
        if (mw == -INFINITY) continue;
        const float ww = __expf(mw - M);
        l += s_ml[w][lane][1] * ww;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const f32x4 ow = s_o[w][db][lane];
#pragma unroll
          for (int t = 0; t < 4; ++t) o[db][t] += ow[t] * ww;
        }
      }
      m = M;
    }
  }

  // lane (r, g) holds O^T[d = db*16 + g*4 + t][row r]
  if (args.num_splits == 1) {
    if (!row_ok) return;
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16_t* out = (bf16_t*)a.out + ((int64_t)token * a.nq + head) * HD;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 ov = {(bf16_t)(o[db][0] * inv), (bf16_t)(o[db][1] * inv),
                   (bf16_t)(o[db][2] * inv), (bf16_t)(o[db][3] * inv)};
      *(bf16x4*)(out + db * 16 + g * 4) = ov;
    }
  } else {
    const int64_t slot = ((int64_t)item * args.num_splits + split) * 16 + r;
    if (row_ok) {
      float* po = args.partial_o + slot * HD;
#pragma unroll
      for (int db = 0; db < DB; ++db) *(f32x4*)(po + db * 16 + g * 4) = o[db];
    }
    if (g == 0) {
      args.partial_ml[slot * 2] = m;
      args.partial_ml[slot * 2 + 1] = l;
    }
  }
}

// Merge the splits of every tile: out = sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M),
// splits taken in order.  One workgroup per item, thread (row, column group).
template <int HD>
__global__ __launch_bounds__(256) void attention_merge_kernel(AttentionMfmaArgs args) {
  const AttentionArgs& a = args.base;
  const int item = blockIdx.x;
  const int tile = item / (a.nkv * args.head_blocks);
  const int kvh = (item / args.head_blocks) % a.nkv;
  const int hb = item % args.head_blocks;
  const int tok0 = args.tiles[tile * 3 + 1], ntok = args.tiles[tile * 3 + 2];
  const int group = a.nq / a.nkv;
  const int r = threadIdx.x / 16, dc = threadIdx.x % 16;
  const int ti = r / args.rows_per_token, hh = hb * 16 + r % args.rows_per_token;
  if (ti >= ntok || hh >= group) return;
  const int64_t base = (int64_t)item * args.num_splits * 16 + r;
  // splits beyond the tile's chunks hold nothing: same arithmetic as the first kernel
  const int pos_first = a.positions[tok0], pos_last = a.positions[tok0 + ntok - 1];
  const int lo_tile = (a.window > 0) ? max(0, pos_first - a.window + 1) : 0;
  const int nchunks = pos_last / kChunk - lo_tile / kChunk + 1;
  const int per = (nchunks - 1 + args.num_splits) / args.num_splits;
  const int used = min(args.num_splits, (nchunks + per - 1) / per);
  float M = -INFINITY;
  for (int s = 0; s < used; ++s)
    M = fmaxf(M, args.partial_ml[(base + (int64_t)s * 16) * 2]);
  float L = 0.f;
  float acc[HD / 16] = {};
  for (int s = 0; s < used; ++s) {
    const int64_t slot = base + (int64_t)s * 16;
    const float ms = args.partial_ml[slot * 2];
    if (ms == -INFINITY) continue;
    const float w = __expf(ms - M);
    L += args.partial_ml[slot * 2 + 1] * w;
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) acc[i] += args.partial_o[slot * HD + i * 16 + dc] * w;
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  bf16_t* out = (bf16_t*)a.out + ((int64_t)(tok0 + ti) * a.nq + kvh * group + hh) * HD;
#pragma unroll
  for (int i = 0; i < HD / 16; ++i) out[i * 16 + dc] = (bf16_t)(acc[i] * inv);
}

int ts_check_attention_args(const AttentionArgs& a, const char* who);

template <int HD>
static int launch_mfma(const AttentionMfmaArgs& args, hipStream_t stream) {
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  if (args.cooperative) {
    hipLaunchKernelGGL((attention_mfma_kernel<HD, true>), dim3(items, args.num_splits),
                       dim3(256), 0, stream, args);
  } else {
    hipLaunchKernelGGL((attention_mfma_kernel<HD, false>), dim3((items + 3) / 4, args.num_splits),
                       dim3(256), 0, stream, args);
  }
  if (args.num_splits > 1)
    hipLaunchKernelGGL(attention_merge_kernel<HD>, dim3(items), dim3(256), 0, stream, args);
  return 0;
}

extern "C" int ts_attention_mfma_chunk() { return kChunk; }

extern "C" int ts_attention_mfma(const AttentionMfmaArgs* p, hipStream_t stream) {
  AttentionMfmaArgs args = *p;
  const AttentionArgs& a = args.base;
  if (a.num_tokens <= 0 || args.num_tiles <= 0) return 0;
  if (ts_check_attention_args(a, "attention_mfma")) return -1;
  if (a.hd % 16) TS_FAIL("attention_mfma: head_dim=%d must be a multiple of 16", a.hd);
  if (a.page_size % 4) TS_FAIL("attention_mfma: page_size=%d must be a multiple of 4", a.page_size);
  const int group = a.nq / a.nkv;
  if (args.rows_per_token != (group < 16 ? group : 16) ||
      args.head_blocks != (group + 15) / 16)
    TS_FAIL("attention_mfma: rows_per_token/head_blocks do not fit a group of %d", group);
  if (args.num_splits < 1 || args.num_splits > 65535) TS_FAIL("attention_mfma: num_splits=%d", args.num_splits);
  if (args.num_splits > 1 && (!args.partial_o || !args.partial_ml))
    TS_FAIL("attention_mfma: splits need partial buffers");
  if (((uintptr_t)a.q | (uintptr_t)a.out | (uintptr_t)a.k_pages | (uintptr_t)a.v_pages) & 15)
    TS_FAIL("attention_mfma: tensors must be 16-byte aligned");
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
