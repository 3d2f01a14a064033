// What happens to q, k and v between their projection and attention: per-head RMSNorm
// on q and k, rotate-half position rotation, and the write of k and v into cache pages.
// One wavefront per (token, head); sums and the rotation in float32.
#include "common.h"

struct QkPrepareArgs {
  const void* qkv;       // [T, (nq + 2*nkv) * hd]
  void* q_out;           // [T, nq, hd]
  void* k_dst;           // pages [num_pages, nkv, P, hd], or flat [T, nkv, hd] if !paged
  void* v_dst;           // pages [num_pages, nkv, hd, P] (transposed), or flat [T, nkv, hd]
  const float* q_weight; // [hd] or null: no norm
  const float* k_weight;
  const float* cos;      // [max_pos, hd/2] or null: no rotation
  const float* sin;
  const int* positions;      // [T]
  const int* entry_of_token; // [T]
  const int* table;          // [B, table_width]
  int table_width;
  int num_tokens, nq, nkv, hd, page_size, max_pos;
  int paged;             // 1: k_dst/v_dst are cache pages; 0: flat buffers
  int store_kv;          // 0: q only
  float eps;
};

template <typename T, typename TC>
__global__ void qk_prepare_kernel(QkPrepareArgs a) {
  const int lane = threadIdx.x % kWave;
  const int heads = a.nq + (a.store_kv ? 2 * a.nkv : 0);
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= (int64_t)a.num_tokens * heads) return;
  const int t = (int)(item / heads);
  const int h = (int)(item % heads);
  const int hd = a.hd, half = hd / 2;
  const int row_width = (a.nq + 2 * a.nkv) * hd;
  const int pos = a.positions[t];

  int src_head;       // head index inside the qkv row
  int kind;           // 0 q, 1 k, 2 v
  if (h < a.nq) { kind = 0; src_head = h; }
  else if (h < a.nq + a.nkv) { kind = 1; src_head = h; }
  else { kind = 2; src_head = h; }
  const T* src = (const T*)a.qkv + (int64_t)t * row_width + (int64_t)src_head * hd;

  // destination row of hd elements
  int64_t dst_off = -1;
  int v_stride = 1;   // distance between consecutive head elements of a value row
  if (kind == 0) {
    dst_off = ((int64_t)t * a.nq + h) * hd;
  } else {
    const int kvh = kind == 1 ? h - a.nq : h - a.nq - a.nkv;
    if (a.paged) {
      const int page = a.table[(int64_t)a.entry_of_token[t] * a.table_width + pos / a.page_size];
      if (page >= 0) {
        if (kind == 1) {
          dst_off = (((int64_t)page * a.nkv + kvh) * a.page_size + pos % a.page_size) * hd;
        } else {
          dst_off = ((int64_t)page * a.nkv + kvh) * a.page_size * hd + pos % a.page_size;
          v_stride = a.page_size;
        }
      }
    } else {
      dst_off = ((int64_t)t * a.nkv + kvh) * hd;
    }
  }
  if (dst_off < 0) return;   // no page behind this position: nothing is written

  if (kind == 2) {
    TC* dst = (TC*)a.v_dst + dst_off;
    for (int i = lane; i < hd; i += kWave)
      dst[(int64_t)i * v_stride] = from_f32<TC>(to_f32(src[i]));
    return;
  }

  const float* w = kind == 0 ? a.q_weight : a.k_weight;
  float ss = 0.f;
  for (int i = lane; i < hd; i += kWave) { const float v = to_f32(src[i]); ss += v * v; }
  const float rstd = w ? rsqrtf(wave_sum(ss) / (float)hd + a.eps) : 1.f;

  const float* cos = a.cos ? a.cos + (int64_t)pos * half : nullptr;
  const float* sin = a.sin ? a.sin + (int64_t)pos * half : nullptr;
  for (int i = lane; i < half; i += kWave) {
    float re = to_f32(src[i]), im = to_f32(src[i + half]);
    if (w) { re = re * rstd * w[i]; im = im * rstd * w[i + half]; }
    float o_re = re, o_im = im;
    if (cos) {
      const float c = cos[i], s = sin[i];
      o_re = re * c - im * s;
      o_im = im * c + re * s;
    }
    if (kind == 0) {
      T* dst = (T*)a.q_out + dst_off;
      dst[i] = from_f32<T>(o_re);
      dst[i + half] = from_f32<T>(o_im);
    } else {
      TC* dst = (TC*)a.k_dst + dst_off;
      dst[i] = from_f32<TC>(o_re);
      dst[i + half] = from_f32<TC>(o_im);
    }
  }
}

// The same for bfloat16 activations and head sizes 16, 32, 64, 128, 256: hd/8 lanes per
// head, eight consecutive elements per lane in one 16-byte load, the rotation partner
// (the element hd/2 further) fetched from the lane hd/16 further.  `with_v` = 0 leaves the
// value heads to the workgroups that store them tile by tile (v_store_tile).
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_qk;
typedef __attribute__((ext_vector_type(4))) float f32x4_qk;

// Values of many tokens into their pages (bfloat16 to bfloat16).  A page holds values
// transposed, [head element][position], so a token's head vector lands two bytes at a
// time, hd rows apart: here 16 lanes take 16 consecutive tokens for the same 8 head
// elements, and since consecutive tokens of a prompt sit at consecutive positions, the 16
// two-byte stores of one row fall into one 32-byte run of the page.  A workgroup of 256
// takes (tile of 16 tokens, key/value head); its 16 lane groups take 8 head elements
// each, in rounds.
__device__ __forceinline__ void v_store_tile(const QkPrepareArgs& a, int tile, int kvh) {
  const int j = threadIdx.x % 16;
  const int t = tile * 16 + j;
  if (t >= a.num_tokens) return;
  const int pos = a.positions[t];
  const int page = a.table[(int64_t)a.entry_of_token[t] * a.table_width + pos / a.page_size];
  if (page < 0) return;
  const int hd = a.hd;
  const bf16_t* src = (const bf16_t*)a.qkv + (int64_t)t * (a.nq + 2 * a.nkv) * hd +
                      (int64_t)(a.nq + a.nkv + kvh) * hd;
  bf16_t* dst = (bf16_t*)a.v_dst + ((int64_t)page * a.nkv + kvh) * a.page_size * hd +
                pos % a.page_size;
  for (int d0 = (threadIdx.x / 16) * 8; d0 < hd; d0 += 128) {
    const bf16x8_qk x = *(const bf16x8_qk*)(src + d0);
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[(int64_t)(d0 + i) * a.page_size] = x[i];
  }
}

// A thread goes through its piece (N of them: one was measured best, more waves do
// better than longer ones) in three rounds: everything that hangs on nothing (the
// elements, the position, the norm weight, the entry), then what hangs on the position
// (cos and sin, the page), then the arithmetic and the stores.  A piece so costs two
// trips to memory, not one per use.
template <typename TC, int N>
__global__ __launch_bounds__(256) void qk_prepare_vec_kernel(QkPrepareArgs a, int lanes_log2,
                                                             int with_v, int v_first_block) {
  // with_v = 0 and v_first_block >= 0: the workgroups from that one on store the values
  // tile by tile (one launch for both: a second launch costs more than its work here)
  if (v_first_block >= 0 && (int)blockIdx.x >= v_first_block) {
    const int idx = blockIdx.x - v_first_block;
    v_store_tile(a, idx / a.nkv, idx % a.nkv);
    return;
  }
  const int L = 1 << lanes_log2;                     // lanes per head
  const int heads_per_wave = kWave >> lanes_log2;
  const int lane = threadIdx.x % kWave;
  const int sub = lane & (L - 1);                    // my 8 elements: [8*sub, 8*sub + 8)
  const int heads = a.nq + (a.store_kv ? (with_v ? 2 : 1) * a.nkv : 0);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int hd = a.hd, half = hd / 2;
  const f32x4_qk zero4 = {0.f, 0.f, 0.f, 0.f};
  const int i0 = (sub & (L / 2 - 1)) * 8;            // index into the half-size table
  struct Piece {
    bool live, norm, rotate, to_page;
    int t, h, kind, pos, entry, page;
    bf16x8_qk x;
    f32x4_qk w0, w1, c0, c1, s0, s1;
  };
  Piece pc[N];
#pragma unroll
  for (int i = 0; i < N; ++i) {
    Piece& p = pc[i];
    const int64_t item = (wave * N + i) * heads_per_wave + (lane >> lanes_log2);
    p.live = item < (int64_t)a.num_tokens * heads;
    const int64_t it = p.live ? item : 0;
    p.t = (int)(it / heads), p.h = (int)(it % heads);
    p.kind = p.h < a.nq ? 0 : (p.h < a.nq + a.nkv ? 1 : 2);
    const bf16_t* src = (const bf16_t*)a.qkv + (int64_t)p.t * (a.nq + 2 * a.nkv) * hd + (int64_t)p.h * hd;
    p.x = *(const bf16x8_qk*)(src + sub * 8);
    p.pos = a.positions[p.t];
    const float* w = p.kind == 0 ? a.q_weight : a.k_weight;
    p.norm = p.kind != 2 && w, p.rotate = p.kind != 2 && a.cos;
    p.to_page = p.kind != 0 && a.paged;
    p.w0 = p.w1 = zero4;
    if (p.norm) {
      p.w0 = *(const f32x4_qk*)(w + sub * 8);
      p.w1 = *(const f32x4_qk*)(w + sub * 8 + 4);
    }
    p.entry = p.to_page ? a.entry_of_token[p.t] : 0;
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    Piece& p = pc[i];
    p.c0 = p.c1 = p.s0 = p.s1 = zero4;
    if (p.rotate) {
      const float* cp = a.cos + (int64_t)p.pos * half + i0;
      const float* sp = a.sin + (int64_t)p.pos * half + i0;
      p.c0 = *(const f32x4_qk*)cp; p.c1 = *(const f32x4_qk*)(cp + 4);
      p.s0 = *(const f32x4_qk*)sp; p.s1 = *(const f32x4_qk*)(sp + 4);
    }
    p.page = p.to_page ? a.table[(int64_t)p.entry * a.table_width + p.pos / a.page_size] : -1;
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const Piece& p = pc[i];
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (float)p.x[j];
    if (p.norm) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
      for (int o = 1; o < L; o <<= 1) ss += __shfl_xor(ss, o, kWave);
      const float rstd = rsqrtf(ss / (float)hd + a.eps);
#pragma unroll
      for (int j = 0; j < 4; ++j) { v[j] *= rstd * p.w0[j]; v[4 + j] *= rstd * p.w1[j]; }
    }
    if (p.rotate) {
      const bool first = sub < L / 2;                  // holds elements i < hd/2
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float other = __shfl_xor(v[j], L / 2, kWave);
        const float c = j < 4 ? p.c0[j] : p.c1[j - 4], sn = j < 4 ? p.s0[j] : p.s1[j - 4];
        // first half: re*c - im*s with im = other; second half: im*c + re*s with re = other
        v[j] = first ? v[j] * c - other * sn : v[j] * c + other * sn;
      }
    }
    if (!p.live) continue;
    const int t = p.t, h = p.h;
    if (p.kind == 0) {
      bf16x8_qk o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (bf16_t)v[j];
      *(bf16x8_qk*)((bf16_t*)a.q_out + ((int64_t)t * a.nq + h) * hd + sub * 8) = o;
      continue;
    }
    const int kvh = p.kind == 1 ? h - a.nq : h - a.nq - a.nkv;
    if (!a.paged) {
      TC* dst = (TC*)(p.kind == 1 ? a.k_dst : a.v_dst) + ((int64_t)t * a.nkv + kvh) * hd + sub * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[j] = from_f32<TC>(v[j]);
      continue;
    }
    if (p.page < 0) continue;
    const int64_t head_base = ((int64_t)p.page * a.nkv + kvh) * a.page_size * hd;
    const int slot = p.pos % a.page_size;
    if (p.kind == 1) {
      TC* dst = (TC*)a.k_dst + head_base + (int64_t)slot * hd + sub * 8;
      if constexpr (sizeof(TC) == 2) {     // one 16-byte store (pages and rows are 16-byte aligned)
        bf16x8_qk o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (bf16_t)v[j];
        *(bf16x8_qk*)dst = o;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = from_f32<TC>(v[j]);
      }
    } else {
      TC* dst = (TC*)a.v_dst + head_base + slot;
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[(int64_t)(sub * 8 + j) * a.page_size] = from_f32<TC>(v[j]);
    }
  }
}

extern "C" int ts_qk_prepare(const QkPrepareArgs* args, int act_type, int cache_type,
                             hipStream_t stream) {
  QkPrepareArgs a = *args;
  if (a.num_tokens <= 0) return 0;
  if (a.hd <= 0 || a.hd % 2) TS_FAIL("qk_prepare: head_dim=%d must be even", a.hd);
  if (a.nq <= 0 || a.nkv < 0) TS_FAIL("qk_prepare: heads nq=%d nkv=%d", a.nq, a.nkv);
  if ((a.cos == nullptr) != (a.sin == nullptr)) TS_FAIL("qk_prepare: cos and sin go together");
  if (a.store_kv && (a.nkv == 0 || !a.k_dst || !a.v_dst))
    TS_FAIL("qk_prepare: store_kv without key/value heads or destination");
  if (a.store_kv && a.paged && (a.page_size <= 0 || !a.table || a.table_width <= 0))
    TS_FAIL("qk_prepare: paged store needs page_size and a block table");
  const int heads = a.nq + (a.store_kv ? 2 * a.nkv : 0);
  const int64_t items = (int64_t)a.num_tokens * heads;
  const int waves_per_block = 4;
  if (act_type == TS_BF16 && a.hd >= 16 && a.hd <= 256 && (a.hd & (a.hd - 1)) == 0 &&
      ((uintptr_t)a.qkv & 15) == 0 && ((uintptr_t)a.q_out & 15) == 0) {
    // portions of prompts: the values go tile by tile, by further workgroups of the same
    // launch
    const bool v_tiles = a.store_kv && a.paged && cache_type == TS_BF16 && a.num_tokens >= 64;
    const int lanes_log2 = __builtin_ctz(a.hd / 8);
    const int heads_per_block = waves_per_block * (kWave >> lanes_log2);
    const int64_t vec_items = v_tiles ? (int64_t)a.num_tokens * (a.nq + a.nkv) : items;
    const int64_t vblocks = (vec_items + heads_per_block - 1) / heads_per_block;
    const int64_t tiles = v_tiles ? (int64_t)((a.num_tokens + 15) / 16) * a.nkv : 0;
    if (vblocks + tiles > 2147483647LL) TS_FAIL("qk_prepare: too many tokens");
    TS_DISPATCH_TYPE(cache_type, TC,
        hipLaunchKernelGGL((qk_prepare_vec_kernel<TC, 1>), dim3((unsigned)(vblocks + tiles)),
                           dim3(waves_per_block * kWave), 0, stream, a, lanes_log2,
                           v_tiles ? 0 : 1, v_tiles ? (int)vblocks : -1));
    TS_CHECK_LAUNCH("qk_prepare");
    return 0;
  }
  const int64_t blocks = (items + waves_per_block - 1) / waves_per_block;
  if (blocks > 2147483647LL) TS_FAIL("qk_prepare: too many tokens");
  TS_DISPATCH_TYPE(act_type, T, TS_DISPATCH_TYPE(cache_type, TC,
      hipLaunchKernelGGL((qk_prepare_kernel<T, TC>), dim3((unsigned)blocks),
                         dim3(waves_per_block * kWave), 0, stream, a)));
  TS_CHECK_LAUNCH("qk_prepare");
  return 0;
}

// ---------------------------------------------------------------- rotation alone
template <typename T>
__global__ void rope_kernel(T* __restrict__ x, const int* __restrict__ positions,
                            const float* __restrict__ cos, const float* __restrict__ sin,
                            int64_t items, int heads, int hd) {
  const int lane = threadIdx.x % kWave;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= items) return;
  const int half = hd / 2;
  const int pos = positions[item / heads];
  T* row = x + item * hd;
  for (int i = lane; i < half; i += kWave) {
    const float re = to_f32(row[i]), im = to_f32(row[i + half]);
    const float c = cos[(int64_t)pos * half + i], s = sin[(int64_t)pos * half + i];
    row[i] = from_f32<T>(re * c - im * s);
    row[i + half] = from_f32<T>(im * c + re * s);
  }
}

extern "C" int ts_rope_inplace(void* x, int type, const int* positions, const float* cos,
                               const float* sin, int num_tokens, int heads, int hd,
                               hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (hd <= 0 || hd % 2) TS_FAIL("rope: head_dim=%d must be even", hd);
  const int64_t items = (int64_t)num_tokens * heads;
  const int64_t blocks = (items + 3) / 4;
  TS_DISPATCH_TYPE(type, T,
                   hipLaunchKernelGGL(rope_kernel<T>, dim3((unsigned)blocks), dim3(256), 0,
                                      stream, (T*)x, positions, cos, sin, items, heads, hd));
  TS_CHECK_LAUNCH("rope");
  return 0;
}

// ---------------------------------------------------------------- store alone
template <typename T, typename TC>
__global__ void kv_store_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                TC* __restrict__ k_pages, TC* __restrict__ v_pages,
                                const int* __restrict__ positions,
                                const int* __restrict__ entry_of_token,
                                const int* __restrict__ table, int table_width, int64_t items,
                                int nkv, int hd, int page_size) {
  const int lane = threadIdx.x % kWave;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= items) return;
  const int t = (int)(item / nkv), kvh = (int)(item % nkv);
  const int pos = positions[t];
  const int page = table[(int64_t)entry_of_token[t] * table_width + pos / page_size];
  if (page < 0) return;
  const int64_t head = ((int64_t)page * nkv + kvh) * page_size * hd;
  const int slot = pos % page_size;
  for (int i = lane; i < hd; i += kWave) {
    k_pages[head + (int64_t)slot * hd + i] = from_f32<TC>(to_f32(k[item * hd + i]));
    v_pages[head + (int64_t)i * page_size + slot] = from_f32<TC>(to_f32(v[item * hd + i]));
  }
}

extern "C" int ts_kv_store(const void* k, const void* v, int act_type, void* k_pages,
                           void* v_pages, int cache_type, const int* positions,
                           const int* entry_of_token, const int* table, int table_width,
                           int num_tokens, int nkv, int hd, int page_size, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (page_size <= 0 || table_width <= 0) TS_FAIL("kv_store: page_size/table_width");
  const int64_t items = (int64_t)num_tokens * nkv;
  const int64_t blocks = (items + 3) / 4;
  TS_DISPATCH_TYPE(act_type, T, TS_DISPATCH_TYPE(cache_type, TC,
      hipLaunchKernelGGL((kv_store_kernel<T, TC>), dim3((unsigned)blocks), dim3(256), 0, stream,
                         (const T*)k, (const T*)v, (TC*)k_pages, (TC*)v_pages, positions,
                         entry_of_token, table, table_width, items, nkv, hd, page_size)));
  TS_CHECK_LAUNCH("kv_store");
  return 0;
}
