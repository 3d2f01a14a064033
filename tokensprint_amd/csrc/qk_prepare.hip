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
