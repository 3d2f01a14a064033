// Paged causal attention for any head size up to 256, any page size, any head grouping,
// float32 or bfloat16 storage, float32 arithmetic throughout: the attention of the
// float32 path and of shapes the matrix-core kernels do not take.
//
// One workgroup of four wavefronts per (query token, query head).  Keys are cut into tiles
// of 64 starting at the first visible key; wavefront w walks tiles w, w + 4, ... and the
// four partial results are merged in wavefront order, so the partition, and with it the
// rounding, depends only on the token's position and the window, never on how the step was
// cut or batched.  (A decode step of few requests has few such pairs: with a wavefront
// each, 32 of 256 compute units worked.)
#include "attention.h"

constexpr int kMaxHeadDim = 256;
constexpr int kWavesPerBlock = 4;

// Four consecutive elements in one load; they are used one after the other, in index
// order, so the sums are those of a loop over single elements.
typedef __attribute__((ext_vector_type(4))) float f32x4_g;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_g;
__device__ __forceinline__ f32x4_g load4_g(const float* p) { return *(const f32x4_g*)p; }
__device__ __forceinline__ f32x4_g load4_g(const bf16_t* p) {
  const bf16x4_g v = *(const bf16x4_g*)p;
  return f32x4_g{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

template <typename T, typename TC>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void attention_generic_kernel(AttentionArgs a) {
  __shared__ float q_s[kWavesPerBlock][kMaxHeadDim];
  __shared__ float p_s[kWavesPerBlock][kWave];
  __shared__ int64_t row_s[kWavesPerBlock][kWave];
  __shared__ float m_s[kWavesPerBlock], l_s[kWavesPerBlock];
  __shared__ float acc_s[kWavesPerBlock][kMaxHeadDim];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t item = blockIdx.x;
  const int t = (int)(item / a.nq), h = (int)(item % a.nq);
  const int kvh = h / (a.nq / a.nkv);
  const int hd = a.hd, P = a.page_size;
  const int pos = a.positions[t];
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int* table = a.table + (int64_t)a.entry_of_token[t] * a.table_width;
  const T* q = (const T*)a.q + item * hd;
  const TC* kp = (const TC*)a.k_pages;
  const TC* vp = (const TC*)a.v_pages;

  // head and page sizes in fours (and a cache that starts on 16 bytes): loads of four
  const bool by4 = hd % 4 == 0 && P % 4 == 0 && (((uintptr_t)kp | (uintptr_t)vp) & 15) == 0;
  for (int d = lane; d < hd; d += kWave) q_s[wave][d] = to_f32(q[d]);
  // a wavefront runs in lockstep and only reads its own rows of LDS: no barrier needed,
  // but the compiler must not reorder the LDS traffic
  __builtin_amdgcn_wave_barrier();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxHeadDim / kWave] = {};
  for (int j0 = lo + wave * kWave; j0 <= pos; j0 += kWavesPerBlock * kWave) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    int64_t row = -1;
    if (valid) {
      const int page = table[j / P];
      if (page >= 0) {
        row = ((int64_t)page * a.nkv + kvh) * P * hd + j % P;   // of the value column
        const TC* kr = kp + ((int64_t)page * a.nkv + kvh) * P * hd + (int64_t)(j % P) * hd;
        float dot = 0.f;
        if (by4) {
          for (int d = 0; d < hd; d += 4) {
            const f32x4_g k4 = load4_g(kr + d);
#pragma unroll
            for (int e = 0; e < 4; ++e) dot = fmaf(q_s[wave][d + e], k4[e], dot);
          }
        } else {
          for (int d = 0; d < hd; ++d) dot = fmaf(q_s[wave][d], to_f32(kr[d]), dot);
        }
        s = dot * a.scale;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    // m_new stays -inf only while no key has been seen (pages given back): keep zeros
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);   // exp(-inf) = 0 at first
    const float p = (row >= 0 && m_new != -INFINITY) ? expf(s - m_new) : 0.f;
    l = l * corr + wave_sum(p);
    p_s[wave][lane] = p;
    row_s[wave][lane] = row;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < kMaxHeadDim / kWave; ++r) acc[r] *= corr;
    const int n = min(kWave, pos - j0 + 1);
    if (by4) {
      // four keys at a time where the group starts at a multiple of four (it then lies in
      // one page, side by side in each value row), key by key elsewhere (a tile starts at
      // the first visible key, which a window puts anywhere); in key order either way
      for (int jj = 0; jj < n; jj += 4) {
        const int64_t vrow = row_s[wave][jj];
        const bool whole = jj + 3 < n && vrow >= 0 && ((j0 + jj) & 3) == 0;
        if (whole) {
#pragma unroll
          for (int r = 0; r < kMaxHeadDim / kWave; ++r) {
            const int d = lane + r * kWave;
            if (d < hd) {
              const f32x4_g v4 = load4_g(vp + vrow + (int64_t)d * P);
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[r] = fmaf(p_s[wave][jj + e], v4[e], acc[r]);
            }
          }
        } else {
          for (int e = 0; e < 4 && jj + e < n; ++e) {
            const int64_t vr = row_s[wave][jj + e];
            if (vr < 0) continue;
            const float pj = p_s[wave][jj + e];
#pragma unroll
            for (int r = 0; r < kMaxHeadDim / kWave; ++r) {
              const int d = lane + r * kWave;
              if (d < hd) acc[r] = fmaf(pj, to_f32(vp[vr + (int64_t)d * P]), acc[r]);
            }
          }
        }
      }
    } else {
      for (int jj = 0; jj < n; ++jj) {
        const int64_t vrow = row_s[wave][jj];
        if (vrow < 0) continue;
        const float pj = p_s[wave][jj];
#pragma unroll
        for (int r = 0; r < kMaxHeadDim / kWave; ++r) {
          const int d = lane + r * kWave;
          if (d < hd) acc[r] = fmaf(pj, to_f32(vp[vrow + (int64_t)d * P]), acc[r]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
    m = m_new;
  }
  // the wavefronts' partial results, merged by the first in wavefront order
  if (lane == 0) { m_s[wave] = m; l_s[wave] = l; }
#pragma unroll
  for (int r = 0; r < kMaxHeadDim / kWave; ++r) {
    const int d = lane + r * kWave;
    if (d < hd) acc_s[wave][d] = acc[r];
  }
  __syncthreads();
  if (wave != 0) return;
  float m_all = -INFINITY;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) m_all = fmaxf(m_all, m_s[w]);
  float weight[kWavesPerBlock];
  l = 0.f;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    weight[w] = m_s[w] == -INFINITY ? 0.f : expf(m_s[w] - m_all);     // a wavefront without keys
    l += l_s[w] * weight[w];
  }
  T* o = (T*)a.out + item * hd;
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int r = 0; r < kMaxHeadDim / kWave; ++r) {
    const int d = lane + r * kWave;
    if (d >= hd) continue;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) sum += weight[w] == 0.f ? 0.f : acc_s[w][d] * weight[w];
    o[d] = from_f32<T>(sum * inv);
  }
}

int ts_check_attention_args(const AttentionArgs& a, const char* who) {
  if (a.hd <= 0 || a.hd > kMaxHeadDim) TS_FAIL("%s: head_dim=%d not in 1..%d", who, a.hd, kMaxHeadDim);
  if (a.nq <= 0 || a.nkv <= 0 || a.nq % a.nkv)
    TS_FAIL("%s: %d query heads cannot share %d key/value heads", who, a.nq, a.nkv);
  if (a.page_size <= 0 || a.table_width <= 0 || a.num_pages <= 0)
    TS_FAIL("%s: page_size=%d table_width=%d num_pages=%d", who, a.page_size, a.table_width,
            a.num_pages);
  if (a.window < 0) TS_FAIL("%s: window=%d", who, a.window);
  return 0;
}

extern "C" int ts_attention_generic(const AttentionArgs* args, int act_type, int cache_type,
                                    hipStream_t stream) {
  AttentionArgs a = *args;
  if (a.num_tokens <= 0) return 0;
  if (ts_check_attention_args(a, "attention_generic")) return -1;
  const int64_t blocks = (int64_t)a.num_tokens * a.nq;       // a workgroup per token and head
  if (blocks > 2147483647LL) TS_FAIL("attention_generic: too many tokens");
  TS_DISPATCH_TYPE(act_type, T, TS_DISPATCH_TYPE(cache_type, TC,
      hipLaunchKernelGGL((attention_generic_kernel<T, TC>), dim3((unsigned)blocks),
                         dim3(kWavesPerBlock * kWave), 0, stream, a)));
  TS_CHECK_LAUNCH("attention_generic");
  return 0;
}
