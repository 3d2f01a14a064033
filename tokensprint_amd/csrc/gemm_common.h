// What the matrix-core product kernels share: vector types, the K step of a wave, the
// store of four results, and the one rule that lays the waves of a workgroup out.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

constexpr int kIterK = 128;   // K elements a wave consumes per iteration (4 MFMA steps)

template <typename TC> __device__ __forceinline__ void store4(TC* p, f32x4 v, int n_left);
template <> __device__ __forceinline__ void store4<float>(float* p, f32x4 v, int n_left) {
  if (n_left >= 4 && ((uintptr_t)p & 15) == 0) { *(f32x4*)p = v; return; }
  for (int t = 0; t < 4 && t < n_left; ++t) p[t] = v[t];
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4 v, int n_left) {
  if (n_left >= 4 && ((uintptr_t)p & 7) == 0) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
    return;
  }
  for (int t = 0; t < 4 && t < n_left; ++t) p[t] = (bf16_t)v[t];
}

// How the waves of a workgroup are laid out: from N and K only, never from M, and the
// same for every kernel, so that a row of C is computed in the same order whatever else
// is in the batch and whichever kernel serves it.
//   wide (a short K): 4 waves along N; deep (a long K and too few rows of W to fill the chip with
//   workgroups of 4): 8 waves split K; otherwise 4 waves split K.
static inline bool layout_wide(int N, int K) { return K < 512; }
static inline bool layout_deep(int N, int K) { return K >= 2048 && N < 4096; }

// Operands of the product whose workgroups own 16 rows of W and split K among their
// waves (every layout but the wide one).
struct DirectArgs {
  const bf16_t* A;          // [M, K], or null in the fused form
  const bf16_t* W;          // [N, K] (pair: [2, N, K])
  void* C;                  // [M, N]
  const float* resid_in;    // fused form: [M, K]
  const bf16_t* delta;      // fused form: [M, K] or null
  const float* norm_w;      // fused form: [K]
  float* resid_out;         // fused form: [M, K], written by workgroup column 0
  int M, N, K;
  float eps;
  // tail form (resid set): nothing goes to C; the product, rounded to bfloat16, is added
  // to the residual stream in place, and the new stream is handed on prepared for the
  // RMSNorm that follows: rows x * tail_w, and per row the sum of x^2 over this
  // workgroup's 16 columns
  float* resid;             // [M, N]
  const float* tail_w;      // [N]
  bf16_t* prepared;         // [M, N] out
  float* sumsq_out;         // [M][gemm_direct_tail_parts(M, N) rounded up to 4] out
  // scaled form (sumsq set): A holds such prepared rows; C's rows are divided by the
  // root mean square that the slices of sums of squares give
  const float* sumsq;       // [M][parts rounded up to 4]
  int parts;
  // merged form (merge_o set; tail form, at most 16 rows): A is not stored either but is a
  // decode step's attention output still lying in the partial sums of its key splits, as
  // the attention kernels leave them for attention_merge; K = heads * merge_hd
  const float* merge_o;     // [items, merge_splits, 16, merge_hd]
  const float* merge_ml;    // [items, merge_splits, 16, 2]: row maximum (log2 units), sum
  const int* merge_pos;     // [M]: position of each row's token
  int merge_splits, merge_nkv, merge_group, merge_hd, merge_window, merge_chunk;
};

// Launches it; `norm` (the fused form) takes at most 16 rows.  Returns 0 or -1 with the
// error text set.
int gemm_direct_launch(const DirectArgs& a, int c_type, bool pair, bool norm, hipStream_t stream);
// Whether the tail and the scaled form take a product of this shape (up to 64 rows).
bool gemm_direct_tail_fits(int M, int N, int K);
int gemm_direct_tail_parts(int M, int N);      // slices the tail form leaves per row
bool gemm_direct_scaled_fits(int M, int N, int K, bool pair, int parts);
