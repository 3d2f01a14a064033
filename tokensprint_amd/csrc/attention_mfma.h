// Declarations shared by the matrix-core attention kernels.
#pragma once
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
  int tiles_per_wave;    // prompt kernel: 16-row tiles a wavefront works on (1, 2 or 4)
};

