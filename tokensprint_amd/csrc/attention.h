// Arguments shared by the paged-attention kernels.
#pragma once
#include "common.h"

struct AttentionArgs {
  const void* q;          // [T, nq, hd]
  void* out;              // [T, nq, hd]
  const void* k_pages;    // [num_pages, nkv, P, hd]
  const void* v_pages;    // [num_pages, nkv, hd, P]: values transposed inside a page
  const int* positions;       // [T]   absolute position of each query token
  const int* entry_of_token;  // [T]   batch entry (row of the block table) of each token
  const int* q_start;         // [B+1] first flat token of each entry
  const int* ctx_len;         // [B]   keys of the entry after this step
  const int* table;           // [B, table_width] logical page -> physical page, -1 none
  int table_width;
  int num_tokens, num_entries, nq, nkv, hd, page_size, num_pages;
  int window;             // 0: every earlier key; W: keys p-W+1..p
  float scale;
};
