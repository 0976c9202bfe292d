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
  const float* sink;      // [nq] or null: a score per query head that joins the softmax's
                          // denominator once, with no key and no value (not scaled)
};

// The sum of a row's softmax weights with the head's sink in it.  `m_log2` is the row's
// largest score in units of log2 (scores times scale times log2(e)), which the weights in
// `sum` are relative to.  A sink far above every score is cut off where the output has
// long become zero, so nothing overflows.
__device__ __forceinline__ float sum_with_sink(float sum, float m_log2, const float* sink,
                                               int head) {
  if (!sink) return sum;
  return sum + __builtin_amdgcn_exp2f(fminf(sink[head] * 1.44269504088896f - m_log2, 100.f));
}
