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
  int chunk;              // 0: none; C: only keys of the query's own stretch of C positions
                          // (floor(key / C) = floor(position / C))
  float softcap;          // 0: none; c: score <- c tanh(score / c), after the scale
  const float* slopes;    // [nq] or null: slope * (position - key) is taken off a score
  float temp_coef;        // the query at position p is multiplied by
  int temp_every;         // 1 + temp_coef ln(floor((p + 1) / temp_every) + 1); 0: by one
};

// The first key the query at `pos` sees.
__device__ __forceinline__ int first_visible(const AttentionArgs& a, int pos) {
  int lo = (a.window > 0) ? max(0, pos - a.window + 1) : 0;
  if (a.chunk > 0) lo = max(lo, max(pos, 0) / a.chunk * a.chunk);
  return lo;
}

// Whether scores are more than scale times the product: a cap, a distance bias or a
// query temperature (the kernels that know these are built apart from those that do not).
__host__ __device__ __forceinline__ bool has_score_extras(const AttentionArgs& a) {
  return a.softcap > 0.f || a.slopes != nullptr || a.temp_every > 0;
}

// What turns a query row's products into scores, when there are such extras.
struct ScoreExtra {
  int pos;                // the query's position (distances are counted from it)
  float row_scale;        // scale times the query's temperature
  float cap, inv_cap;     // cap 0: none
  float slope;            // of the row's head; 0: none
};

__device__ __forceinline__ ScoreExtra score_extra(const AttentionArgs& a, int head, int pos) {
  ScoreExtra x;
  x.pos = pos;
  float temp = 1.f;
  if (a.temp_every > 0)
    temp = 1.f + a.temp_coef * logf((float)((max(pos, 0) + 1) / a.temp_every + 1));
  x.row_scale = a.scale * temp;
  x.cap = a.softcap;
  x.inv_cap = a.softcap > 0.f ? 1.f / a.softcap : 0.f;
  x.slope = (a.slopes && pos >= 0) ? a.slopes[head] : 0.f;
  return x;
}

// A score from the product q . k for the key at position `key`.  FAST: the hyperbolic
// tangent as 1 - 2 / (exp(2 z) + 1) by the hardware's exponential and reciprocal (for
// kernels whose operands are bfloat16; the float32 kernel takes the library's).
template <bool FAST = false>
__device__ __forceinline__ float extra_score(const ScoreExtra& x, float dot, int key) {
  float s = dot * x.row_scale;
  if (x.cap > 0.f) {
    const float z = s * x.inv_cap;
    const float th = FAST ? 1.f - 2.f * __builtin_amdgcn_rcpf(
                                      __builtin_amdgcn_exp2f(fminf(z * 2.88539008177792681f, 126.f)) + 1.f)
                          : tanhf(z);
    s = x.cap * th;
  }
  return s - x.slope * (float)(x.pos - key);
}

// The sum of a row's softmax weights with the head's sink in it.  `m_log2` is the row's
// largest score in units of log2 (scores times scale times log2(e)), which the weights in
// `sum` are relative to.  A sink far above every score is cut off where the output has
// long become zero, so nothing overflows.
__device__ __forceinline__ float sum_with_sink(float sum, float m_log2, const float* sink,
                                               int head) {
  if (!sink) return sum;
  return sum + __builtin_amdgcn_exp2f(fminf(sink[head] * 1.44269504088896f - m_log2, 100.f));
}
