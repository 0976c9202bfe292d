// Kernels of a selective state-space mixer with one scalar decay per head and token:
// the short causal convolution with SiLU, the recurrence itself, and the gated group norm
// behind it.  All arithmetic in float32; the recurrence's state and the convolution's last
// inputs live in float32 per-request slots and are carried from step to step.
//
// A request's state is read only where a portion does not start at position 0, and is
// written once a portion, by the thread that owns the element.
#include "common.h"

struct BatchView {
  const int* positions;       // [T]
  const int* entry_of_token;  // [T]
  const int* q_start;         // [B + 1]
  const int* slot_ids;        // [B]
};

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// ---------------------------------------------------------------- convolution
// u = rows of `proj` (leading dimension ld) from column `col`, `channels` wide.
// (bias may be null: none.)
// out_t[c] = silu(bias[c] + sum_k w[c][k] * u_(t - (taps-1) + k)[c]); inputs in front of
// the sequence are zero, inputs in front of the portion come from state[slot][taps-1][C],
// whose row j holds the input at position start - (taps-1) + j.

// `in_bias` (may be null): added to every input of the sequence before the convolution (the
// zeros in front of the sequence stay zeros; the state holds inputs with it added).
// `plain` 1: no activation behind the convolution.

// One thread per (token, channel); writes no state.
__global__ __launch_bounds__(256) void conv_silu_kernel(
    const float* __restrict__ proj, int ld, int col, int channels, int taps,
    const float* __restrict__ w, const float* __restrict__ bias, const float* __restrict__ state,
    float* __restrict__ out, BatchView b, int num_tokens, const float* __restrict__ in_bias,
    int plain) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_tokens * channels) return;
  const int t = (int)(idx / channels), c = (int)(idx % channels);
  const int e = b.entry_of_token[t];
  const int first = b.q_start[e], pos = b.positions[t];
  const float* st = state + (int64_t)b.slot_ids[e] * (taps - 1) * channels;
  float acc = bias ? bias[c] : 0.f;
  const float ib = in_bias ? in_bias[c] : 0.f;
  for (int k = 0; k < taps; ++k) {
    const int back = taps - 1 - k;
    if (pos - back < 0) continue;
    float v;
    if (t - back >= first) v = proj[(int64_t)(t - back) * ld + col + c] + ib;
    else v = st[(int64_t)(taps - 1 - (first - (t - back))) * channels + c];
    acc = fmaf(w[c * taps + k], v, acc);
  }
  out[(int64_t)t * channels + c] = plain ? acc : silu_f(acc);
}

// The same for long steps: a thread takes kConvRun consecutive tokens of one channel, so an
// input is read once for all the taps that meet it (kept in registers) instead of once a
// tap.  An output's sum runs over the taps in the same order as in the kernel above.
constexpr int kConvRun = 8, kConvMaxTaps = 8;
__global__ __launch_bounds__(256) void conv_silu_run_kernel(
    const float* __restrict__ proj, int ld, int col, int channels, int taps,
    const float* __restrict__ w, const float* __restrict__ bias, const float* __restrict__ state,
    float* __restrict__ out, BatchView b, int num_tokens, const float* __restrict__ in_bias,
    int plain) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int t0 = blockIdx.y * kConvRun;
  const float ib = in_bias ? in_bias[c] : 0.f, bc = bias ? bias[c] : 0.f;
  float wk[kConvMaxTaps], raw[kConvRun + kConvMaxTaps - 1];
#pragma unroll
  for (int k = 0; k < kConvMaxTaps; ++k) wk[k] = k < taps ? w[c * taps + k] : 0.f;
  // raw[j]: the input of flat row t0 - (taps - 1) + j (whatever entry it belongs to)
#pragma unroll
  for (int j = 0; j < kConvRun + kConvMaxTaps - 1; ++j) {
    const int row = t0 - (taps - 1) + j;
    raw[j] = (j < kConvRun + taps - 1 && row >= 0 && row < num_tokens)
                 ? proj[(int64_t)row * ld + col + c] + ib : 0.f;
  }
#pragma unroll
  for (int i = 0; i < kConvRun; ++i) {
    const int t = t0 + i;
    if (t >= num_tokens) break;
    const int e = b.entry_of_token[t];
    const int first = b.q_start[e], pos = b.positions[t];
    const float* st = state + (int64_t)b.slot_ids[e] * (taps - 1) * channels;
    float acc = bc;
#pragma unroll
    for (int k = 0; k < kConvMaxTaps; ++k) {
      if (k >= taps) break;
      const int back = taps - 1 - k;
      if (pos - back < 0) continue;
      float v;
      if (t - back >= first) v = raw[i + k];
      else v = st[(int64_t)(taps - 1 - (first - (t - back))) * channels + c];
      acc = fmaf(wk[k], v, acc);
    }
    out[(int64_t)t * channels + c] = plain ? acc : silu_f(acc);
  }
}

// One thread per (entry, channel): the state after the portion.  Row j takes the input at
// position end - (taps-1) + j: from the portion, from the old state further up (read before
// any row at or above it is written: j ascends), or zero in front of the sequence.
__global__ __launch_bounds__(256) void conv_state_kernel(
    const float* __restrict__ proj, int ld, int col, int channels, int taps,
    float* __restrict__ state, BatchView b, int num_entries, const float* __restrict__ in_bias) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_entries * channels) return;
  const int e = (int)(idx / channels), c = (int)(idx % channels);
  const int first = b.q_start[e], n = b.q_start[e + 1] - first;
  const int start = b.positions[first];
  float* st = state + (int64_t)b.slot_ids[e] * (taps - 1) * channels;
  for (int j = 0; j < taps - 1; ++j) {
    const int p = start + n - (taps - 1) + j;
    float v = 0.f;
    if (p >= start) v = proj[(int64_t)(first + p - start) * ld + col + c] + (in_bias ? in_bias[c] : 0.f);
    else if (p >= 0) v = st[(int64_t)(j + n) * channels + c];
    st[(int64_t)j * channels + c] = v;
  }
}

// One thread per (entry, channel) walks the entry's tokens with the last inputs in
// registers and leaves the state: one kernel for steps of few tokens per entry.
constexpr int kMaxTapsInRegisters = 8;
__global__ __launch_bounds__(256) void conv_silu_walk_kernel(
    const float* __restrict__ proj, int ld, int col, int channels, int taps,
    const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ state,
    float* __restrict__ out, BatchView b, int num_entries, const float* __restrict__ in_bias,
    int plain) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_entries * channels) return;
  const int e = (int)(idx / channels), c = (int)(idx % channels);
  const int first = b.q_start[e], end = b.q_start[e + 1];
  const float ib = in_bias ? in_bias[c] : 0.f;
  const int start = b.positions[first];
  float* st = state + (int64_t)b.slot_ids[e] * (taps - 1) * channels;
  float hist[kMaxTapsInRegisters], wk[kMaxTapsInRegisters];
#pragma unroll
  for (int j = 0; j < kMaxTapsInRegisters; ++j) {
    hist[j] = 0.f;
    wk[j] = j < taps ? w[c * taps + j] : 0.f;
    // hist[j], j < taps-1: the input at position start - (taps-1) + j
    if (j < taps - 1 && start - (taps - 1) + j >= 0) hist[j] = st[(int64_t)j * channels + c];
  }
  const float bc = bias ? bias[c] : 0.f;
  for (int t = first; t < end; ++t) {
    const float v = proj[(int64_t)t * ld + col + c] + ib;
    float acc = bc;
#pragma unroll
    for (int k = 0; k < kMaxTapsInRegisters; ++k) {
      if (k < taps - 1) acc = fmaf(wk[k], hist[k], acc);
      else if (k == taps - 1) acc = fmaf(wk[k], v, acc);
    }
    out[(int64_t)t * channels + c] = plain ? acc : silu_f(acc);
#pragma unroll
    for (int k = 0; k < kMaxTapsInRegisters - 1; ++k) {
      if (k < taps - 2) hist[k] = hist[k + 1];
      else if (k == taps - 2) hist[k] = v;
    }
  }
#pragma unroll
  for (int j = 0; j < kMaxTapsInRegisters; ++j)
    if (j < taps - 1) st[(int64_t)j * channels + c] = hist[j];
}

extern "C" int ts_conv_silu(const float* proj, int ld, int col, int channels, int taps,
                            const float* w, const float* bias, float* state, float* out,
                            const int* positions, const int* entry_of_token, const int* q_start,
                            const int* slot_ids, int num_tokens, int num_entries, int max_q_len,
                            const float* in_bias, int plain, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (channels <= 0 || taps < 1 || col < 0 || col + channels > ld)
    TS_FAIL("conv_silu: bad sizes channels=%d taps=%d col=%d ld=%d", channels, taps, col, ld);
  BatchView b{positions, entry_of_token, q_start, slot_ids};
  if (max_q_len <= 4 && taps <= kMaxTapsInRegisters) {
    const int64_t n = (int64_t)num_entries * channels;
    hipLaunchKernelGGL(conv_silu_walk_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       stream, proj, ld, col, channels, taps, w, bias, state, out, b,
                       num_entries, in_bias, plain);
    TS_CHECK_LAUNCH("conv_silu (walk)");
    return 0;
  }
  if (taps <= kConvMaxTaps && num_tokens >= 256 && (num_tokens + kConvRun - 1) / kConvRun <= 65535) {
    hipLaunchKernelGGL(conv_silu_run_kernel,
                       dim3((unsigned)((channels + 255) / 256), (unsigned)((num_tokens + kConvRun - 1) / kConvRun)),
                       dim3(256), 0, stream, proj, ld, col, channels, taps, w, bias, state, out, b,
                       num_tokens, in_bias, plain);
    TS_CHECK_LAUNCH("conv_silu (runs)");
  } else {
    const int64_t n = (int64_t)num_tokens * channels;
    hipLaunchKernelGGL(conv_silu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                       proj, ld, col, channels, taps, w, bias, state, out, b, num_tokens, in_bias, plain);
    TS_CHECK_LAUNCH("conv_silu");
  }
  if (taps > 1) {
    const int64_t m = (int64_t)num_entries * channels;
    hipLaunchKernelGGL(conv_state_kernel, dim3((unsigned)((m + 255) / 256)), dim3(256), 0, stream,
                       proj, ld, col, channels, taps, state, b, num_entries, in_bias);
    TS_CHECK_LAUNCH("conv_state");
  }
  return 0;
}

// ---------------------------------------------------------------- recurrence
// Per head h (group g): d = softplus(dt + dt_bias[h]), a = exp(-exp(A_log[h]) d),
//   S <- a S + (d B_g) x_h^T   (S: N x P),   y_h = S^T C_g + D[h] x_h.
// A workgroup serves one (run of tokens, head, 64 columns of P): a thread keeps eight-strided
// rows of four columns in registers, walks the tokens in order and adds the eight slices of
// a column's dot product through the wavefront.
//
// Steps of few tokens per entry walk each entry whole (kScanWhole).  A long portion is cut
// into chunks of 64 tokens that run side by side, in three launches: every chunk's
// recurrence from an empty state (its own contribution and the product of its decays,
// kScanLocal); per entry, the state in front of every chunk, one after the other, and the
// state the portion leaves (combine); every chunk once more from its true start state,
// now writing y (kScanOutput).  Twice the arithmetic, a sixty-fourth of the chain.
struct ScanArgs {
  const float* xbc;       // [T, channels]: x (heads*P) | B (groups*N) | C (groups*N)
  const float* proj;      // [T, ld]: dt at column dt_col
  const float* dt_bias;   // [heads]
  const float* a_log;     // [heads]
  const float* d_skip;    // [heads]
  float* state;           // [slots, heads, N, P]
  float* y;               // [T, heads*P]
  BatchView b;
  int ld, dt_col, channels, heads, P, N, groups;
  const int* chunks;      // [num_chunks, 3]: first token, one past the last, entry
  const int* entry_chunks;  // [B + 1]: the chunks of entry e are [entry_chunks[e], entry_chunks[e+1])
  float* chunk_state;     // [num_chunks, heads, N, P]: local contribution, then start state
  float* chunk_decay;     // [num_chunks, heads]
};

constexpr int kScanSlices = 8;
constexpr int kScanCols = 32;              // columns of a workgroup of the combine kernel
constexpr int kScanWhole = 0, kScanLocal = 1, kScanOutput = 2;
constexpr int kScanThreads = 128;          // the walking kernel: 8 slices x 16 groups of columns
constexpr int kScanPerThread = 4;          // columns a thread owns
constexpr int kScanBlockCols = kScanThreads / kScanSlices * kScanPerThread;   // 64
constexpr int kScanStage = 16;             // tokens staged in LDS at a time
static_assert(kScanStage * kScanBlockCols == 8 * kScanThreads, "a stage's x: eight loads a thread");

// (The output pass is held to 168 registers so that three wavefronts share a SIMD: its
// time went from 292 to 220 us at 64 heads of 64 columns and 128 state rows, 2,048 tokens.)
// Thread (cg, s) = (tid / 8, tid % 8) keeps rows s, s + 8, ... of four columns in registers.
// Sixteen tokens' operands (B, C, the workgroup's columns of x, the step and the decay,
// computed once a token) are staged in LDS by all threads together, then walked in order:
// a token costs a thread 2 NI + 3 LDS reads for 8 NI multiply-adds.
template <int NI, int MODE>
__global__ __launch_bounds__(kScanThreads, (MODE == kScanOutput && NI <= 16) ? 3 : 1)
void ssm_scan_kernel(ScanArgs a) {
  extern __shared__ float lds[];
  const int N = a.N;
  float* B_s = lds;                                  // [stage][N]
  float* C_s = B_s + kScanStage * N;                 // [stage][N]
  float* x_s = C_s + kScanStage * N;                 // [stage][64]
  float* d_s = x_s + kScanStage * kScanBlockCols;    // [stage]: step size
  float* a_s = d_s + kScanStage;                     // [stage]: decay
  const int h = blockIdx.x;
  const int s = threadIdx.x % kScanSlices, cg = threadIdx.x / kScanSlices;
  const int col0 = blockIdx.z * kScanBlockCols;
  const int p0 = col0 + cg * kScanPerThread;
  const int g = h / (a.heads / a.groups);
  int first, end, e;
  if (MODE == kScanWhole) {
    e = blockIdx.y;
    first = a.b.q_start[e];
    end = a.b.q_start[e + 1];
  } else {
    first = a.chunks[3 * blockIdx.y];
    end = a.chunks[3 * blockIdx.y + 1];
    e = a.chunks[3 * blockIdx.y + 2];
  }
  const int inner = a.heads * a.P;
  float* st = MODE == kScanWhole
      ? a.state + ((int64_t)a.b.slot_ids[e] * a.heads + h) * N * a.P
      : a.chunk_state + ((int64_t)blockIdx.y * a.heads + h) * N * a.P;
  float S[NI][kScanPerThread];
  const bool fresh = MODE == kScanLocal || (MODE == kScanWhole && a.b.positions[first] == 0);
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s + kScanSlices * i;
#pragma unroll
    for (int c = 0; c < kScanPerThread; ++c)
      S[i][c] = (!fresh && n < N && p0 + c < a.P) ? st[(int64_t)n * a.P + p0 + c] : 0.f;
  }
  const float decay_rate = -expf(a.a_log[h]);
  const float bias = a.dt_bias[h], skip = a.d_skip[h];
  const int b_col = inner + g * N, c_col = inner + a.groups * N + g * N;
  float total_decay = 1.f;

  for (int t0 = first; t0 < end; t0 += kScanStage) {
    const int nt = min(kScanStage, end - t0);
    __syncthreads();                                  // the stage before has been walked
    // Loads in batches of eight, all issued before the first is stored, so that a stage
    // costs a few trips to memory and not one per element.
    {
      const int total = nt * N;
      constexpr int U = 8;
      for (int base = 0; base < total; base += kScanThreads * U) {
        float vb[U], vc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = base + u * kScanThreads + threadIdx.x;
          vb[u] = vc[u] = 0.f;
          if (i < total) {
            const float* row = a.xbc + (int64_t)(t0 + i / N) * a.channels;
            vb[u] = row[b_col + i % N];
            if (MODE != kScanLocal) vc[u] = row[c_col + i % N];
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = base + u * kScanThreads + threadIdx.x;
          if (i < total) {
            B_s[i] = vb[u];
            if (MODE != kScanLocal) C_s[i] = vc[u];
          }
        }
      }
      float vx[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {         // 16 tokens x 64 columns: eight a thread
        const int i = u * kScanThreads + threadIdx.x;
        const int tt = i / kScanBlockCols, c = i % kScanBlockCols;
        vx[u] = (tt < nt && col0 + c < a.P)
            ? a.xbc[(int64_t)(t0 + tt) * a.channels + h * a.P + col0 + c] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) x_s[u * kScanThreads + threadIdx.x] = vx[u];
    }
    if (threadIdx.x < nt) {
      const float d = softplus_f(a.proj[(int64_t)(t0 + threadIdx.x) * a.ld + a.dt_col + h] + bias);
      d_s[threadIdx.x] = d;
      a_s[threadIdx.x] = expf(decay_rate * d);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float d = d_s[tt], decay = a_s[tt];
      float dx[kScanPerThread], x[kScanPerThread], acc[kScanPerThread];
#pragma unroll
      for (int c = 0; c < kScanPerThread; ++c) {
        x[c] = x_s[tt * kScanBlockCols + cg * kScanPerThread + c];
        dx[c] = d * x[c];
        acc[c] = 0.f;
      }
      if (MODE == kScanLocal) {
        total_decay *= decay;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int n = s + kScanSlices * i;
          const float Bv = n < N ? B_s[tt * N + n] : 0.f;
#pragma unroll
          for (int c = 0; c < kScanPerThread; ++c) S[i][c] = fmaf(decay, S[i][c], Bv * dx[c]);
        }
        continue;
      }
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = s + kScanSlices * i;
        const float Bv = n < N ? B_s[tt * N + n] : 0.f;
        const float Cv = n < N ? C_s[tt * N + n] : 0.f;
#pragma unroll
        for (int c = 0; c < kScanPerThread; ++c) {
          S[i][c] = fmaf(decay, S[i][c], Bv * dx[c]);
          acc[c] = fmaf(S[i][c], Cv, acc[c]);
        }
      }
#pragma unroll
      for (int c = 0; c < kScanPerThread; ++c) {
        acc[c] += __shfl_xor(acc[c], 1, kWave);
        acc[c] += __shfl_xor(acc[c], 2, kWave);
        acc[c] += __shfl_xor(acc[c], 4, kWave);
        if (s == 0 && p0 + c < a.P)
          a.y[(int64_t)(t0 + tt) * inner + h * a.P + p0 + c] = fmaf(skip, x[c], acc[c]);
      }
    }
  }
  if (MODE == kScanOutput) return;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s + kScanSlices * i;
#pragma unroll
    for (int c = 0; c < kScanPerThread; ++c)
      if (n < N && p0 + c < a.P) st[(int64_t)n * a.P + p0 + c] = S[i][c];
  }
  if (MODE == kScanLocal && blockIdx.z == 0 && threadIdx.x == 0)
    a.chunk_decay[(int64_t)blockIdx.y * a.heads + h] = total_decay;
}

// Per (head, entry, 32 columns): walks the entry's chunks in order.  chunk_state[c] holds
// the chunk's own contribution and receives the state in front of the chunk; the state
// behind the last chunk goes to the request's slot.
template <int NI>
__global__ __launch_bounds__(kScanSlices* kScanCols) void ssm_combine_kernel(ScanArgs a) {
  const int h = blockIdx.x, e = blockIdx.y;
  const int p = blockIdx.z * kScanCols + threadIdx.x / kScanSlices;
  const int s = threadIdx.x % kScanSlices;
  if (p >= a.P) return;
  const int N = a.N;
  float* st = a.state + ((int64_t)a.b.slot_ids[e] * a.heads + h) * N * a.P;
  const bool fresh = a.b.positions[a.b.q_start[e]] == 0;
  float S[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s + kScanSlices * i;
    S[i] = (!fresh && n < N) ? st[(int64_t)n * a.P + p] : 0.f;
  }
  const int c_begin = a.entry_chunks[e], c_end = a.entry_chunks[e + 1];
  float next[NI], next_decay = 0.f;
  auto fetch = [&](int c) {                 // a chunk's contribution, ahead of its turn
    const float* cs = a.chunk_state + ((int64_t)c * a.heads + h) * N * a.P;
    next_decay = a.chunk_decay[(int64_t)c * a.heads + h];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = s + kScanSlices * i;
      next[i] = n < N ? cs[(int64_t)n * a.P + p] : 0.f;
    }
  };
  if (c_begin < c_end) fetch(c_begin);
  for (int c = c_begin; c < c_end; ++c) {
    float* cs = a.chunk_state + ((int64_t)c * a.heads + h) * N * a.P;
    float local[NI];
    const float decay = next_decay;
#pragma unroll
    for (int i = 0; i < NI; ++i) local[i] = next[i];
    if (c + 1 < c_end) fetch(c + 1);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = s + kScanSlices * i;
      if (n < N) {
        cs[(int64_t)n * a.P + p] = S[i];
        S[i] = fmaf(decay, S[i], local[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s + kScanSlices * i;
    if (n < N) st[(int64_t)n * a.P + p] = S[i];
  }
}

template <int NI>
static void launch_scan(const ScanArgs& a, int num_entries, int num_chunks, hipStream_t stream) {
  const dim3 block(kScanThreads);
  const unsigned z = (a.P + kScanBlockCols - 1) / kScanBlockCols;
  const size_t lds = (size_t)(kScanStage * (2 * a.N + kScanBlockCols + 2)) * sizeof(float);
  if (num_chunks <= 0) {
    hipLaunchKernelGGL((ssm_scan_kernel<NI, kScanWhole>), dim3(a.heads, num_entries, z), block,
                       lds, stream, a);
    return;
  }
  hipLaunchKernelGGL((ssm_scan_kernel<NI, kScanLocal>), dim3(a.heads, num_chunks, z), block, lds,
                     stream, a);
  hipLaunchKernelGGL(ssm_combine_kernel<NI>, dim3(a.heads, num_entries, (a.P + kScanCols - 1) / kScanCols),
                     dim3(kScanSlices * kScanCols), 0, stream, a);
  hipLaunchKernelGGL((ssm_scan_kernel<NI, kScanOutput>), dim3(a.heads, num_chunks, z), block, lds,
                     stream, a);
}

extern "C" int ts_ssm_scan_chunk() { return 64; }

// `num_chunks` 0: every entry is walked whole.  Else `chunks` [num_chunks, 3] cuts every
// entry into runs of tokens (first, one past the last, entry), in order, `entry_chunks`
// [B + 1] says which are whose, and chunk_state [num_chunks, heads, N, P], chunk_decay
// [num_chunks, heads] are scratch.
extern "C" int ts_ssm_scan(const float* xbc, const float* proj, int ld, int dt_col,
                           const float* dt_bias, const float* a_log, const float* d_skip,
                           float* state, float* y, const int* positions,
                           const int* entry_of_token, const int* q_start, const int* slot_ids,
                           int num_tokens, int num_entries, int heads, int P, int N, int groups,
                           const int* chunks, const int* entry_chunks, int num_chunks,
                           float* chunk_state, float* chunk_decay, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || P <= 0 || N <= 0 || groups <= 0 || heads % groups)
    TS_FAIL("ssm_scan: bad sizes heads=%d vdim=%d state=%d groups=%d", heads, P, N, groups);
  if (N > kScanSlices * 32) TS_FAIL("ssm_scan: state of %d rows, at most %d are built", N, kScanSlices * 32);
  if (dt_col < 0 || dt_col + heads > ld) TS_FAIL("ssm_scan: dt columns outside the projection");
  if (num_chunks > 0 && (!chunks || !entry_chunks || !chunk_state || !chunk_decay))
    TS_FAIL("ssm_scan: chunked without its lists and scratch");
  ScanArgs a{xbc, proj, dt_bias, a_log, d_skip, state, y,
             BatchView{positions, entry_of_token, q_start, slot_ids},
             ld, dt_col, heads * P + 2 * groups * N, heads, P, N, groups,
             chunks, entry_chunks, chunk_state, chunk_decay};
  const int ni = (N + kScanSlices - 1) / kScanSlices;
  if (ni <= 2) launch_scan<2>(a, num_entries, num_chunks, stream);
  else if (ni <= 4) launch_scan<4>(a, num_entries, num_chunks, stream);
  else if (ni <= 8) launch_scan<8>(a, num_entries, num_chunks, stream);
  else if (ni <= 16) launch_scan<16>(a, num_entries, num_chunks, stream);
  else launch_scan<32>(a, num_entries, num_chunks, stream);
  TS_CHECK_LAUNCH("ssm_scan");
  return 0;
}

// ---------------------------------------------------------------- gate and group norm
// v = y * silu(z) (z: the first `inner` columns of proj); each of `groups` equal parts of
// a row is divided by its own root mean square; out = that * w.
template <typename TO>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    const float* __restrict__ y, const float* __restrict__ proj, int ld,
    const float* __restrict__ w, TO* __restrict__ out, int inner, int groups, float eps) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const int grp = blockIdx.y, size = inner / groups;
  const float* yr = y + t * inner + grp * size;
  const float* zr = proj + t * ld + grp * size;
  float ss = 0.f;
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    const float v = yr[i] * silu_f(zr[i]);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / (float)size + eps);
  TO* o = out + t * inner + grp * size;
  const float* wr = w + grp * size;
  for (int i = threadIdx.x; i < size; i += blockDim.x)
    o[i] = from_f32<TO>(yr[i] * silu_f(zr[i]) * r * wr[i]);
}

extern "C" int ts_gated_group_norm(const float* y, const float* proj, int ld, const float* w,
                                   void* out, int out_type, int rows, int inner, int groups,
                                   float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (inner <= 0 || groups <= 0 || inner % groups || inner > ld)
    TS_FAIL("gated_group_norm: bad sizes inner=%d groups=%d ld=%d", inner, groups, ld);
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(gated_group_norm_kernel<TO>, dim3(rows, groups), dim3(256),
                                      0, stream, y, proj, ld, w, (TO*)out, inner, groups, eps));
  TS_CHECK_LAUNCH("gated_group_norm");
  return 0;
}
