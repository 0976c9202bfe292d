// Kernels of a gated diagonal linear recurrence (the real-gated linear recurrent unit):
// per channel c, with u the recurrence's input (the convolved branch),
//
//   r = sigmoid(Wa_b u_b + ba),  i = sigmoid(Wi_b u_b + bi)      gates, block by block: the
//                                                                channels stand in equal
//                                                                blocks, each with square
//                                                                matrices of its own
//   log a = rate[c] * r          (rate = -c0 * softplus(lam), made once by the host)
//   S_t = a S_(t-1) + sqrt(1 - a^2) (i u)                        from S = 0 at a sequence's start
//   out_t = S_t * gelu_tanh(y_t + by)                            y: the other branch
//
// All arithmetic in float32.  The state lives in float32 per-request slots; a request's slot
// is read only where a portion does not start at position 0 and written once a portion.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_lru;
typedef __attribute__((ext_vector_type(4))) float f32x4_lru;

struct LruBatch {
  const int* positions;       // [T]
  const int* entry_of_token;  // [T]
  const int* q_start;         // [B + 1]
  const int* slot_ids;        // [B]
};

__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---------------------------------------------------------------- gates
// A workgroup per (TT tokens, block).  The tokens' inputs of the block lie in LDS; a thread
// owns output channels of the block and walks its two weight rows once for all TT tokens.
// A (token, channel)'s sums are added in the order of the block's inputs whatever the tile.
// Leaves a [T, width] and x = sqrt(1 - a^2) i u [T, width].
template <typename W>
__device__ __forceinline__ void load8(const W* p, float (&v)[8]);
template <>
__device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
  const f32x4_lru lo = *(const f32x4_lru*)p, hi = *(const f32x4_lru*)(p + 4);
#pragma unroll
  for (int k = 0; k < 4; ++k) { v[k] = lo[k]; v[4 + k] = hi[k]; }
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&v)[8]) {
  const bf16x8_lru x = *(const bf16x8_lru*)p;
#pragma unroll
  for (int k = 0; k < 8; ++k) v[k] = (float)x[k];
}

template <typename W, int TT>
__global__ __launch_bounds__(256) void rglru_gates_kernel(
    const float* __restrict__ u, const W* __restrict__ wa, const W* __restrict__ wi,
    const float* __restrict__ ba, const float* __restrict__ bi, const float* __restrict__ rate,
    float* __restrict__ a_out, float* __restrict__ x_out, int T, int width, int bw) {
  extern __shared__ float u_s[];                 // [TT][bw]
  const int t0 = blockIdx.x * TT, b = blockIdx.y;
  for (int idx = threadIdx.x; idx < TT * bw; idx += blockDim.x) {
    const int tt = idx / bw, j = idx % bw;
    u_s[idx] = t0 + tt < T ? u[(int64_t)(t0 + tt) * width + b * bw + j] : 0.f;
  }
  __syncthreads();
  const bool vec = bw % 8 == 0;
  for (int o = threadIdx.x; o < bw; o += blockDim.x) {
    const int c = b * bw + o;
    const W* ra = wa + (int64_t)c * bw;
    const W* ri = wi + (int64_t)c * bw;
    float sr[TT], si[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) sr[tt] = si[tt] = 0.f;
    if (vec) {
      for (int j = 0; j < bw; j += 8) {
        float va[8], vi[8];
        load8<W>(ra + j, va);
        load8<W>(ri + j, vi);
#pragma unroll
        for (int k = 0; k < 8; ++k)
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            const float x = u_s[tt * bw + j + k];
            sr[tt] = fmaf(va[k], x, sr[tt]);
            si[tt] = fmaf(vi[k], x, si[tt]);
          }
      }
    } else {
      for (int j = 0; j < bw; ++j) {
        const float va = to_f32(ra[j]), vi = to_f32(ri[j]);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          const float x = u_s[tt * bw + j];
          sr[tt] = fmaf(va, x, sr[tt]);
          si[tt] = fmaf(vi, x, si[tt]);
        }
      }
    }
    const float rb = ba[c], ib = bi[c], rt = rate[c];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      if (t0 + tt >= T) break;
      const float r = sigmoid_f(sr[tt] + rb), g = sigmoid_f(si[tt] + ib);
      const float log_a = rt * r;
      // 1 - a^2 = -(exp(2 log a) - 1), without the cancellation next to a = 1
      const float feed = sqrtf(-expm1f(2.0f * log_a)) * g * u_s[tt * bw + o];
      a_out[(int64_t)(t0 + tt) * width + c] = expf(log_a);
      x_out[(int64_t)(t0 + tt) * width + c] = feed;
    }
  }
}

// The same on the matrix cores, for bfloat16 weights and blocks whose size is a multiple of
// 16: D = W U^T by v_mfma_f32_16x16x32_bf16, the first operand 16 output channels of a
// gate's matrix straight from global memory (lane (r, g), r = lane % 16, g = lane / 16, holds
// W[channel r][k = g * 8 .. + 7]), the second 16 tokens' inputs, rounded to bfloat16 and
// staged in LDS for all of the workgroup's waves; lane (r, g) then holds D[channel g * 4 +
// e][token r], e = 0 .. 3: four neighbouring channels of one token, written as one 16-byte
// store.  A workgroup takes kGateTokens tokens of one block and 16 channels a wave; K runs
// in chunks of kGateChunk inputs (a wave's weights of a chunk stay in registers over the
// token tiles).  The sums are float32, in the order of K whatever else is in the launch;
// sigmoid, decay and feed are float32 on them and on the unrounded input.
constexpr int kGateTokens = 64, kGateChunk = 256, kGateStride = kGateChunk + 8;

__global__ __launch_bounds__(256) void rglru_gates_mfma_kernel(
    const float* __restrict__ u, const bf16_t* __restrict__ wa, const bf16_t* __restrict__ wi,
    const float* __restrict__ ba, const float* __restrict__ bi, const float* __restrict__ rate,
    float* __restrict__ a_out, float* __restrict__ x_out, int T, int width, int bw) {
  __shared__ __attribute__((aligned(16))) bf16_t u_s[kGateTokens * kGateStride];
  constexpr int NT = kGateTokens / 16, KS = kGateChunk / 32;
  const int nwaves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int per_block = (bw / 16 + nwaves - 1) / nwaves;       // workgroups a block
  const int b = blockIdx.y / per_block;
  const int ct = (blockIdx.y % per_block) * nwaves + wave;      // the wave's tile of 16 channels
  const bool has_tile = ct * 16 < bw;
  const int t0 = blockIdx.x * kGateTokens;
  const int nt_used = min(NT, (min(T - t0, kGateTokens) + 15) / 16);
  f32x4_lru acc[NT][2];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt][0] = acc[nt][1] = f32x4_lru{0.f, 0.f, 0.f, 0.f};
  const bf16x8_lru zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int64_t wrow = ((int64_t)b * bw + ct * 16 + r) * bw;    // this lane's weight row
  for (int kc = 0; kc < bw; kc += kGateChunk) {
    const int len = min(kGateChunk, bw - kc);
    __syncthreads();                           // the chunk before has been read
    for (int idx = threadIdx.x; idx < nt_used * 16 * (kGateChunk / 8); idx += blockDim.x) {
      const int tt = idx / (kGateChunk / 8), k8 = (idx % (kGateChunk / 8)) * 8;
      bf16x8_lru v = zero8;
      if (t0 + tt < T && k8 < len) {
        const float* src = u + (int64_t)(t0 + tt) * width + b * bw + kc + k8;
        const f32x4_lru lo = *(const f32x4_lru*)src, hi = *(const f32x4_lru*)(src + 4);
#pragma unroll
        for (int k = 0; k < 4; ++k) { v[k] = (bf16_t)lo[k]; v[4 + k] = (bf16_t)hi[k]; }
      }
      *(bf16x8_lru*)(u_s + tt * kGateStride + k8) = v;
    }
    bf16x8_lru ra[KS], ri[KS];
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) {
      const int k = s2 * 32 + g * 8;
      const bool ok = has_tile && k < len;
      ra[s2] = ok ? *(const bf16x8_lru*)(wa + wrow + kc + k) : zero8;
      ri[s2] = ok ? *(const bf16x8_lru*)(wi + wrow + kc + k) : zero8;
    }
    __syncthreads();
    if (!has_tile) continue;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (nt < nt_used) {
#pragma unroll
        for (int s2 = 0; s2 < KS; ++s2) {
          if (s2 * 32 < len) {
            const bf16x8_lru uo =
                *(const bf16x8_lru*)(u_s + (nt * 16 + r) * kGateStride + s2 * 32 + g * 8);
            acc[nt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ra[s2], uo, acc[nt][0], 0, 0, 0);
            acc[nt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ri[s2], uo, acc[nt][1], 0, 0, 0);
          }
        }
      }
    }
  }
  if (!has_tile) return;
  const int c = b * bw + ct * 16 + g * 4;                       // four channels from here
  const f32x4_lru rb = *(const f32x4_lru*)(ba + c), ib = *(const f32x4_lru*)(bi + c),
                  rt = *(const f32x4_lru*)(rate + c);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int t = t0 + nt * 16 + r;
    if (nt >= nt_used || t >= T) continue;
    const f32x4_lru uv = *(const f32x4_lru*)(u + (int64_t)t * width + c);
    f32x4_lru av, xv;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float rr = sigmoid_f(acc[nt][0][e] + rb[e]), gg = sigmoid_f(acc[nt][1][e] + ib[e]);
      const float log_a = rt[e] * rr;
      av[e] = expf(log_a);
      xv[e] = sqrtf(-expm1f(2.0f * log_a)) * gg * uv[e];
    }
    *(f32x4_lru*)(a_out + (int64_t)t * width + c) = av;
    *(f32x4_lru*)(x_out + (int64_t)t * width + c) = xv;
  }
}

// ---------------------------------------------------------------- recurrence
// Walk: a thread per (entry, channel) takes the entry's tokens in order.
template <typename T>
__global__ __launch_bounds__(256) void rglru_walk_kernel(
    const float* __restrict__ a, const float* __restrict__ x, const float* __restrict__ yproj,
    int ld, int ycol, const float* __restrict__ ybias, float* __restrict__ state,
    T* __restrict__ out, LruBatch b, int num_entries, int width) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_entries * width) return;
  const int e = (int)(idx / width), c = (int)(idx % width);
  const int first = b.q_start[e], end = b.q_start[e + 1];
  if (end <= first) return;
  float* st = state + (int64_t)b.slot_ids[e] * width + c;
  float S = b.positions[first] > 0 ? *st : 0.f;
  const float yb = ybias ? ybias[c] : 0.f;
#pragma unroll 4
  for (int t = first; t < end; ++t) {
    S = fmaf(a[(int64_t)t * width + c], S, x[(int64_t)t * width + c]);
    out[(int64_t)t * width + c] = from_f32<T>(S * gelu_tanh_f(yproj[(int64_t)t * ld + ycol + c] + yb));
  }
  *st = S;
}

// Chunks side by side, three launches.  Local: a thread per (chunk, channel) walks the chunk
// from S = 0 and leaves what the chunk adds and the product of its decays.
__global__ __launch_bounds__(256) void rglru_local_kernel(
    const float* __restrict__ a, const float* __restrict__ x, const int* __restrict__ chunks,
    float* __restrict__ chunk_state, float* __restrict__ chunk_decay, int num_chunks, int width) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_chunks * width) return;
  const int k = (int)(idx / width), c = (int)(idx % width);
  const int first = chunks[3 * k], end = chunks[3 * k + 1];
  float S = 0.f, P = 1.f;
#pragma unroll 8
  for (int t = first; t < end; ++t) {
    const float at = a[(int64_t)t * width + c];
    S = fmaf(at, S, x[(int64_t)t * width + c]);
    P *= at;
  }
  chunk_state[idx] = S;
  chunk_decay[idx] = P;
}

// Carry: a thread per (entry, channel) takes the entry's chunks in order; chunk_state
// receives the state in front of each chunk, the request's slot the state behind the last.
__global__ __launch_bounds__(256) void rglru_carry_kernel(
    const int* __restrict__ entry_chunks, float* __restrict__ chunk_state,
    const float* __restrict__ chunk_decay, float* __restrict__ state, LruBatch b,
    int num_entries, int width) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_entries * width) return;
  const int e = (int)(idx / width), c = (int)(idx % width);
  const int k0 = entry_chunks[e], k1 = entry_chunks[e + 1];
  if (k1 <= k0) return;
  float* st = state + (int64_t)b.slot_ids[e] * width + c;
  float S = b.positions[b.q_start[e]] > 0 ? *st : 0.f;
  for (int k = k0; k < k1; ++k) {
    const int64_t at = (int64_t)k * width + c;
    const float own = chunk_state[at];
    chunk_state[at] = S;
    S = fmaf(chunk_decay[at], S, own);
  }
  *st = S;
}

// Output: every chunk once more from the state in front of it.
template <typename T>
__global__ __launch_bounds__(256) void rglru_output_kernel(
    const float* __restrict__ a, const float* __restrict__ x, const float* __restrict__ yproj,
    int ld, int ycol, const float* __restrict__ ybias, const int* __restrict__ chunks,
    const float* __restrict__ chunk_state, T* __restrict__ out, int num_chunks, int width) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)num_chunks * width) return;
  const int k = (int)(idx / width), c = (int)(idx % width);
  const int first = chunks[3 * k], end = chunks[3 * k + 1];
  float S = chunk_state[idx];
  const float yb = ybias ? ybias[c] : 0.f;
#pragma unroll 8
  for (int t = first; t < end; ++t) {
    S = fmaf(a[(int64_t)t * width + c], S, x[(int64_t)t * width + c]);
    out[(int64_t)t * width + c] = from_f32<T>(S * gelu_tanh_f(yproj[(int64_t)t * ld + ycol + c] + yb));
  }
}

// ---------------------------------------------------------------- entry points
// u [T, width] float32; wa, wi [blocks, bw, bw] ([out, in] per block) of `w_type`; ba, bi,
// rate float32 [width].
extern "C" int ts_rglru_gates(const float* u, const void* wa, const void* wi, int w_type,
                              const float* ba, const float* bi, const float* rate, float* a_out,
                              float* x_out, int num_tokens, int width, int blocks,
                              hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || blocks <= 0 || width % blocks) TS_FAIL("rglru_gates: width=%d blocks=%d", width, blocks);
  const int bw = width / blocks;
  if (bw % 8 == 0 && ((((uintptr_t)wa | (uintptr_t)wi) & 15) != 0))
    TS_FAIL("rglru_gates: gate weights must be 16-byte aligned");
  if (w_type == TS_BF16 && bw % 16 == 0 &&
      ((((uintptr_t)u | (uintptr_t)ba | (uintptr_t)bi | (uintptr_t)rate | (uintptr_t)a_out |
         (uintptr_t)x_out) & 15) == 0)) {
    // few tokens: a wave a workgroup, so that the weights' rows are spread over the chip
    const int waves = num_tokens <= 16 ? 1 : 4;
    const int per_block = (bw / 16 + waves - 1) / waves;
    const dim3 grid((num_tokens + kGateTokens - 1) / kGateTokens, blocks * per_block);
    hipLaunchKernelGGL(rglru_gates_mfma_kernel, grid, dim3(waves * kWave), 0, stream, u,
                       (const bf16_t*)wa, (const bf16_t*)wi, ba, bi, rate, a_out, x_out,
                       num_tokens, width, bw);
    TS_CHECK_LAUNCH("rglru_gates (matrix cores)");
    return 0;
  }
  // tokens a workgroup: as many as keep the chip busy and the inputs in LDS
  int tt = num_tokens * blocks >= 2048 ? 8 : num_tokens * blocks >= 512 ? 4 : num_tokens > 1 ? 2 : 1;
  while (tt > 1 && (size_t)tt * bw * sizeof(float) > 60 * 1024) tt /= 2;
  if ((size_t)tt * bw * sizeof(float) > 60 * 1024) TS_FAIL("rglru_gates: blocks of %d channels are more than the kernel holds", bw);
  const dim3 grid((num_tokens + tt - 1) / tt, blocks);
  const size_t lds = (size_t)tt * bw * sizeof(float);
#define TS_LAUNCH(W, TT)                                                                       \
  hipLaunchKernelGGL((rglru_gates_kernel<W, TT>), grid, dim3(256), lds, stream, u, (const W*)wa, \
                     (const W*)wi, ba, bi, rate, a_out, x_out, num_tokens, width, bw)
#define TS_PICK(W)                                                        \
  switch (tt) { case 8: TS_LAUNCH(W, 8); break; case 4: TS_LAUNCH(W, 4); break; \
                case 2: TS_LAUNCH(W, 2); break; default: TS_LAUNCH(W, 1); }
  TS_DISPATCH_TYPE(w_type, W, TS_PICK(W));
#undef TS_PICK
#undef TS_LAUNCH
  TS_CHECK_LAUNCH("rglru_gates");
  return 0;
}

// a, x [T, width]; y: `width` columns of yproj (float32, leading dimension ld) from ycol, plus
// ybias (may be null); state [slots, width]; out [T, width] of out_type.  `num_chunks` 0:
// every entry is walked whole.  Else `chunks` [num_chunks, 3] (first token, one past the
// last, entry) cuts every entry into runs in order, `entry_chunks` [B + 1] says which are
// whose, chunk_state and chunk_decay [num_chunks, width] are scratch.
extern "C" int ts_rglru_scan(const float* a, const float* x, const float* yproj, int ld, int ycol,
                             const float* ybias, float* state, void* out, int out_type,
                             const int* positions, const int* entry_of_token, const int* q_start,
                             const int* slot_ids, int num_tokens, int num_entries, int width,
                             const int* chunks, const int* entry_chunks, int num_chunks,
                             float* chunk_state, float* chunk_decay, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || ycol < 0 || ycol + width > ld) TS_FAIL("rglru_scan: width=%d ycol=%d ld=%d", width, ycol, ld);
  if (num_chunks > 0 && (!chunks || !entry_chunks || !chunk_state || !chunk_decay))
    TS_FAIL("rglru_scan: chunked without its lists and scratch");
  LruBatch b{positions, entry_of_token, q_start, slot_ids};
  const int64_t per_entry = (int64_t)num_entries * width;
  if (num_chunks <= 0) {
    TS_DISPATCH_TYPE(out_type, T,
                     hipLaunchKernelGGL(rglru_walk_kernel<T>, dim3((unsigned)((per_entry + 255) / 256)),
                                        dim3(256), 0, stream, a, x, yproj, ld, ycol, ybias, state,
                                        (T*)out, b, num_entries, width));
    TS_CHECK_LAUNCH("rglru_scan (walk)");
    return 0;
  }
  const int64_t per_chunk = (int64_t)num_chunks * width;
  hipLaunchKernelGGL(rglru_local_kernel, dim3((unsigned)((per_chunk + 255) / 256)), dim3(256), 0,
                     stream, a, x, chunks, chunk_state, chunk_decay, num_chunks, width);
  TS_CHECK_LAUNCH("rglru_scan (local)");
  hipLaunchKernelGGL(rglru_carry_kernel, dim3((unsigned)((per_entry + 255) / 256)), dim3(256), 0,
                     stream, entry_chunks, chunk_state, chunk_decay, state, b, num_entries, width);
  TS_CHECK_LAUNCH("rglru_scan (carry)");
  TS_DISPATCH_TYPE(out_type, T,
                   hipLaunchKernelGGL(rglru_output_kernel<T>, dim3((unsigned)((per_chunk + 255) / 256)),
                                      dim3(256), 0, stream, a, x, yproj, ld, ycol, ybias, chunks,
                                      chunk_state, (T*)out, num_chunks, width));
  TS_CHECK_LAUNCH("rglru_scan (output)");
  return 0;
}

// ---------------------------------------------------------------- activations of rows
// out = relu(x)^2, element by element.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void relu_squared_kernel(const TI* __restrict__ x,
                                                           TO* __restrict__ out, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float v = fmaxf(to_f32(x[i]), 0.f);
    out[i] = from_f32<TO>(v * v);
  }
}

// Eight bfloat16 a thread: 16-byte loads and stores.
__global__ __launch_bounds__(256) void relu_squared_bf16x8_kernel(const bf16_t* __restrict__ x,
                                                                  bf16_t* __restrict__ out,
                                                                  int64_t units) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < units;
       i += (int64_t)gridDim.x * blockDim.x) {
    const bf16x8_lru v = *(const bf16x8_lru*)(x + i * 8);
    bf16x8_lru o;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float f = fmaxf((float)v[k], 0.f);
      o[k] = (bf16_t)(f * f);
    }
    *(bf16x8_lru*)(out + i * 8) = o;
  }
}

extern "C" int ts_relu_squared(const void* x, int x_type, void* out, int out_type, int64_t n,
                               hipStream_t stream) {
  if (n <= 0) return 0;
  if (x_type == TS_BF16 && out_type == TS_BF16 && n % 8 == 0 &&
      (((uintptr_t)x | (uintptr_t)out) & 15) == 0) {
    const int64_t units = n / 8;
    const int blocks8 = (int)((units + 255) / 256 > 16384 ? 16384 : (units + 255) / 256);
    hipLaunchKernelGGL(relu_squared_bf16x8_kernel, dim3(blocks8), dim3(256), 0, stream,
                       (const bf16_t*)x, (bf16_t*)out, units);
    TS_CHECK_LAUNCH("relu_squared");
    return 0;
  }
  const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
  TS_DISPATCH_TYPE(x_type, TI, TS_DISPATCH_TYPE(out_type, TO,
      hipLaunchKernelGGL((relu_squared_kernel<TI, TO>), dim3(blocks), dim3(256), 0, stream,
                         (const TI*)x, (TO*)out, n)));
  TS_CHECK_LAUNCH("relu_squared");
  return 0;
}

// out[r][c] = x[r][c] * sigmoid(gate[r][gate_col + c]); gate rows have leading dimension ld.
template <typename TX, typename TG, typename TO>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(
    const TX* __restrict__ x, const TG* __restrict__ gate, int ld, int gate_col,
    TO* __restrict__ out, int64_t total, int cols, int group) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cols;
    const int c = (int)(i - r * cols) / group;
    out[i] = from_f32<TO>(to_f32(x[i]) * sigmoid_f(to_f32(gate[r * ld + gate_col + c])));
  }
}

// `group`: columns of x that share one gate (1: a gate a column; a head's size: a gate a head).
extern "C" int ts_sigmoid_gate(const void* x, int x_type, const void* gate, int gate_type, int ld,
                               int gate_col, void* out, int out_type, int rows, int cols,
                               int group, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (cols <= 0 || group <= 0 || cols % group || gate_col < 0 || gate_col + cols / group > ld)
    TS_FAIL("sigmoid_gate: cols=%d group=%d gate_col=%d ld=%d", cols, group, gate_col, ld);
  const int64_t total = (int64_t)rows * cols;
  const int blocks = (int)((total + 255) / 256 > 65535 ? 65535 : (total + 255) / 256);
  TS_DISPATCH_TYPE(x_type, TX, TS_DISPATCH_TYPE(gate_type, TG, TS_DISPATCH_TYPE(out_type, TO,
      hipLaunchKernelGGL((sigmoid_gate_kernel<TX, TG, TO>), dim3(blocks), dim3(256), 0, stream,
                         (const TX*)x, (const TG*)gate, ld, gate_col, (TO*)out, total, cols,
                         group))));
  TS_CHECK_LAUNCH("sigmoid_gate");
  return 0;
}
