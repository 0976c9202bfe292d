// Routed experts: the choice of a token's experts, and the experts' gated activation.
#include "common.h"

// ---------------------------------------------------------------- router
// One wavefront per token.  scores = softmax(logits) over the E experts; the experts stand in
// `group_count` equal groups of neighbours, a group's score is its best expert's, and only
// the `group_keep` best groups' experts can be chosen; of those the `top` with the largest
// scores (equal scores: the lower index).  weights[t][e] = score / (sum of the chosen scores
// + 1e-20) for the chosen experts and 0 for the others.
// `sigmoid_scores`: scores = sigmoid(logits), each expert by itself, instead of the softmax;
// groups and experts are then ranked by the logits themselves (the same order, also where
// large logits' sigmoids round to the same number).  `normalize` 0: the weights are the
// chosen experts' scores as they are.  `correction` (float32 [E] or null): groups and experts
// are ranked by score + correction, the weights stay the scores.  `weight_scale`: a factor on
// the weights.
__global__ __launch_bounds__(256) void route_experts_kernel(
    const float* __restrict__ logits, float* __restrict__ weights, int rows, int E, int top,
    int group_count, int group_keep, int sigmoid_scores, int normalize,
    const float* __restrict__ correction, float weight_scale) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t t = (int64_t)blockIdx.x * (blockDim.x / kWave) + wave;
  const bool live = t < rows;                    // (every wavefront meets every barrier)
  float* score = lds + (size_t)wave * (3 * E + group_count);
  float* open = score + E;                       // the rank while the expert can be chosen, else -inf
  float* taken = open + E;                       // 1 for a chosen expert
  float* best = taken + E;                       // [group_count]
  const float* z = logits + (live ? t : 0) * E;
  const int per = E / group_count;
  if (sigmoid_scores) {
    for (int e = lane; e < E; e += kWave) {
      score[e] = 1.0f / (1.0f + expf(-z[e]));
      open[e] = z[e];
    }
  } else {
    float m = -INFINITY;
    for (int e = lane; e < E; e += kWave) m = fmaxf(m, z[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += kWave) {
      const float p = expf(z[e] - m);
      score[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    for (int e = lane; e < E; e += kWave) open[e] = score[e] *= inv;
  }
  if (correction)
    for (int e = lane; e < E; e += kWave) open[e] = score[e] + correction[e];
  for (int e = lane; e < E; e += kWave) taken[e] = 0.f;
  __syncthreads();
  for (int g = lane; g < group_count; g += kWave) {
    float b = -INFINITY;
    for (int i = 0; i < per; ++i) b = fmaxf(b, open[g * per + i]);
    best[g] = b;
  }
  __syncthreads();
  for (int g = lane; g < group_count; g += kWave) {
    int ahead = 0;                               // groups that come before this one
    for (int o = 0; o < group_count; ++o)
      ahead += best[o] > best[g] || (best[o] == best[g] && o < g);
    const bool kept = ahead < group_keep;
    if (!kept)
      for (int i = 0; i < per; ++i) open[g * per + i] = -INFINITY;
  }
  __syncthreads();
  float chosen_sum = 0.f;
  float* w = weights + (live ? t : 0) * E;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = E;
    for (int e = lane; e < E; e += kWave)
      if (open[e] > bv) bv = open[e], bi = e;    // ascending e: the lower index at equal scores
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, kWave);
      const int oi = __shfl_xor(bi, o, kWave);
      if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
    }
    if (bi < E) {
      chosen_sum += score[bi];
      if (lane == 0) open[bi] = -INFINITY, taken[bi] = 1.f;
    }
    __syncthreads();
  }
  const float norm = (normalize ? 1.0f / (chosen_sum + 1e-20f) : 1.0f) * weight_scale;
  if (live)
    for (int e = lane; e < E; e += kWave) w[e] = taken[e] != 0.f ? score[e] * norm : 0.f;
}

extern "C" int ts_route_experts(const float* logits, float* weights, int rows, int experts,
                                int top, int group_count, int group_keep, int sigmoid_scores,
                                int normalize, const float* correction, float weight_scale,
                                hipStream_t stream) {
  if (rows <= 0) return 0;
  if (experts <= 0 || group_count <= 0 || experts % group_count || group_keep <= 0 ||
      group_keep > group_count || top <= 0 || top > group_keep * (experts / group_count))
    TS_FAIL("route_experts: %d experts in %d groups, %d kept, cannot give %d", experts,
            group_count, group_keep, top);
  const size_t lds = (size_t)4 * (3 * experts + group_count) * sizeof(float);
  if (lds > 64 * 1024) TS_FAIL("route_experts: %d experts are more than the kernel holds", experts);
  if (correction && sigmoid_scores) TS_FAIL("route_experts: a correction goes with softmax scores");
  hipLaunchKernelGGL(route_experts_kernel, dim3((rows + 3) / 4), dim3(256), lds, stream, logits,
                     weights, rows, experts, top, group_count, group_keep, sigmoid_scores, normalize,
                     correction, weight_scale);
  TS_CHECK_LAUNCH("route_experts");
  return 0;
}

// ---------------------------------------------------------------- activation
// gate_up [rows, E, gate | up] (inner columns each) -> out [rows, E, inner]:
// g = min(gate, limit), u = clamp(up, -limit, limit), out = g sigmoid(1.702 g) (u + 1) times
// the token's weight for the expert; zeros (and no reads) where the weight is zero.
// `weighted_input`: the expert is a plain gated unit whose input was the token times its
// weight w, and both products are linear in it: out = silu(w gate) (w up).
template <typename T>
__global__ __launch_bounds__(256) void expert_activation_kernel(
    const T* __restrict__ gate_up, const float* __restrict__ weights, T* __restrict__ out,
    int64_t total, int E, int inner, float limit, int weighted_input) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t te = idx / inner;                 // token * E + expert
  const int i = (int)(idx % inner);
  const float w = weights[te];
  float y = 0.f;
  if (w != 0.f) {
    const T* src = gate_up + te * 2 * inner;
    if (weighted_input) {
      const float g = w * to_f32(src[i]), u = w * to_f32(src[inner + i]);
      out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
      return;
    }
    const float g = fminf(to_f32(src[i]), limit);
    const float u = fminf(fmaxf(to_f32(src[inner + i]), -limit), limit);
    y = g / (1.0f + expf(-1.702f * g)) * (u + 1.0f) * w;
  }
  out[idx] = from_f32<T>(y);
}

// The same, eight bfloat16 a thread (inner a multiple of 8): 16-byte loads and stores.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_exp;
__global__ __launch_bounds__(256) void expert_activation_bf16x8_kernel(
    const bf16_t* __restrict__ gate_up, const float* __restrict__ weights,
    bf16_t* __restrict__ out, int64_t units, int inner8, float limit, int weighted_input) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= units) return;
  const int64_t te = idx / inner8;                // token * E + expert
  const int i = (int)(idx % inner8) * 8;
  const int inner = inner8 * 8;
  const float w = weights[te];
  bf16x8_exp y = {0, 0, 0, 0, 0, 0, 0, 0};
  if (w != 0.f) {
    const bf16_t* src = gate_up + te * 2 * inner;
    const bf16x8_exp gv = *(const bf16x8_exp*)(src + i), uv = *(const bf16x8_exp*)(src + inner + i);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (weighted_input) {
        const float g = w * (float)gv[k], u = w * (float)uv[k];
        y[k] = (bf16_t)(g / (1.0f + expf(-g)) * u);
      } else {
        const float g = fminf((float)gv[k], limit);
        const float u = fminf(fmaxf((float)uv[k], -limit), limit);
        y[k] = (bf16_t)(g / (1.0f + expf(-1.702f * g)) * (u + 1.0f) * w);
      }
    }
  }
  *(bf16x8_exp*)(out + idx * 8) = y;
}

extern "C" int ts_expert_activation(const void* gate_up, const float* weights, void* out, int type,
                                    int rows, int experts, int inner, float limit,
                                    int weighted_input, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (experts <= 0 || inner <= 0) TS_FAIL("expert_activation: bad sizes");
  const int64_t total = (int64_t)rows * experts * inner;
  if (type == TS_BF16 && inner % 8 == 0 && (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0) {
    const int64_t units = total / 8;
    hipLaunchKernelGGL(expert_activation_bf16x8_kernel, dim3((unsigned)((units + 255) / 256)),
                       dim3(256), 0, stream, (const bf16_t*)gate_up, weights, (bf16_t*)out, units,
                       inner / 8, limit, weighted_input);
    TS_CHECK_LAUNCH("expert_activation");
    return 0;
  }
  TS_DISPATCH_TYPE(type, T,
                   hipLaunchKernelGGL(expert_activation_kernel<T>,
                                      dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                                      (const T*)gate_up, weights, (T*)out, total, experts, inner,
                                      limit, weighted_input));
  TS_CHECK_LAUNCH("expert_activation");
  return 0;
}

// ---------------------------------------------------------------- plain gated units
// gate_up [rows, E x (gate | up) | shared gate | shared up] -> out [rows, E x inner | shared]:
// silu(gate) up times the token's weight for the expert (weights [rows, ld_w], the experts'
// in the first E columns; zeros, and no reads, where the weight is zero), and silu(gate) up
// as it is for the `shared` columns of the unit that every token uses.
template <typename T>
__global__ __launch_bounds__(256) void expert_silu_kernel(
    const T* __restrict__ gate_up, const float* __restrict__ weights, T* __restrict__ out,
    int64_t total, int E, int inner, int shared, int ld_w) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int out_ld = E * inner + shared;
  const int64_t t = idx / out_ld;
  const int c = (int)(idx - t * out_ld);
  const T* row = gate_up + t * (int64_t)(2 * out_ld);
  float y = 0.f;
  if (c < E * inner) {
    const int e = c / inner, i = c - e * inner;
    const float w = weights[t * ld_w + e];
    if (w != 0.f) {
      const float g = to_f32(row[e * 2 * inner + i]), u = to_f32(row[e * 2 * inner + inner + i]);
      y = g / (1.0f + expf(-g)) * u * w;
    }
  } else {
    const int i = c - E * inner;
    const float g = to_f32(row[E * 2 * inner + i]), u = to_f32(row[E * 2 * inner + shared + i]);
    y = g / (1.0f + expf(-g)) * u;
  }
  out[idx] = from_f32<T>(y);
}

// The same, eight bfloat16 a thread (inner and shared multiples of 8): 16-byte loads and
// stores.
__global__ __launch_bounds__(256) void expert_silu_bf16x8_kernel(
    const bf16_t* __restrict__ gate_up, const float* __restrict__ weights,
    bf16_t* __restrict__ out, int64_t units, int E, int inner, int shared, int ld_w) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= units) return;
  const int out_ld = E * inner + shared;
  const int per_row = out_ld / 8;
  const int64_t t = idx / per_row;
  const int c = (int)(idx - t * per_row) * 8;
  const bf16_t* row = gate_up + t * (int64_t)(2 * out_ld);
  bf16x8_exp y = {0, 0, 0, 0, 0, 0, 0, 0};
  float w = 1.f;
  const bf16_t *gp, *up;
  if (c < E * inner) {
    const int e = c / inner, i = c - e * inner;
    w = weights[t * ld_w + e];
    gp = row + e * 2 * inner + i;
    up = gp + inner;
  } else {
    gp = row + E * 2 * inner + (c - E * inner);
    up = gp + shared;
  }
  if (w != 0.f) {
    const bf16x8_exp gv = *(const bf16x8_exp*)gp, uv = *(const bf16x8_exp*)up;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float g = (float)gv[k];
      y[k] = (bf16_t)(g / (1.0f + expf(-g)) * (float)uv[k] * w);
    }
  }
  *(bf16x8_exp*)(out + idx * 8) = y;
}

extern "C" int ts_expert_silu(const void* gate_up, const float* weights, void* out, int type,
                              int rows, int experts, int inner, int shared, int ld_w,
                              hipStream_t stream) {
  if (rows <= 0) return 0;
  if (experts <= 0 || inner <= 0 || shared < 0 || ld_w < experts)
    TS_FAIL("expert_silu: %d experts of %d, %d shared, weights of %d", experts, inner, shared, ld_w);
  const int64_t total = (int64_t)rows * ((int64_t)experts * inner + shared);
  if (type == TS_BF16 && inner % 8 == 0 && shared % 8 == 0 &&
      (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0) {
    const int64_t units = total / 8;
    hipLaunchKernelGGL(expert_silu_bf16x8_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256),
                       0, stream, (const bf16_t*)gate_up, weights, (bf16_t*)out, units, experts,
                       inner, shared, ld_w);
    TS_CHECK_LAUNCH("expert_silu");
    return 0;
  }
  TS_DISPATCH_TYPE(type, T,
                   hipLaunchKernelGGL(expert_silu_kernel<T>, dim3((unsigned)((total + 255) / 256)),
                                      dim3(256), 0, stream, (const T*)gate_up, weights, (T*)out,
                                      total, experts, inner, shared, ld_w));
  TS_CHECK_LAUNCH("expert_silu");
  return 0;
}

// out[t] += h[t] * (weights[t][col] + ... + weights[t][col + count - 1]): the share of experts
// that give back what they read.  out float32 [rows, width], h either type.
template <typename T>
__global__ __launch_bounds__(256) void add_weighted_rows_kernel(
    float* __restrict__ out, const T* __restrict__ h, const float* __restrict__ weights,
    int64_t total, int width, int ld_w, int col, int count) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t t = idx / width;
  float w = 0.f;
  for (int i = 0; i < count; ++i) w += weights[t * ld_w + col + i];
  if (w != 0.f) out[idx] = fmaf(w, to_f32(h[idx]), out[idx]);
}

extern "C" int ts_add_weighted_rows(float* out, const void* h, int h_type, const float* weights,
                                    int rows, int width, int ld_w, int col, int count,
                                    hipStream_t stream) {
  if (rows <= 0 || count <= 0) return 0;
  if (width <= 0 || col < 0 || col + count > ld_w) TS_FAIL("add_weighted_rows: columns outside the weights");
  const int64_t total = (int64_t)rows * width;
  TS_DISPATCH_TYPE(h_type, T,
                   hipLaunchKernelGGL(add_weighted_rows_kernel<T>, dim3((unsigned)((total + 255) / 256)),
                                      dim3(256), 0, stream, out, (const T*)h, weights, total, width,
                                      ld_w, col, count));
  TS_CHECK_LAUNCH("add_weighted_rows");
  return 0;
}
