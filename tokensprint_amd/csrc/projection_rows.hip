// Rows of a q/k/v projection between the product and attention: biases, a norm over a whole
// projection, keys that serve as values.
#include "common.h"

// x[r][c] += bias[c] for the first `n` columns of float32 rows of `ld` columns, in place.
__global__ __launch_bounds__(256) void add_bias_kernel(float* __restrict__ x,
                                                       const float* __restrict__ bias,
                                                       int64_t total, int n, int ld) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t r = idx / n;
  const int c = (int)(idx - r * n);
  x[r * ld + c] += bias[c];
}

extern "C" int ts_add_bias(float* x, const float* bias, int rows, int n, int ld,
                           hipStream_t stream) {
  if (rows <= 0 || n <= 0) return 0;
  if (n > ld) TS_FAIL("add_bias: %d biases for rows of %d", n, ld);
  const int64_t total = (int64_t)rows * n;
  hipLaunchKernelGGL(add_bias_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                     x, bias, total, n, ld);
  TS_CHECK_LAUNCH("add_bias");
  return 0;
}

// One workgroup a row.  in [rows, q | k | v | extra] float32, where v is absent with
// `values_from_keys`; out [rows, q | k | v | extra] in either type.
//   x = in + bias (bias over the first `bias_n` columns of `in`, or null)
//   q <- q / sqrt(sum(q^2) / q_count + eps) * q_norm   (q_norm null: q as it is), k likewise
//   v <- k as it was before its norm (values_from_keys), else the row's own v
// The counts are those of the values that are not padding, so the mean is the model's.
template <typename TO>
__global__ __launch_bounds__(256) void finish_projection_kernel(
    const float* __restrict__ in, const float* __restrict__ bias, int bias_n,
    const float* __restrict__ q_norm, const float* __restrict__ k_norm, TO* __restrict__ out,
    int q_cols, int k_cols, int v_cols, int extra, int values_from_keys, float q_count,
    float k_count, float eps) {
  __shared__ float scratch[8];
  const int in_v = values_from_keys ? 0 : v_cols;
  const int in_ld = q_cols + k_cols + in_v + extra, out_ld = q_cols + k_cols + v_cols + extra;
  const float* x = in + (int64_t)blockIdx.x * in_ld;
  TO* o = out + (int64_t)blockIdx.x * out_ld;
  float rq = 1.f, rk = 1.f;
  if (q_norm) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < q_cols; c += blockDim.x) {
      const float v = x[c] + (bias && c < bias_n ? bias[c] : 0.f);
      ss = fmaf(v, v, ss);
    }
    rq = 1.0f / sqrtf(block_sum(ss, scratch) / q_count + eps);
  }
  if (k_norm) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < k_cols; c += blockDim.x) {
      const float v = x[q_cols + c] + (bias && q_cols + c < bias_n ? bias[q_cols + c] : 0.f);
      ss = fmaf(v, v, ss);
    }
    rk = 1.0f / sqrtf(block_sum(ss, scratch) / k_count + eps);
  }
  for (int c = threadIdx.x; c < in_ld; c += blockDim.x) {
    const float v = x[c] + (bias && c < bias_n ? bias[c] : 0.f);
    if (c < q_cols) {
      o[c] = from_f32<TO>(q_norm ? v * rq * q_norm[c] : v);
    } else if (c < q_cols + k_cols) {
      const int j = c - q_cols;
      o[c] = from_f32<TO>(k_norm ? v * rk * k_norm[j] : v);
      if (values_from_keys) o[c + k_cols] = from_f32<TO>(v);
    } else {
      o[c + (values_from_keys ? v_cols : 0)] = from_f32<TO>(v);
    }
  }
}

// The same for rows whose parts all begin at multiples of four columns: a thread asks for
// all its columns at once, sixteen bytes each (up to kKeep fours a thread), so that a step
// of few rows costs one trip to memory, and keeps them in registers between the sums of
// squares and the write.
typedef __attribute__((ext_vector_type(4))) float f32x4_p;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_p;
__device__ __forceinline__ void store4_p(float* p, f32x4_p v) { *(f32x4_p*)p = v; }
__device__ __forceinline__ void store4_p(bf16_t* p, f32x4_p v) {
  *(bf16x4_p*)p = bf16x4_p{(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
}

template <typename TO>
__global__ __launch_bounds__(512) void finish_projection_vec_kernel(
    const float* __restrict__ in, const float* __restrict__ bias, int bias_n,
    const float* __restrict__ q_norm, const float* __restrict__ k_norm, TO* __restrict__ out,
    int q_cols, int k_cols, int v_cols, int extra, int values_from_keys, float q_count,
    float k_count, float eps) {
  constexpr int kKeep = 8;
  __shared__ float scratch[8];
  const int in_v = values_from_keys ? 0 : v_cols;
  const int in_ld = q_cols + k_cols + in_v + extra, out_ld = q_cols + k_cols + v_cols + extra;
  const float* x = in + (int64_t)blockIdx.x * in_ld;
  TO* o = out + (int64_t)blockIdx.x * out_ld;
  f32x4_p keep[kKeep];
  float ssq = 0.f, ssk = 0.f;
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int c = (j * blockDim.x + threadIdx.x) * 4;
    keep[j] = c < in_ld ? *(const f32x4_p*)(x + c) : f32x4_p{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int c = (j * blockDim.x + threadIdx.x) * 4;
    if (c >= in_ld) continue;
    if (bias && c < bias_n) keep[j] += *(const f32x4_p*)(bias + c);
    const f32x4_p v = keep[j];
    const float sq = v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    if (c < q_cols) ssq += sq;
    else if (c < q_cols + k_cols) ssk += sq;
  }
  float rq = 1.f, rk = 1.f;
  if (q_norm) rq = 1.0f / sqrtf(block_sum(ssq, scratch) / q_count + eps);
  if (k_norm) rk = 1.0f / sqrtf(block_sum(ssk, scratch) / k_count + eps);
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int c = (j * blockDim.x + threadIdx.x) * 4;
    if (c >= in_ld) continue;
    const f32x4_p v = keep[j];
    if (c < q_cols) {
      store4_p(o + c, q_norm ? v * rq * *(const f32x4_p*)(q_norm + c) : v);
    } else if (c < q_cols + k_cols) {
      store4_p(o + c, k_norm ? v * rk * *(const f32x4_p*)(k_norm + (c - q_cols)) : v);
      if (values_from_keys) store4_p(o + c + k_cols, v);
    } else {
      store4_p(o + c + (values_from_keys ? v_cols : 0), v);
    }
  }
}

extern "C" int ts_finish_projection(const float* in, const float* bias, int bias_n,
                                    const float* q_norm, const float* k_norm, void* out,
                                    int out_type, int rows, int q_cols, int k_cols, int v_cols,
                                    int extra, int values_from_keys, int q_count, int k_count,
                                    float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  const int in_ld = q_cols + k_cols + (values_from_keys ? 0 : v_cols) + extra;
  if (q_cols <= 0 || k_cols < 0 || v_cols < 0 || extra < 0 || bias_n < 0 || bias_n > in_ld ||
      (values_from_keys && v_cols != k_cols) || (q_norm && q_count <= 0) ||
      (k_norm && (k_count <= 0 || k_cols == 0)))
    TS_FAIL("finish_projection: q=%d k=%d v=%d extra=%d bias=%d", q_cols, k_cols, v_cols, extra,
            bias_n);
  const bool fours = ((q_cols | k_cols | v_cols | extra | bias_n) & 3) == 0 &&
                     (((uintptr_t)in | (uintptr_t)bias | (uintptr_t)q_norm | (uintptr_t)k_norm |
                       (uintptr_t)out) & 15) == 0;
  if (fours && in_ld <= 512 * 8 * 4) {
    const int want = (in_ld / 4 + 63) / 64 * 64;          // a thread a four, in whole waves
    const int vthreads = want > 512 ? 512 : want;
    TS_DISPATCH_TYPE(out_type, TO,
                     hipLaunchKernelGGL(finish_projection_vec_kernel<TO>, dim3(rows), dim3(vthreads),
                                        0, stream, in, bias, bias_n, q_norm, k_norm, (TO*)out, q_cols,
                                        k_cols, v_cols, extra, values_from_keys, (float)q_count,
                                        (float)k_count, eps));
    TS_CHECK_LAUNCH("finish_projection");
    return 0;
  }
  const int threads = in_ld >= 1024 ? 256 : (in_ld >= 256 ? 128 : 64);
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(finish_projection_kernel<TO>, dim3(rows), dim3(threads), 0,
                                      stream, in, bias, bias_n, q_norm, k_norm, (TO*)out, q_cols,
                                      k_cols, v_cols, extra, values_from_keys, (float)q_count,
                                      (float)k_count, eps));
  TS_CHECK_LAUNCH("finish_projection");
  return 0;
}
