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
  const int threads = in_ld >= 1024 ? 256 : (in_ld >= 256 ? 128 : 64);
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(finish_projection_kernel<TO>, dim3(rows), dim3(threads), 0,
                                      stream, in, bias, bias_n, q_norm, k_norm, (TO*)out, q_cols,
                                      k_cols, v_cols, extra, values_from_keys, (float)q_count,
                                      (float)k_count, eps));
  TS_CHECK_LAUNCH("finish_projection");
  return 0;
}
