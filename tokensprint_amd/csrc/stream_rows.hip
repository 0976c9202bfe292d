// Sums of rows around the residual stream (float32 [rows, width]) for layers whose
// sub-layers run side by side.
#include "common.h"

// resid += (a + b), then resid += row; a, b (either element type) and row (float32 [width],
// or, `row_stride` = width, [rows, width]: a row of its own for every row of the stream)
// may each be absent (b only with a).
template <typename TA, typename TB>
__global__ __launch_bounds__(256) void stream_add_kernel(
    float* __restrict__ resid, const TA* __restrict__ a, const TB* __restrict__ b,
    const float* __restrict__ row, int row_stride, int64_t total, int width) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float v = resid[idx];
  if (a) v += b ? to_f32(a[idx]) + to_f32(b[idx]) : to_f32(a[idx]);
  if (row) v += row[(idx / width) * row_stride + idx % width];
  resid[idx] = v;
}

extern "C" int ts_stream_add(float* resid, const void* a, int a_type, const void* b, int b_type,
                             const float* row, int row_stride, int rows, int width,
                             hipStream_t stream) {
  if (rows <= 0) return 0;
  if (b && !a) TS_FAIL("stream_add: a second term without a first");
  if (row_stride != 0 && row_stride != width) TS_FAIL("stream_add: row_stride=%d", row_stride);
  const int64_t total = (int64_t)rows * width;
  const dim3 grid((unsigned)((total + 255) / 256));
  TS_DISPATCH_TYPE(a ? a_type : TS_F32, TA,
    TS_DISPATCH_TYPE(b ? b_type : TS_F32, TB,
      hipLaunchKernelGGL((stream_add_kernel<TA, TB>), grid, dim3(256), 0, stream, resid,
                         (const TA*)a, (const TB*)b, row, row_stride, total, width)));
  TS_CHECK_LAUNCH("stream_add");
  return 0;
}

// The same sum, and the RMS norm of the new stream: out = resid / sqrt(mean(resid^2) + eps) * w.
// One workgroup a row; the row's values wait in registers between the two passes (up to
// eight a thread), or are read back.
template <typename TA, typename TB, typename TO>
__global__ __launch_bounds__(256) void stream_add_norm_kernel(
    float* __restrict__ resid, const TA* __restrict__ a, const TB* __restrict__ b,
    const float* __restrict__ row, int row_stride, const float* __restrict__ w,
    TO* __restrict__ out, int width, float eps) {
  __shared__ float scratch[8];
  constexpr int kKeep = 8;
  const int64_t base = (int64_t)blockIdx.x * width;
  if (row) row += (int64_t)blockIdx.x * row_stride;
  float keep[kKeep], ss = 0.f;
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int c = j * blockDim.x + threadIdx.x;
    keep[j] = 0.f;
    if (c < width) {
      float v = resid[base + c];
      v += b ? to_f32(a[base + c]) + to_f32(b[base + c]) : to_f32(a[base + c]);
      if (row) v += row[c];
      resid[base + c] = keep[j] = v;
      ss = fmaf(v, v, ss);
    }
  }
  for (int c = kKeep * blockDim.x + threadIdx.x; c < width; c += blockDim.x) {
    float v = resid[base + c];
    v += b ? to_f32(a[base + c]) + to_f32(b[base + c]) : to_f32(a[base + c]);
    if (row) v += row[c];
    resid[base + c] = v;
    ss = fmaf(v, v, ss);
  }
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int c = j * blockDim.x + threadIdx.x;
    if (c < width) out[base + c] = from_f32<TO>(keep[j] * r * w[c]);
  }
  for (int c = kKeep * blockDim.x + threadIdx.x; c < width; c += blockDim.x)
    out[base + c] = from_f32<TO>(resid[base + c] * r * w[c]);
}

extern "C" int ts_stream_add_norm(float* resid, const void* a, int a_type, const void* b,
                                  int b_type, const float* row, int row_stride, const float* w,
                                  void* out, int out_type, int rows, int width, float eps,
                                  hipStream_t stream) {
  if (rows <= 0) return 0;
  if (row_stride != 0 && row_stride != width) TS_FAIL("stream_add_norm: row_stride=%d", row_stride);
  if (!a || !w || !out || width <= 0) TS_FAIL("stream_add_norm: a term, a weight and an output");
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  TS_DISPATCH_TYPE(a_type, TA,
    TS_DISPATCH_TYPE(b ? b_type : TS_F32, TB,
      TS_DISPATCH_TYPE(out_type, TO,
        hipLaunchKernelGGL((stream_add_norm_kernel<TA, TB, TO>), dim3(rows), dim3(threads), 0,
                           stream, resid, (const TA*)a, (const TB*)b, row, row_stride, w,
                           (TO*)out, width, eps))));
  TS_CHECK_LAUNCH("stream_add_norm");
  return 0;
}

// out = sa * a + sb * b (float32 out).
template <typename TA, typename TB>
__global__ __launch_bounds__(256) void scaled_sum_kernel(
    const TA* __restrict__ a, float sa, const TB* __restrict__ b, float sb,
    float* __restrict__ out, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = sa * to_f32(a[idx]) + sb * to_f32(b[idx]);
}

extern "C" int ts_scaled_sum(const void* a, int a_type, float sa, const void* b, int b_type,
                             float sb, float* out, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  const int64_t total = (int64_t)rows * width;
  const dim3 grid((unsigned)((total + 255) / 256));
  TS_DISPATCH_TYPE(a_type, TA,
    TS_DISPATCH_TYPE(b_type, TB,
      hipLaunchKernelGGL((scaled_sum_kernel<TA, TB>), grid, dim3(256), 0, stream, (const TA*)a,
                         sa, (const TB*)b, sb, out, total)));
  TS_CHECK_LAUNCH("scaled_sum");
  return 0;
}

// out [rows, count] = columns [col, col + count) of x [rows, ld] (float32), in either type.
template <typename TO>
__global__ __launch_bounds__(256) void take_columns_kernel(
    const float* __restrict__ x, int ld, int col, int count, TO* __restrict__ out, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = from_f32<TO>(x[(idx / count) * ld + col + idx % count]);
}

extern "C" int ts_take_columns(const float* x, int ld, int col, int count, void* out, int out_type,
                               int rows, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (col < 0 || count <= 0 || col + count > ld) TS_FAIL("take_columns: columns outside the rows");
  const int64_t total = (int64_t)rows * count;
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(take_columns_kernel<TO>, dim3((unsigned)((total + 255) / 256)),
                                      dim3(256), 0, stream, x, ld, col, count, (TO*)out, total));
  TS_CHECK_LAUNCH("take_columns");
  return 0;
}
