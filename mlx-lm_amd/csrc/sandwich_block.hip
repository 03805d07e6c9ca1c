// The sums of a layer whose sublayers are normed on both sides:
//   h += mult * LN(y; w_post)            (y: a sublayer's output, 32-bit rows)
//   out = LN(h; w_next)                  (optional: the norm ahead of the next sublayer)
// with LN(x; w) = (x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations, no
// bias.  Means, variances, the scaled sum and the stream are 32-bit; `out` is float or bfloat16.
// A block a row; the new row of the stream waits in LDS for its own norm, so the stream is read
// and written once.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void add_normed_kernel(float* __restrict__ h, int ldh, const float* __restrict__ y,
                                                         int ldy, const float* __restrict__ w_post, float mult,
                                                         float eps, const float* __restrict__ w_next,
                                                         T* __restrict__ out, int width) {
  extern __shared__ float row[];
  __shared__ float red[32];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* yr = y + (size_t)r * ldy;
  float* hr = h + (size_t)r * ldh;
  float s = 0.f;
  for (int k = tid; k < width; k += 256) s += (row[k] = yr[k]);
  const float mean = block_sum(s, red) / (float)width;
  float q = 0.f;
  for (int k = tid; k < width; k += 256) {
    const float d = row[k] - mean;
    q += d * d;
  }
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  s = 0.f;
  for (int k = tid; k < width; k += 256) {
    const float v = hr[k] + mult * ((row[k] - mean) * rstd * w_post[k]);
    hr[k] = v, row[k] = v, s += v;
  }
  if (!w_next) return;
  const float mean2 = block_sum(s, red) / (float)width;
  q = 0.f;
  for (int k = tid; k < width; k += 256) {
    const float d = row[k] - mean2;
    q += d * d;
  }
  const float rstd2 = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  for (int k = tid; k < width; k += 256) out[(size_t)r * width + k] = from_f32<T>((row[k] - mean2) * rstd2 * w_next[k]);
}

// The same for few rows (a decode step): a wave a row with the row in registers (NV values a
// lane, width <= 64 NV), every load on its way at once and no barrier: what a row costs is two
// trips to memory.
template <typename T, int NV>
__global__ __launch_bounds__(256) void add_normed_rows_kernel(float* __restrict__ h, int ldh, const float* __restrict__ y,
                                                              int ldy, const float* __restrict__ w_post, float mult,
                                                              float eps, const float* __restrict__ w_next,
                                                              T* __restrict__ out, int n_rows, int width) {
  const int lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;  // whole waves leave; no barrier follows
  const float* yr = y + (size_t)r * ldy;
  float* hr = h + (size_t)r * ldh;
  float yv[NV], hv[NV], wp[NV], wn[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = min(lane + 64 * i, width - 1);
    yv[i] = yr[k], hv[i] = hr[k], wp[i] = w_post[k], wn[i] = w_next ? w_next[k] : 0.f;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) s += lane + 64 * i < width ? yv[i] : 0.f;
  const float mean = wave_sum(s) / (float)width;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const float d = lane + 64 * i < width ? yv[i] - mean : 0.f;
    q += d * d;
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
  s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    hv[i] += mult * ((yv[i] - mean) * rstd * wp[i]);
    if (lane + 64 * i < width) hr[lane + 64 * i] = hv[i], s += hv[i];
  }
  if (!w_next) return;
  const float mean2 = wave_sum(s) / (float)width;
  q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const float d = lane + 64 * i < width ? hv[i] - mean2 : 0.f;
    q += d * d;
  }
  const float rstd2 = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if (lane + 64 * i < width) out[(size_t)r * width + lane + 64 * i] = from_f32<T>((hv[i] - mean2) * rstd2 * wn[i]);
}

DEFINE_LAST_ERROR(mlxlm_last_error)

#define MAX_ROW_WIDTH 15360  // floats of a row that fit the 60 KB of LDS a block asks for

extern "C" int add_normed(float* h, int ldh, const float* y, int ldy, const float* w_post, float mult, float eps,
                          const float* w_next, void* out, int n_rows, int width, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!h || !y || !w_post) FAIL("add_normed: null pointer");
  if (width <= 0 || width > MAX_ROW_WIDTH || ldh < width || ldy < width)
    FAIL("add_normed: width %d (at most %d), row strides %d and %d", width, MAX_ROW_WIDTH, ldh, ldy);
  if (w_next && !out) FAIL("add_normed: a next norm needs an output");
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("add_normed: unknown dtype code %d", out_dtype);
  const int nv = (width + 63) / 64;
  if (n_rows <= 64 && nv <= 32) {
    dim3 grid((n_rows + 3) / 4), block(256);
#define ROWS(T, NV) \
  hipLaunchKernelGGL((add_normed_rows_kernel<T, NV>), grid, block, 0, stream, h, ldh, y, ldy, w_post, mult, eps, w_next, (T*)out, n_rows, width)
#define BY_WIDTH(T)           \
  do {                        \
    if (nv <= 4) ROWS(T, 4);  \
    else if (nv <= 8) ROWS(T, 8);   \
    else if (nv <= 16) ROWS(T, 16); \
    else ROWS(T, 32);         \
  } while (0)
    if (out_dtype == DT_F32)
      BY_WIDTH(float);
    else
      BY_WIDTH(bf16);
#undef BY_WIDTH
#undef ROWS
    CHECK_LAUNCH("add_normed");
    return 0;
  }
  const size_t lds = (size_t)width * sizeof(float);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(add_normed_kernel<float>, dim3(n_rows), dim3(256), lds, stream, h, ldh, y, ldy, w_post, mult, eps,
                       w_next, (float*)out, width);
  else
    hipLaunchKernelGGL(add_normed_kernel<bf16>, dim3(n_rows), dim3(256), lds, stream, h, ldh, y, ldy, w_post, mult, eps,
                       w_next, (bf16*)out, width);
  CHECK_LAUNCH("add_normed");
  return 0;
}

// y = a * ya + b * yb (or y += ...): the sum of two mixers that read the same input.
__global__ __launch_bounds__(256) void scaled_pair_sum_kernel(float* __restrict__ y, float a, const float* __restrict__ ya,
                                                              float b, const float* __restrict__ yb, long n, int accumulate) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = a * ya[i] + b * yb[i];
  y[i] = accumulate ? y[i] + v : v;
}

extern "C" int scaled_pair_sum(float* y, float a, const float* ya, float b, const float* yb, long n, int accumulate,
                               hipStream_t stream) {
  if (n <= 0) return 0;
  if (!y || !ya || !yb) FAIL("scaled_pair_sum: null pointer");
  hipLaunchKernelGGL(scaled_pair_sum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, y, a, ya, b, yb, n, accumulate);
  CHECK_LAUNCH("scaled_pair_sum");
  return 0;
}
