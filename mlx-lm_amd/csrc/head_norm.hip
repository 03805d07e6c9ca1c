// RMS norm of every head of a row, in place:
//   x[t, h, 0:dim] <- x[t, h, 0:dim] / sqrt(mean(x[t, h, 0:dim]^2) + eps) * w[0:dim]
// for rows whose heads lie `head_stride` columns apart (a head may be padded beyond `dim`; the
// padding is neither read nor written).  One weight of `dim` values is shared by all heads (w may
// be absent).  The mean of squares, the root and the product are 32-bit.  A wave a (row, head).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(T* __restrict__ x, int ld, int n_rows, int n_heads,
                                                           int head_stride, int dim, const float* __restrict__ w,
                                                           float eps) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)n_rows * n_heads) return;  // whole waves leave; no barrier follows
  T* p = x + (size_t)(item / n_heads) * ld + (size_t)(item % n_heads) * head_stride;
  float q = 0.f;
  for (int k = lane; k < dim; k += 64) {
    const float v = to_f32(p[k]);
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)dim + eps);
  for (int k = lane; k < dim; k += 64) p[k] = from_f32<T>(to_f32(p[k]) * rstd * (w ? w[k] : 1.f));
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int head_rmsnorm(void* x, int ld, int n_rows, int n_heads, int head_stride, int dim, const float* w,
                            float eps, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || n_heads <= 0) return 0;
  if (!x) FAIL("head_rmsnorm: null pointer");
  if (dim <= 0 || dim > head_stride || (long)(n_heads - 1) * head_stride + dim > ld)
    FAIL("head_rmsnorm: %d heads of %d columns, %d apart, in rows of %d", n_heads, dim, head_stride, ld);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("head_rmsnorm: unknown dtype code %d", dtype);
  const long items = (long)n_rows * n_heads;
  dim3 grid((unsigned)((items + 3) / 4)), block(256);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(head_rmsnorm_kernel<float>, grid, block, 0, stream, (float*)x, ld, n_rows, n_heads, head_stride, dim, w, eps);
  else
    hipLaunchKernelGGL(head_rmsnorm_kernel<bf16>, grid, block, 0, stream, (bf16*)x, ld, n_rows, n_heads, head_stride, dim, w, eps);
  CHECK_LAUNCH("head_rmsnorm");
  return 0;
}
