// RMS norm over the last axis of the 32-bit residual stream:
//   y = x / sqrt(mean(x^2) + eps) * gamma          (eps inside the root; gamma may be absent)
// The mean of squares, the root and the scale are computed in 32-bit; the output is float or
// bfloat16.  With `rows` given, output row r is made from input row rows[r] (the rows whose
// logits are wanted).  A wave a row, the row read twice (the second time from the caches).
//
// Also the native part that stands for such a norm in a model (engine_parts.h).
#include "common.h"
#include "engine_parts.h"

template <typename T, int VEC>
__global__ __launch_bounds__(256) void rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ x, int ldx,
                                                      const int* __restrict__ rows, const float* __restrict__ gamma,
                                                      float eps, int n_rows, int width) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;  // whole waves leave; no barrier follows
  const float* xr = x + (size_t)(rows ? rows[r] : r) * ldx;
  float q = 0.f;
  if (VEC == 4) {
    for (int k = lane * 4; k < width; k += 256) {
      const float4 v = *(const float4*)(xr + k);
      q += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
  } else {
    for (int k = lane; k < width; k += 64) q += xr[k] * xr[k];
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
  T* o = out + (size_t)r * width;
  for (int k = lane; k < width; k += 64) o[k] = from_f32<T>(xr[k] * rstd * (gamma ? gamma[k] : 1.f));
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int rmsnorm(void* out, const float* x, int ldx, const int* rows, const float* gamma, float eps, int n_rows,
                       int width, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || ldx < width) FAIL("rmsnorm: width %d, row stride %d", width, ldx);
  if (!out || !x) FAIL("rmsnorm: null pointer");
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("rmsnorm: unknown dtype code %d", out_dtype);
  const bool vec = width % 4 == 0 && ldx % 4 == 0 && !((uintptr_t)x & 15);
  dim3 grid((n_rows + 3) / 4), block(256);
  if (out_dtype == DT_F32) {
    if (vec)
      hipLaunchKernelGGL((rmsnorm_kernel<float, 4>), grid, block, 0, stream, (float*)out, x, ldx, rows, gamma, eps, n_rows, width);
    else
      hipLaunchKernelGGL((rmsnorm_kernel<float, 1>), grid, block, 0, stream, (float*)out, x, ldx, rows, gamma, eps, n_rows, width);
  } else {
    if (vec)
      hipLaunchKernelGGL((rmsnorm_kernel<bf16, 4>), grid, block, 0, stream, (bf16*)out, x, ldx, rows, gamma, eps, n_rows, width);
    else
      hipLaunchKernelGGL((rmsnorm_kernel<bf16, 1>), grid, block, 0, stream, (bf16*)out, x, ldx, rows, gamma, eps, n_rows, width);
  }
  CHECK_LAUNCH("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// the part

static const EngHost* host = nullptr;

struct RmsNorm : Norm {
  int width;
  float eps;
  const float* gamma;
  RmsNorm(int w, float e, const float* g) : width(w), eps(e), gamma(g) {}
  int forward(EngCtx* ctx, const EngMat& x, const int* rows, int n_rows, bool, const EngWeight*, bool,
              EngValue* out) override {
    if (x.cols != width || x.dtype != DT_F32) return host->fail("rmsnorm: float32 rows of width %d", width);
    *out = EngValue{};
    if (host->take(ctx, rows ? n_rows : x.rows, width, ctx->dtype, &out->m)) return 1;
    if (rmsnorm(out->m.p, (const float*)x.p, x.ld, rows, gamma, eps, out->m.rows, width, ctx->dtype, ctx->stream))
      return host->fail("%s", g_err);
    host->launched(ctx);
    return 0;
  }
};

extern "C" EngPart* make_rmsnorm(const EngHost* h, int width, float eps, const float* gamma) {
  host = h;
  return new RmsNorm(width, eps, gamma);
}
