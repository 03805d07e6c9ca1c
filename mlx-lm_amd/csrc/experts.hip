// A feed-forward of many small gated experts of which every token uses a few:
//   router_choice   s = softmax(z) over all router outputs; the `top` largest of s + correction
//                   are chosen (the lower index on a tie); their weights are s itself.
//   silu_mul        act = silu(gate) * up for rows [gate | up]   (a dense gated feed-forward)
//   expert_rows_up / expert_rows_down
//                   a token's chosen experts read straight from the stacked expert weights, a
//                   wave a feature: act[t, j, :] = w_tj silu(Wg_e x_t) * (Wu_e x_t), then
//                   y[t, :] += sum_j Wd_e act[t, j, :] + sum_(j: e is an identity expert) w_tj x_t.
//                   Only the chosen experts' weights are read: the kernels for few tokens.
// The router's softmax, the choice and the weights are 32-bit; products accumulate in 32-bit.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// A thread a token.  The k-th pick is the largest (choice, lowest index first) below the pick
// before it, so nothing has to be remembered but the last pick.
__global__ __launch_bounds__(256) void router_choice_kernel(const float* __restrict__ z, int ldz,
                                                            const float* __restrict__ correction, int n_tokens,
                                                            int n_out, int top, int* __restrict__ idx,
                                                            float* __restrict__ weight) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= n_tokens) return;
  const float* zr = z + (size_t)t * ldz;
  float m = zr[0];
  for (int e = 1; e < n_out; ++e) m = fmaxf(m, zr[e]);
  float sum = 0.f;
  for (int e = 0; e < n_out; ++e) sum += expf(zr[e] - m);
  const float inv = 1.0f / sum;
  float last_c = INFINITY;
  int last_e = -1;
  for (int j = 0; j < top; ++j) {
    float best_c = -INFINITY, best_s = 0.f;
    int best_e = -1;
    for (int e = 0; e < n_out; ++e) {
      const float s = expf(zr[e] - m) * inv;
      const float c = correction ? s + correction[e] : s;
      const bool after = c < last_c || (c == last_c && e > last_e);  // not picked yet
      if (after && (best_e < 0 || c > best_c)) best_c = c, best_e = e, best_s = s;
    }
    idx[(size_t)t * top + j] = best_e, weight[(size_t)t * top + j] = best_s;
    last_c = best_c, last_e = best_e;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gu, int ld, T* __restrict__ out, int ldo,
                                                       int n_rows, int F) {
  const int f = blockIdx.y * 256 + threadIdx.x, r = blockIdx.x;
  if (f >= F) return;
  const T* row = gu + (size_t)r * ld;
  out[(size_t)r * ldo + f] = from_f32<T>(silu_f(to_f32(row[f])) * to_f32(row[F + f]));
}

// Block (token x pick, feature group): a wave a feature at a time, lanes along the width.
template <typename T>
__global__ __launch_bounds__(256) void expert_rows_up_kernel(const T* __restrict__ x, int ldx,
                                                             const T* __restrict__ w_gate, const T* __restrict__ w_up,
                                                             const int* __restrict__ idx,
                                                             const float* __restrict__ weight, int n_experts, int top,
                                                             int F, int width, T* __restrict__ act, int feats_a_block) {
  const int item = blockIdx.x, t = item / top;
  const int e = idx[item];
  if (e >= n_experts) return;  // an identity expert: nothing to compute
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float wt = weight[item];
  const T* xr = x + (size_t)t * ldx;
  const int f_end = min(F, ((int)blockIdx.y + 1) * feats_a_block);
  for (int f = blockIdx.y * feats_a_block + wave; f < f_end; f += 4) {
    const T* g = w_gate + ((size_t)e * F + f) * width;
    const T* u = w_up + ((size_t)e * F + f) * width;
    float sg = 0.f, su = 0.f;
    for (int k = lane; k < width; k += 64) {
      const float xv = to_f32(xr[k]);
      sg += to_f32(g[k]) * xv, su += to_f32(u[k]) * xv;
    }
    sg = wave_sum(sg), su = wave_sum(su);
    if (lane == 0) act[(size_t)item * F + f] = from_f32<T>(wt * silu_f(sg) * su);
  }
}

// Block (token, column group): a wave an output column at a time, lanes along the features.
template <typename T>
__global__ __launch_bounds__(256) void expert_rows_down_kernel(const T* __restrict__ act, const T* __restrict__ w_down,
                                                               const int* __restrict__ idx,
                                                               const float* __restrict__ weight,
                                                               const T* __restrict__ x, int ldx, int n_experts, int top,
                                                               int F, int width, float* __restrict__ y, int ldy,
                                                               int cols_a_block, int accumulate) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n_end = min(width, ((int)blockIdx.y + 1) * cols_a_block);
  for (int n = blockIdx.y * cols_a_block + wave; n < n_end; n += 4) {
    float s = 0.f, same = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = idx[(size_t)t * top + j];
      if (e >= n_experts) {
        same += weight[(size_t)t * top + j];
        continue;
      }
      const T* d = w_down + ((size_t)e * width + n) * F;
      const T* a = act + ((size_t)t * top + j) * F;
      for (int f = lane; f < F; f += 64) s += to_f32(d[f]) * to_f32(a[f]);
    }
    s = wave_sum(s);
    if (lane == 0) {
      const float v = s + same * to_f32(x[(size_t)t * ldx + n]);
      float* o = y + (size_t)t * ldy + n;
      *o = accumulate ? *o + v : v;
    }
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int router_choice(const float* z, int ldz, const float* correction, int n_tokens, int n_out, int top,
                             int* idx, float* weight, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!z || !idx || !weight) FAIL("router_choice: null pointer");
  if (n_out <= 0 || top <= 0 || top > n_out || ldz < n_out) FAIL("router_choice: %d of %d outputs, rows of %d", top, n_out, ldz);
  hipLaunchKernelGGL(router_choice_kernel, dim3((n_tokens + 255) / 256), dim3(256), 0, stream, z, ldz, correction,
                     n_tokens, n_out, top, idx, weight);
  CHECK_LAUNCH("router_choice");
  return 0;
}

extern "C" int silu_mul(const void* gu, int ld, void* out, int ldo, int n_rows, int F, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || F <= 0) return 0;
  if (!gu || !out) FAIL("silu_mul: null pointer");
  if (ld < 2 * F || ldo < F) FAIL("silu_mul: rows of %d for 2 x %d, output rows of %d", ld, F, ldo);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("silu_mul: unknown dtype code %d", dtype);
  dim3 grid(n_rows, (F + 255) / 256), block(256);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, ld, (float*)out, ldo, n_rows, F);
  else
    hipLaunchKernelGGL(silu_mul_kernel<bf16>, grid, block, 0, stream, (const bf16*)gu, ld, (bf16*)out, ldo, n_rows, F);
  CHECK_LAUNCH("silu_mul");
  return 0;
}

// act: [n_tokens * top, F] of the compute dtype; y: float rows.
extern "C" int expert_rows(const void* x, int ldx, const void* w_gate, const void* w_up, const void* w_down,
                           const int* idx, const float* weight, int n_tokens, int n_experts, int top, int F, int width,
                           void* act, float* y, int ldy, int accumulate, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!x || !idx || !weight || !y || (n_experts > 0 && (!w_gate || !w_up || !w_down || !act)))
    FAIL("expert_rows: null pointer");
  if (top <= 0 || F <= 0 || width <= 0 || ldx < width || ldy < width) FAIL("expert_rows: sizes");
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("expert_rows: unknown dtype code %d", dtype);
  const int feats = 16, cols = 16;
  dim3 block(256), up_grid(n_tokens * top, (F + feats - 1) / feats), down_grid(n_tokens, (width + cols - 1) / cols);
#define RUN(T)                                                                                                        \
  do {                                                                                                                \
    if (n_experts > 0)                                                                                                \
      hipLaunchKernelGGL(expert_rows_up_kernel<T>, up_grid, block, 0, stream, (const T*)x, ldx, (const T*)w_gate,     \
                         (const T*)w_up, idx, weight, n_experts, top, F, width, (T*)act, feats);                      \
    hipLaunchKernelGGL(expert_rows_down_kernel<T>, down_grid, block, 0, stream, (const T*)act, (const T*)w_down, idx, \
                       weight, (const T*)x, ldx, n_experts, top, F, width, y, ldy, cols, accumulate);                 \
  } while (0)
  if (dtype == DT_F32)
    RUN(float);
  else
    RUN(bf16);
#undef RUN
  CHECK_LAUNCH("expert_rows");
  return 0;
}
