// A layer whose norms come after the sums:
//   u = shift(h);  h <- N1(alpha h + s1 * mixer(u));  h <- N2(alpha h + s2 * ffn(h))
// with N an RMS norm with a weight, s1 and s2 optional per-column scales of the sublayers'
// outputs, and shift an optional mix of each row with the row before it,
//   u_t = h_t + (h_{t-1} - h_t) * mu        (per column; the row before a request's first: zeros)
// whose h_{t-1}, for the first row of a portion, is the request's row of a state tensor: the last
// row of the portion before, as it was when that portion's shift read it.
//
// Everything here is computed in 32-bit on the 32-bit stream.  Kernels:
//  * token_shift: the mixer's input in the compute dtype (without mu: a plain conversion).
//  * residual_rmsnorm: h <- N(alpha h + s * y) in place, a wave a row; on the way it can keep
//    the old rows that end a request's portion in the state tensor (the shift of the next step
//    reads them) and leave a copy of the new rows in the compute dtype for the product that
//    reads them next.
// and the native arrangement that launches them around its mixer and feed-forward.
#include "common.h"
#include "engine_parts.h"

template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(T* __restrict__ out, const float* __restrict__ x, int ldx,
                                                          const float* __restrict__ mu,
                                                          const float* __restrict__ state, size_t state_stride,
                                                          const int* __restrict__ slot_ids,
                                                          const int* __restrict__ token_req, int n_rows, int width) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  const float* xr = x + (size_t)r * ldx;
  T* o = out + (size_t)r * width;
  if (!mu) {
    for (int k = lane; k < width; k += 64) o[k] = from_f32<T>(xr[k]);
    return;
  }
  const int req = token_req[r];
  const bool first = r == 0 || token_req[r - 1] != req;  // a request's rows are consecutive
  const float* prev = first ? state + (size_t)slot_ids[req] * state_stride : xr - ldx;
  for (int k = lane; k < width; k += 64) {
    const float v = xr[k];
    o[k] = from_f32<T>(v + (prev[k] - v) * mu[k]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void residual_rmsnorm_kernel(float* __restrict__ h, int ldh,
                                                               const float* __restrict__ y, int ldy, float alpha,
                                                               const float* __restrict__ s,
                                                               const float* __restrict__ gamma, float eps,
                                                               float* __restrict__ state, size_t state_stride,
                                                               const int* __restrict__ slot_ids,
                                                               const int* __restrict__ token_req,
                                                               T* __restrict__ copy, int n_rows, int width) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  float* hr = h + (size_t)r * ldh;
  const float* yr = y + (size_t)r * ldy;
  float* keep = nullptr;
  if (state) {
    const int req = token_req[r];
    if (r == n_rows - 1 || token_req[r + 1] != req) keep = state + (size_t)slot_ids[req] * state_stride;
  }
  float q = 0.f;
  for (int k = lane; k < width; k += 64) {
    const float old = hr[k];
    if (keep) keep[k] = old;
    const float v = alpha * old + (s ? s[k] : 1.f) * yr[k];
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
  for (int k = lane; k < width; k += 64) {
    const float v = alpha * hr[k] + (s ? s[k] : 1.f) * yr[k];
    const float n = v * rstd * (gamma ? gamma[k] : 1.f);
    hr[k] = n;
    if (copy) copy[(size_t)r * width + k] = from_f32<T>(n);
  }
}

__global__ void zero_rows_kernel(float* p, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

DEFINE_LAST_ERROR(mlxlm_last_error)

// out [n_rows, width] (out_dtype) = shift(x); mu null: a conversion.  state [slots, state_stride] float32.
extern "C" int token_shift(void* out, const float* x, int ldx, const float* mu, const float* state,
                           size_t state_stride, const int* slot_ids, const int* token_req, int n_rows, int width,
                           int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || ldx < width) FAIL("token_shift: width %d, row stride %d", width, ldx);
  if (!out || !x) FAIL("token_shift: null pointer");
  if (mu && (!state || !slot_ids || !token_req || state_stride < (size_t)width))
    FAIL("token_shift: the shift needs the state tensor (rows of %d), slot ids and token_req", width);
  dim3 grid((n_rows + 3) / 4), block(256);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(token_shift_kernel<float>, grid, block, 0, stream, (float*)out, x, ldx, mu, state, state_stride,
                       slot_ids, token_req, n_rows, width);
  else if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(token_shift_kernel<bf16>, grid, block, 0, stream, (bf16*)out, x, ldx, mu, state, state_stride,
                       slot_ids, token_req, n_rows, width);
  else
    FAIL("token_shift: unknown dtype code %d", out_dtype);
  CHECK_LAUNCH("token_shift");
  return 0;
}

// h [n_rows, width] float32 (row stride ldh) <- N(alpha h + s * y) * gamma, in place.  s, gamma: null = ones.
// state non-null: the old row that ends each request's run of rows goes to the request's row of it.
// copy non-null: the new rows once more, contiguous, in copy_dtype.
extern "C" int residual_rmsnorm(float* h, int ldh, const float* y, int ldy, float alpha, const float* s,
                                const float* gamma, float eps, float* state, size_t state_stride,
                                const int* slot_ids, const int* token_req, void* copy, int copy_dtype, int n_rows,
                                int width, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || ldh < width || ldy < width) FAIL("residual_rmsnorm: width %d, row strides %d and %d", width, ldh, ldy);
  if (!h || !y) FAIL("residual_rmsnorm: null pointer");
  if (state && (!slot_ids || !token_req || state_stride < (size_t)width))
    FAIL("residual_rmsnorm: keeping rows needs slot ids, token_req and state rows of %d", width);
  dim3 grid((n_rows + 3) / 4), block(256);
  if (copy && copy_dtype == DT_BF16)
    hipLaunchKernelGGL(residual_rmsnorm_kernel<bf16>, grid, block, 0, stream, h, ldh, y, ldy, alpha, s, gamma, eps, state,
                       state_stride, slot_ids, token_req, (bf16*)copy, n_rows, width);
  else if (!copy || copy_dtype == DT_F32)
    hipLaunchKernelGGL(residual_rmsnorm_kernel<float>, grid, block, 0, stream, h, ldh, y, ldy, alpha, s, gamma, eps, state,
                       state_stride, slot_ids, token_req, (float*)copy, n_rows, width);
  else
    FAIL("residual_rmsnorm: unknown dtype code %d", copy_dtype);
  CHECK_LAUNCH("residual_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// the arrangement

static const EngHost* host = nullptr;

struct PostNormBlock : Block {
  Mixer* mixer = nullptr;
  FeedForward* ffn = nullptr;  // may be absent: the layer is its mixer's half then
  int width = 0;
  float alpha = 1.f, eps = 0.f;
  const float* gamma1 = nullptr;
  const float* gamma2 = nullptr;
  const float* scale1 = nullptr;  // null: the sublayer's output as it is
  const float* scale2 = nullptr;
  const float* mu = nullptr;  // null: no shift

  int zero(EngCtx* ctx, const EngMat& y) {
    const size_t n = (size_t)y.rows * y.ld;
    hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, (float*)y.p, n);
    if (hipGetLastError() != hipSuccess) return host->fail("post-norm block: the launch failed");
    host->launched(ctx);
    return 0;
  }

  int forward(EngCtx* ctx, const EngMat& h, int slot, bool writes, int state_slot) override {
    if (h.cols != width || h.dtype != DT_F32) return host->fail("post-norm block: a float32 stream of width %d", width);
    const int T = h.rows;
    if (T == 0) return 0;
    float* state = nullptr;
    size_t state_stride = 0;
    if (mu) {
      if (state_slot < 0 || state_slot >= ctx->n_slots) return host->fail("post-norm block: state slot %d of %d", state_slot, ctx->n_slots);
      const EngSlot& s = ctx->slots[state_slot];
      if (s.group != -2 || !s.k || s.dtype != DT_F32 || s.page_stride < (size_t)width)
        return host->fail("post-norm block: cache slot %d is not a float32 state of width %d", state_slot, width);
      state = (float*)s.k, state_stride = s.page_stride;
    }
    const size_t mark = ctx->scratch->offset;
    // what the mixer reads
    EngValue u = {};
    if (mu || ctx->dtype != DT_F32 || h.ld != width) {
      if (host->take(ctx, T, width, ctx->dtype, &u.m)) return 1;
      if (token_shift(u.m.p, (const float*)h.p, h.ld, mu, state, state_stride, ctx->slot_ids, ctx->token_req, T, width,
                      ctx->dtype, ctx->stream))
        return host->fail("%s", g_err);
      host->launched(ctx);
    } else {
      u.m = h;
    }
    EngMat y;
    if (host->take(ctx, T, width, DT_F32, &y)) return 1;
    if (!mixer->overwrite && zero(ctx, y)) return 1;
    if (int rc = mixer->forward(ctx, u, y, slot, writes)) return rc;
    // the first sum and norm; the rows that end a portion are kept for the next step's shift; the
    // feed-forward's product reads a copy in the compute dtype
    EngValue x = {};
    x.m = h;
    if (ffn && ctx->dtype != DT_F32) {
      if (host->take(ctx, T, width, ctx->dtype, &x.m)) return 1;
    }
    if (residual_rmsnorm((float*)h.p, h.ld, (const float*)y.p, y.ld, alpha, scale1, gamma1, eps, state, state_stride,
                         ctx->slot_ids, ctx->token_req, x.m.p != h.p ? x.m.p : nullptr, ctx->dtype, T, width, ctx->stream))
      return host->fail("%s", g_err);
    host->launched(ctx);
    if (ffn) {
      if (!ffn->overwrite && zero(ctx, y)) return 1;
      if (int rc = ffn->forward(ctx, x, y)) return rc;
      if (residual_rmsnorm((float*)h.p, h.ld, (const float*)y.p, y.ld, alpha, scale2, gamma2, eps, nullptr, 0, nullptr,
                           nullptr, nullptr, 0, T, width, ctx->stream))
        return host->fail("%s", g_err);
      host->launched(ctx);
    }
    ctx->scratch->offset = mark;
    return 0;
  }
};

// gamma1 / gamma2: the two norms' weights; scale1 / scale2 and mu may be null; ffn may be null.
extern "C" EngPart* make_post_norm_block(const EngHost* h, EngPart* mixer, EngPart* ffn, int width, float alpha,
                                         float eps, const float* gamma1, const float* gamma2, const float* scale1,
                                         const float* scale2, const float* mu) {
  host = h;
  if (!mixer || mixer->kind != KIND_MIXER || (ffn && ffn->kind != KIND_FFN)) {
    h->fail("make_post_norm_block: a mixer and (or no) feed-forward are needed");
    return nullptr;
  }
  PostNormBlock* b = new PostNormBlock();
  b->mixer = static_cast<Mixer*>(mixer), b->ffn = ffn ? static_cast<FeedForward*>(ffn) : nullptr;
  b->width = width, b->alpha = alpha, b->eps = eps;
  b->gamma1 = gamma1, b->gamma2 = gamma2, b->scale1 = scale1, b->scale2 = scale2, b->mu = mu;
  // the parts of this layer write their outputs where they can, instead of adding to rows of zeros
  if (b->mixer->can_overwrite) b->mixer->overwrite = true;
  if (b->ffn && b->ffn->can_overwrite) b->ffn->overwrite = true;
  return b;
}
