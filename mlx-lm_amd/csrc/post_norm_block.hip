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
//  * residual_rmsnorm: h <- N(alpha h + s * y) in place (y as rows, or as the parts of a product
//    that split its inner size, or both); on the way it can keep
//    the old rows that end a request's portion in the state tensor (the shift of the next step
//    reads them) and leave a copy of the new rows in the compute dtype for the product that
//    reads them next.
// and the native arrangement that launches them around its mixer and feed-forward.
#include "common.h"
#include "engine_parts.h"

// A block a row, the row in registers (NV float4 a thread, width <= 1024 NV): every load of the
// row is on its way before the first is used, so a row costs one trip to memory, not one a
// stretch of 64 columns.  Columns beyond the width are read from inside it and dropped.
template <typename T, int NV>
__global__ __launch_bounds__(256) void token_shift_kernel(T* __restrict__ out, const float* __restrict__ x, int ldx,
                                                          const float* __restrict__ mu,
                                                          const float* __restrict__ state, size_t state_stride,
                                                          const int* __restrict__ slot_ids,
                                                          const int* __restrict__ token_req, int width,
                                                          int packed_kblocks) {
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* xr = x + (size_t)r * ldx;
  const float* prev = xr;
  if (mu) {
    const int req = token_req[r];
    const bool first = r == 0 || token_req[r - 1] != req;  // a request's rows are consecutive
    prev = first ? state + (size_t)slot_ids[req] * state_stride : xr - ldx;
  }
  float4 v[NV], pv[NV], m[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = min((tid + 256 * i) * 4, width - 4);
    v[i] = *(const float4*)(xr + k);
    if (mu) pv[i] = *(const float4*)(prev + k), m[i] = *(const float4*)(mu + k);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = (tid + 256 * i) * 4;
    if (k >= width) continue;
    float o[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    if (mu) {
      o[0] += (pv[i].x - v[i].x) * m[i].x, o[1] += (pv[i].y - v[i].y) * m[i].y;
      o[2] += (pv[i].z - v[i].z) * m[i].z, o[3] += (pv[i].w - v[i].w) * m[i].w;
    }
    // (packed_kblocks > 0: the order of packed_at, in which four columns from a multiple of four on stay together)
    T* at = out + (packed_kblocks > 0 ? packed_at(r, k, packed_kblocks) : (size_t)r * width + k);
#pragma unroll
    for (int c = 0; c < 4; ++c) at[c] = from_f32<T>(o[c]);
  }
}

// y: the sublayer's output rows (null: nothing but the parts); parts: n_parts partial products
// [n_parts][n_rows][width] that still have to be added up (a product that split its inner size).
template <typename T, int NV>
__global__ __launch_bounds__(256) void residual_rmsnorm_kernel(float* __restrict__ h, int ldh,
                                                               const float* __restrict__ y, int ldy,
                                                               const float* __restrict__ parts, int n_parts,
                                                               float alpha, const float* __restrict__ s,
                                                               const float* __restrict__ gamma, float eps,
                                                               float* __restrict__ state, size_t state_stride,
                                                               const int* __restrict__ slot_ids,
                                                               const int* __restrict__ token_req,
                                                               T* __restrict__ copy, int n_rows, int width,
                                                               int packed_kblocks) {
  __shared__ float red[32];
  const int r = blockIdx.x, tid = threadIdx.x;
  float* hr = h + (size_t)r * ldh;
  float* keep = nullptr;
  if (state) {
    const int req = token_req[r];
    if (r == n_rows - 1 || token_req[r + 1] != req) keep = state + (size_t)slot_ids[req] * state_stride;
  }
  float4 old[NV], out[NV], sc[NV], g[NV];
  const size_t part_step = (size_t)n_rows * width;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = min((tid + 256 * i) * 4, width - 4);
    old[i] = *(const float4*)(hr + k);
    out[i] = y ? *(const float4*)(y + (size_t)r * ldy + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    sc[i] = s ? *(const float4*)(s + k) : make_float4(1.f, 1.f, 1.f, 1.f);
    g[i] = gamma ? *(const float4*)(gamma + k) : make_float4(1.f, 1.f, 1.f, 1.f);
    const float* pr = parts + (size_t)r * width + k;
    for (int p0 = 0; p0 < n_parts; p0 += 4) {  // four parts' loads at a time, added in their order
      float4 t[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) t[j] = *(const float4*)(pr + min(p0 + j, n_parts - 1) * part_step);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (p0 + j < n_parts) out[i].x += t[j].x, out[i].y += t[j].y, out[i].z += t[j].z, out[i].w += t[j].w;
    }
  }
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = (tid + 256 * i) * 4;
    out[i].x = alpha * old[i].x + sc[i].x * out[i].x, out[i].y = alpha * old[i].y + sc[i].y * out[i].y;
    out[i].z = alpha * old[i].z + sc[i].z * out[i].z, out[i].w = alpha * old[i].w + sc[i].w * out[i].w;
    if (k < width) q += (out[i].x * out[i].x + out[i].y * out[i].y) + (out[i].z * out[i].z + out[i].w * out[i].w);
  }
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = (tid + 256 * i) * 4;
    if (k >= width) continue;
    if (keep) *(float4*)(keep + k) = old[i];
    const float4 n = make_float4(out[i].x * rstd * g[i].x, out[i].y * rstd * g[i].y, out[i].z * rstd * g[i].z,
                                 out[i].w * rstd * g[i].w);
    *(float4*)(hr + k) = n;
    if (copy) {
      T* at = copy + (packed_kblocks > 0 ? packed_at(r, k, packed_kblocks) : (size_t)r * width + k);
      at[0] = from_f32<T>(n.x), at[1] = from_f32<T>(n.y), at[2] = from_f32<T>(n.z), at[3] = from_f32<T>(n.w);
    }
  }
}

// The same two for any width and alignment: a wave a row, a column a lane at a time.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_any_kernel(T* __restrict__ out, const float* __restrict__ x, int ldx,
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
  const bool first = r == 0 || token_req[r - 1] != req;
  const float* prev = first ? state + (size_t)slot_ids[req] * state_stride : xr - ldx;
  for (int k = lane; k < width; k += 64) {
    const float v = xr[k];
    o[k] = from_f32<T>(v + (prev[k] - v) * mu[k]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void residual_rmsnorm_any_kernel(float* __restrict__ h, int ldh,
                                                                   const float* __restrict__ y, int ldy,
                                                                   const float* __restrict__ parts, int n_parts,
                                                                   float alpha, const float* __restrict__ s,
                                                                   const float* __restrict__ gamma, float eps,
                                                                   float* __restrict__ state, size_t state_stride,
                                                                   const int* __restrict__ slot_ids,
                                                                   const int* __restrict__ token_req,
                                                                   T* __restrict__ copy, int n_rows, int width) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  float* hr = h + (size_t)r * ldh;
  float* keep = nullptr;
  if (state) {
    const int req = token_req[r];
    if (r == n_rows - 1 || token_req[r + 1] != req) keep = state + (size_t)slot_ids[req] * state_stride;
  }
  const size_t part_step = (size_t)n_rows * width;
  auto sum_at = [&](int k) {
    float v = y ? y[(size_t)r * ldy + k] : 0.f;
    for (int p = 0; p < n_parts; ++p) v += parts[p * part_step + (size_t)r * width + k];
    return alpha * hr[k] + (s ? s[k] : 1.f) * v;
  };
  float q = 0.f;
  for (int k = lane; k < width; k += 64) {
    if (keep) keep[k] = hr[k];
    const float v = sum_at(k);
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
  for (int k = lane; k < width; k += 64) {
    const float n = sum_at(k) * rstd * (gamma ? gamma[k] : 1.f);
    hr[k] = n;
    if (copy) copy[(size_t)r * width + k] = from_f32<T>(n);
  }
}

__global__ void zero_rows_kernel(float* p, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

DEFINE_LAST_ERROR(mlxlm_last_error)

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// NV float4 a thread cover `width` columns with 256 threads; 0: too wide for the registers
static inline int vectors_for(int width) {
  const int nv = (width / 4 + 255) / 256;
  return nv <= 1 ? 1 : nv <= 2 ? 2 : nv <= 4 ? 4 : nv <= 8 ? 8 : 0;
}

#define BY_VECTORS(nv, LAUNCH) \
  do {                         \
    if (nv == 1) LAUNCH(1);    \
    else if (nv == 2) LAUNCH(2); \
    else if (nv == 4) LAUNCH(4); \
    else LAUNCH(8);            \
  } while (0)

// Whether the kernels that hold a row in registers take this width (they alone write the packed order).
extern "C" int post_norm_rows_in_registers(int width) { return width % 4 == 0 && vectors_for(width) > 0; }

// out [n_rows, width] (out_dtype) = shift(x); mu null: a conversion.  state [slots, state_stride] float32.
// out_packed: a bfloat16 out in tiles of 16 rows x 64 columns, the order of packed_at (common.h).
extern "C" int token_shift(void* out, const float* x, int ldx, const float* mu, const float* state,
                           size_t state_stride, const int* slot_ids, const int* token_req, int n_rows, int width,
                           int out_dtype, int out_packed, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const int kblocks = out_packed ? (width + 63) / 64 : 0;
  if (width <= 0 || ldx < width) FAIL("token_shift: width %d, row stride %d", width, ldx);
  if (!out || !x) FAIL("token_shift: null pointer");
  if (mu && (!state || !slot_ids || !token_req || state_stride < (size_t)width))
    FAIL("token_shift: the shift needs the state tensor (rows of %d), slot ids and token_req", width);
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("token_shift: unknown dtype code %d", out_dtype);
  const int nv = vectors_for(width);
  const bool vec = nv > 0 && width % 4 == 0 && ldx % 4 == 0 && state_stride % 4 == 0 && aligned16(x) && aligned16(mu) &&
                   aligned16(state);
  if (out_packed && (!vec || out_dtype != DT_BF16)) FAIL("token_shift: the packed order is for bfloat16 rows that fit the registers");
  if (vec) {
#define LAUNCH(NV)                                                                                                     \
  if (out_dtype == DT_F32)                                                                                             \
    hipLaunchKernelGGL((token_shift_kernel<float, NV>), dim3(n_rows), dim3(256), 0, stream, (float*)out, x, ldx, mu,  \
                       state, state_stride, slot_ids, token_req, width, 0);                                           \
  else                                                                                                                 \
    hipLaunchKernelGGL((token_shift_kernel<bf16, NV>), dim3(n_rows), dim3(256), 0, stream, (bf16*)out, x, ldx, mu,    \
                       state, state_stride, slot_ids, token_req, width, kblocks)
    BY_VECTORS(nv, LAUNCH);
#undef LAUNCH
  } else {
    dim3 grid((n_rows + 3) / 4), block(256);
    if (out_dtype == DT_F32)
      hipLaunchKernelGGL(token_shift_any_kernel<float>, grid, block, 0, stream, (float*)out, x, ldx, mu, state,
                         state_stride, slot_ids, token_req, n_rows, width);
    else
      hipLaunchKernelGGL(token_shift_any_kernel<bf16>, grid, block, 0, stream, (bf16*)out, x, ldx, mu, state,
                         state_stride, slot_ids, token_req, n_rows, width);
  }
  CHECK_LAUNCH("token_shift");
  return 0;
}

// h [n_rows, width] float32 (row stride ldh) <- N(alpha h + s * (y + the parts)) * gamma, in place.
// y: the sublayer's rows (null: none); parts: n_parts partial products [n_parts][n_rows][width] still
// to be added (null: none).  s, gamma: null = ones.  state non-null: the old row that ends each
// request's run of rows goes to the request's row of it.  copy non-null: the new rows once more,
// contiguous, in copy_dtype.
extern "C" int residual_rmsnorm(float* h, int ldh, const float* y, int ldy, const float* parts, int n_parts,
                                float alpha, const float* s, const float* gamma, float eps, float* state,
                                size_t state_stride, const int* slot_ids, const int* token_req, void* copy,
                                int copy_dtype, int copy_packed, int n_rows, int width, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const int kblocks = copy && copy_packed ? (width + 63) / 64 : 0;
  if (width <= 0 || ldh < width || (y && ldy < width)) FAIL("residual_rmsnorm: width %d, row strides %d and %d", width, ldh, ldy);
  if (!h || (!y && !parts)) FAIL("residual_rmsnorm: null pointer");
  if (!parts) n_parts = 0;
  if (n_parts < 0) FAIL("residual_rmsnorm: %d parts", n_parts);
  if (state && (!slot_ids || !token_req || state_stride < (size_t)width))
    FAIL("residual_rmsnorm: keeping rows needs slot ids, token_req and state rows of %d", width);
  if (copy && copy_dtype != DT_F32 && copy_dtype != DT_BF16) FAIL("residual_rmsnorm: unknown dtype code %d", copy_dtype);
  const bool half = copy && copy_dtype == DT_BF16;
  const int nv = vectors_for(width);
  const bool vec = nv > 0 && width % 4 == 0 && ldh % 4 == 0 && ldy % 4 == 0 && state_stride % 4 == 0 && aligned16(h) &&
                   aligned16(y) && aligned16(parts) && aligned16(s) && aligned16(gamma) && aligned16(state);
  if (kblocks && (!vec || !half)) FAIL("residual_rmsnorm: the packed order is for a bfloat16 copy of rows that fit the registers");
  if (vec) {
#define LAUNCH(NV)                                                                                                       \
  if (half)                                                                                                              \
    hipLaunchKernelGGL((residual_rmsnorm_kernel<bf16, NV>), dim3(n_rows), dim3(256), 0, stream, h, ldh, y, ldy, parts,   \
                       n_parts, alpha, s, gamma, eps, state, state_stride, slot_ids, token_req, (bf16*)copy, n_rows,    \
                       width, kblocks);                                                                                 \
  else                                                                                                                   \
    hipLaunchKernelGGL((residual_rmsnorm_kernel<float, NV>), dim3(n_rows), dim3(256), 0, stream, h, ldh, y, ldy, parts,  \
                       n_parts, alpha, s, gamma, eps, state, state_stride, slot_ids, token_req, (float*)copy, n_rows,   \
                       width, 0)
    BY_VECTORS(nv, LAUNCH);
#undef LAUNCH
  } else {
    dim3 grid((n_rows + 3) / 4), block(256);
    if (half)
      hipLaunchKernelGGL(residual_rmsnorm_any_kernel<bf16>, grid, block, 0, stream, h, ldh, y, ldy, parts, n_parts, alpha,
                         s, gamma, eps, state, state_stride, slot_ids, token_req, (bf16*)copy, n_rows, width);
    else
      hipLaunchKernelGGL(residual_rmsnorm_any_kernel<float>, grid, block, 0, stream, h, ldh, y, ldy, parts, n_parts, alpha,
                         s, gamma, eps, state, state_stride, slot_ids, token_req, (float*)copy, n_rows, width);
  }
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

  // What the sum-and-norm reads for a sublayer's output: its rows, or (and) parts still pending on them.
  struct Parts {
    const float* y;
    const float* ws;
    int n;
  };
  int take_parts(EngCtx* ctx, const EngMat& y, bool y_holds_rows, Parts* out) {
    EngPending* p = &ctx->pending;
    out->y = (const float*)y.p, out->ws = nullptr, out->n = 0;
    if (!p->target) return 0;
    if ((void*)p->target != y.p || p->rows != y.rows || p->cols != y.cols || p->ld != y.cols || p->bias)
      return host->settle(ctx, p);  // (a sum of another shape: added the plain way)
    out->ws = p->ws, out->n = p->n_splits;
    if (!y_holds_rows) out->y = nullptr;  // (a product that writes left nothing but its parts)
    p->target = nullptr;
    return 0;
  }

  // Whether the product of n_rows rows with w reads its rows faster in the packed order (the
  // host's answer), and the rows' own kernels here can write it.
  typedef int (*fn_wants_packed)(const EngCtx*, const EngWeight*, int);
  fn_wants_packed host_wants_packed = nullptr;
  bool wants_packed(EngCtx* ctx, int n_rows, const EngWeight* w) {
    if (!w || ctx->dtype != DT_BF16 || !post_norm_rows_in_registers(width)) return false;
    if (!host_wants_packed) host_wants_packed = (fn_wants_packed)host->kernel("engine", "eng_wants_packed_rows");
    return host_wants_packed && host_wants_packed(ctx, w, n_rows) != 0;
  }
  // Rows of the compute dtype for a product: row-major, or whole tiles of 16 rows x 64 columns.
  int take_rows(EngCtx* ctx, int n_rows, bool packed, EngValue* out) {
    if (!packed) return host->take(ctx, n_rows, width, ctx->dtype, &out->m);
    if (host->take(ctx, (n_rows + 15) / 16 * 16, (width + 63) / 64 * 64, DT_BF16, &out->m)) return 1;
    out->m.rows = n_rows, out->m.cols = width, out->m.ld = 0, out->packed = 1;
    return 0;
  }

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
      // (in the packed order where the mixer's first product reads its rows faster so)
      const bool pack = mixer->accepts_packed && wants_packed(ctx, T, mixer->first_weight);
      if (take_rows(ctx, T, pack, &u)) return 1;
      if (token_shift(u.m.p, (const float*)h.p, h.ld, mu, state, state_stride, ctx->slot_ids, ctx->token_req, T, width,
                      ctx->dtype, pack ? 1 : 0, ctx->stream))
        return host->fail("%s", g_err);
      host->launched(ctx);
    } else {
      u.m = h;
    }
    EngMat y;
    if (host->take(ctx, T, width, DT_F32, &y)) return 1;
    // A sublayer's last product may split its inner size and leave the parts where they are
    // (EngPending.allowed == 2: also a product that writes, not adds): the sum-and-norm adds them up.
    EngPending* pending = &ctx->pending;
    if (host->settle(ctx, pending)) return 1;
    pending->allowed = 2;
    if (!mixer->overwrite && zero(ctx, y)) return 1;
    int rc = mixer->forward(ctx, u, y, slot, writes);
    pending->allowed = 0;
    if (rc) return rc;
    Parts parts;
    if (take_parts(ctx, y, !mixer->overwrite, &parts)) return 1;
    // the first sum and norm; the rows that end a portion are kept for the next step's shift; the
    // feed-forward's product reads a copy in the compute dtype
    EngValue x = {};
    x.m = h;
    if (ffn && ctx->dtype != DT_F32) {
      if (take_rows(ctx, T, ffn->accepts_packed && wants_packed(ctx, T, ffn->first_weight), &x)) return 1;
    }
    if (residual_rmsnorm((float*)h.p, h.ld, parts.y, y.ld, parts.ws, parts.n, alpha, scale1, gamma1, eps, state,
                         state_stride, ctx->slot_ids, ctx->token_req, x.m.p != h.p ? x.m.p : nullptr, ctx->dtype, x.packed, T,
                         width, ctx->stream))
      return host->fail("%s", g_err);
    host->launched(ctx);
    if (ffn) {
      pending->allowed = 2;
      if (!ffn->overwrite && zero(ctx, y)) return 1;
      rc = ffn->forward(ctx, x, y);
      pending->allowed = 0;
      if (rc) return rc;
      if (take_parts(ctx, y, !ffn->overwrite, &parts)) return 1;
      if (residual_rmsnorm((float*)h.p, h.ld, parts.y, y.ld, parts.ws, parts.n, alpha, scale2, gamma2, eps, nullptr, 0,
                           nullptr, nullptr, nullptr, 0, 0, T, width, ctx->stream))
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
