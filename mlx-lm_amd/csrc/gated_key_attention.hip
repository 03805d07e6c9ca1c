// Attention whose values are its keys, with unit-RMS queries and keys, a temperature per head,
// a bias that grows with distance, a sliding window that keeps the first keys, and an output gate:
//   q = Wq u + bq,  k = Wk u + bk,  v = k                       (no value projection)
//   q^, k^ = q, k divided by their root mean square over a head (eps inside the root)
//   s_ij   = (q^_i . k^_j) * c_h - m_h (i - j)                  c_h = scale * temperature_h
//   j is seen from i  <=>  j <= i and (i - j < window or j < keep_first)
//   out    = Wo (softmax(s) v * sigmoid(Wg u))
// One product gives q, k and the gate's input side by side.  `qk_prepare` norms the queries in
// place and puts each token's normed keys into the key half of its page and the keys as projected
// into the value half; the attention kernels (attention.hip, with the optional score terms) do the
// rest, the gate in their epilogue.  Norms, scores and softmax are computed in 32-bit.
#include "common.h"
#include "engine_parts.h"
#include "attention_tiles.h"

// grid (n_tokens, ceil((n_heads + n_kv_heads) / 4)), 256 threads: a wave a head (the query heads,
// then the key heads), its columns in registers (up to four a lane: head sizes to 256), so that a
// head costs one trip to memory
template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(T* __restrict__ qk, int ld, int n_heads, int n_kv_heads,
                                                         int head_dim, float eps, T* __restrict__ k_pages,
                                                         T* __restrict__ v_pages, size_t page_stride,
                                                         const int* __restrict__ block_table, int max_blocks,
                                                         const int* __restrict__ token_req,
                                                         const int* __restrict__ positions, int page_size) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int u = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (u >= n_heads + n_kv_heads) return;  // (whole waves; no barrier follows)
  T* v = qk + (size_t)t * ld + (size_t)u * head_dim;  // (the keys' columns follow the queries')
  T raw[4];
  float f[4], q = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    raw[i] = v[min(d, head_dim - 1)];
    f[i] = d < head_dim ? to_f32(raw[i]) : 0.f;
    q += f[i] * f[i];
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)head_dim + eps);
  if (u < n_heads) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (lane + 64 * i < head_dim) v[lane + 64 * i] = from_f32<T>(f[i] * rstd);
  } else if (k_pages) {
    const int pos = positions[t];
    const int page = block_table[(size_t)token_req[t] * max_blocks + pos / page_size];
    const size_t dst = (size_t)page * page_stride + ((size_t)(u - n_heads) * page_size + pos % page_size) * head_dim;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < head_dim) v_pages[dst + d] = raw[i], k_pages[dst + d] = from_f32<T>(f[i] * rstd);
    }
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

// qk [n_tokens, >= (n_heads + n_kv_heads) * head_dim] (row stride ld): queries then keys as projected.
// k_pages null: only the queries are normed (a run that reads a cache another run wrote).
extern "C" int qk_prepare(void* qk, int ld, int n_tokens, int n_heads, int n_kv_heads, int head_dim, float eps,
                          void* k_pages, void* v_pages, size_t page_stride, const int* block_table, int max_blocks,
                          const int* token_req, const int* positions, int page_size, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!qk || n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || head_dim > 256 || ld < (n_heads + n_kv_heads) * head_dim)
    FAIL("qk_prepare: %d + %d heads of %d in rows of stride %d", n_heads, n_kv_heads, head_dim, ld);
  if (k_pages && (!v_pages || !block_table || !token_req || !positions || page_size <= 0 ||
                  page_stride < (size_t)n_kv_heads * page_size * head_dim))
    FAIL("qk_prepare: the cache write needs pages, block table, token_req and positions");
  dim3 grid(n_tokens, (n_heads + n_kv_heads + 3) / 4), block(256);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(qk_prepare_kernel<float>, grid, block, 0, stream, (float*)qk, ld, n_heads, n_kv_heads, head_dim, eps,
                       (float*)k_pages, (float*)v_pages, page_stride, block_table, max_blocks, token_req, positions, page_size);
  else if (dtype == DT_BF16)
    hipLaunchKernelGGL(qk_prepare_kernel<bf16>, grid, block, 0, stream, (bf16*)qk, ld, n_heads, n_kv_heads, head_dim, eps,
                       (bf16*)k_pages, (bf16*)v_pages, page_stride, block_table, max_blocks, token_req, positions, page_size);
  else
    FAIL("qk_prepare: unknown dtype code %d", dtype);
  CHECK_LAUNCH("qk_prepare");
  return 0;
}

// ---------------------------------------------------------------------------
// the mixer

static const EngHost* host = nullptr;

typedef int (*fn_attn_tile_biased)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                                   const int*, const int*, const int*, int, int, int, int, int, int, float, int,
                                   const float*, const float*, const void*, int, int, hipStream_t);
typedef int (*fn_attn_row_biased)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                                  const int*, const int*, const int*, int, int, int, int, int, int, float, int, float*,
                                  float*, int, const float*, const float*, const void*, int, int, hipStream_t);
typedef int (*fn_attn_prefill_biased)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                                      const int*, const int*, const int*, int, int, int, int, int, int, float,
                                      const float*, const float*, const void*, int, int, hipStream_t);
typedef int (*fn_attn_decode_biased)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                                     const int*, const int*, const int*, int, int, int, int, int, int, float, int,
                                     float*, float*, int, const void*, size_t, int, int, int, int, int, const float*,
                                     const float*, const void*, int, int, hipStream_t);
typedef const char* (*fn_error)();
#define ROW_KERNEL_MAX_HEAD_DIM 144  // beyond it the tile kernel takes single rows too

// the attention part's step arrays, from `array_base` on (parts/attention.py)
enum { ARR_TILES = 0, ARR_ROWS, ARR_ALL_TILES, ARR_BIG_TILES, ARR_MAX_ROW_CONTEXT, ARR_ROWS_ARE_REQUESTS };

struct GatedKeyAttention : Mixer {
  int width, n_heads, n_kv_heads, head_dim, window, keep_first, q_width, kv_width, array_base;
  float eps;
  EngWeight qkg_w, out_w;
  const float* qkg_b;       // [2 q_width + kv_width]: the queries' and keys' biases, zeros for the gate
  const float* head_scale;  // [n_heads]: scale * temperature
  const float* slopes;      // [n_heads]
  fn_attn_tile_biased attn_tile = nullptr;
  fn_attn_row_biased attn_row = nullptr;
  fn_attn_prefill_biased attn_prefill = nullptr;
  fn_attn_decode_biased attn_decode = nullptr;
  fn_error attn_error = nullptr, prefill_error = nullptr, decode_error = nullptr;

  typedef int (*fn_wants_packed)(const EngCtx*, const EngWeight*, int);
  fn_wants_packed wants_packed = nullptr;

  GatedKeyAttention() { can_overwrite = true, accepts_packed = true; }

  int kernels() {
    if (!attn_tile) {
      attn_tile = (fn_attn_tile_biased)host->kernel("attention", "attn_tile_biased");
      attn_row = (fn_attn_row_biased)host->kernel("attention", "attn_row_biased");
      attn_error = (fn_error)host->kernel("attention", "mlxlm_last_error");
      if (!attn_tile || !attn_row || !attn_error) {
        attn_tile = nullptr;
        return host->fail("gated key attention: the 'attention' kernels are not loaded");
      }
    }
    return 0;
  }
  // (the kernels for the head sizes that the matrix cores and the register-streaming rows take
  // are in libraries of their own, looked up only where a model has such heads)
  int prefill_kernel() {
    if (!attn_prefill) {
      attn_prefill = (fn_attn_prefill_biased)host->kernel("attention_prefill", "attn_prefill_biased");
      prefill_error = (fn_error)host->kernel("attention_prefill", "mlxlm_last_error");
      if (!attn_prefill || !prefill_error) return host->fail("gated key attention: the 'attention_prefill' kernels are not loaded");
    }
    return 0;
  }
  int decode_kernel() {
    if (!attn_decode) {
      attn_decode = (fn_attn_decode_biased)host->kernel("attention_decode", "attn_decode_rows_biased");
      decode_error = (fn_error)host->kernel("attention_decode", "mlxlm_last_error");
      if (!attn_decode || !decode_error) return host->fail("gated key attention: the 'attention_decode' kernels are not loaded");
    }
    return 0;
  }

  // In how many parts a row's keys go, so that the row kernel's launch fills the GPU.
  int row_splits(const EngCtx* ctx, int n_rows, long longest) const {
    long c = longest;
    if (window > 0 && c > window + keep_first + 126) c = window + keep_first + 126;
    long most = (c + 255) / 256;
    if (most < 1) most = 1;
    const long blocks = n_rows * n_heads < 1 ? 1 : (long)n_rows * n_heads;
    long want = (2L * ctx->n_compute_units + blocks - 1) / blocks;
    if (want > most) want = most;
    if (want > 64) want = 64;
    return want < 1 ? 1 : (int)want;
  }

  int forward(EngCtx* ctx, const EngValue& x, const EngMat& y, int slot, bool writes) override {
    if (kernels()) return 1;
    const int T = x.m.rows;
    if (T == 0) return 0;
    EngScatter kv;
    if (host->slot_pages(ctx, slot, q_width, kv_width, &kv)) return 1;
    if (kv.n_kv_heads != n_kv_heads || kv.head_dim != head_dim)
      return host->fail("gated key attention: cache slot %d holds %d heads of %d, the mixer has %d of %d", slot,
                        kv.n_kv_heads, kv.head_dim, n_kv_heads, head_dim);
    if (kv.dtype != ctx->dtype) return host->fail("gated key attention: the cache's dtype differs from the step's");
    // queries, keys and the gate's input from one product
    EngMat qkg;
    if (host->take(ctx, T, 2 * q_width + kv_width, ctx->dtype, &qkg)) return 1;
    EngLinear call = {};
    call.out = qkg, call.a = x, call.w = qkg_w, call.bias = qkg_b;
    if (host->linear(ctx, &call, nullptr)) return 1;  // (nothing of this product may stay pending)
    if (qk_prepare(qkg.p, qkg.ld, T, n_heads, n_kv_heads, head_dim, eps, writes ? kv.k : nullptr, kv.v, kv.page_stride,
                   kv.block_table, kv.max_blocks, kv.token_req, kv.positions, kv.page_size, ctx->dtype, ctx->stream))
      return host->fail("%s", g_err);
    host->launched(ctx);

    const int n_tiles_ = (int)ctx->counts[array_base + ARR_TILES] / 2;
    const int n_rows_ = (int)ctx->counts[array_base + ARR_ROWS];
    const int key_bytes_ = head_dim * (ctx->dtype == DT_BF16 ? 2 : 4);
    // Where every row goes to the kernel that streams keys through registers, that kernel writes
    // the packed order (tiles of 16 rows x 64 columns) if the output product reads it faster so.
    if (!wants_packed) wants_packed = (fn_wants_packed)host->kernel("engine", "eng_wants_packed_rows");
    const bool pack = ctx->dtype == DT_BF16 && n_tiles_ == 0 && n_rows_ == T && head_dim <= ROW_KERNEL_MAX_HEAD_DIM &&
                      (key_bytes_ == 64 || key_bytes_ == 128 || key_bytes_ == 256) && kv.page_size % (1024 / key_bytes_) == 0 &&
                      wants_packed && wants_packed(ctx, &out_w, T);
    EngMat o;
    if (pack) {
      if (host->take(ctx, (T + 15) / 16 * 16, (q_width + 63) / 64 * 64, DT_BF16, &o)) return 1;
      o.rows = T, o.cols = q_width, o.ld = 0;
    } else if (host->take(ctx, T, q_width, ctx->dtype, &o)) {
      return 1;
    }
    const char* gate = (const char*)qkg.p + (size_t)(q_width + kv_width) * (ctx->dtype == DT_BF16 ? 2 : 4);
    const int* tiles = ctx->arrays[array_base + ARR_TILES];
    const int* rows = ctx->arrays[array_base + ARR_ROWS];
    const int* all_tiles = ctx->arrays[array_base + ARR_ALL_TILES];
    const int* big_tiles = ctx->arrays[array_base + ARR_BIG_TILES];
    const int n_tiles = (int)ctx->counts[array_base + ARR_TILES] / 2;
    const int n_rows = (int)ctx->counts[array_base + ARR_ROWS];
    const int n_all_tiles = (int)ctx->counts[array_base + ARR_ALL_TILES] / 2;
    const int n_big_tiles = (int)ctx->counts[array_base + ARR_BIG_TILES] / 2;
    const long longest = ctx->counts[array_base + ARR_MAX_ROW_CONTEXT];
    const int rows_are_requests = ctx->counts[array_base + ARR_ROWS_ARE_REQUESTS] != 0;
    if (n_tiles == 0 && n_rows == 0) return host->fail("gated key attention: the step carries no work lists for its %d rows", T);
    const bool bf16 = ctx->dtype == DT_BF16;
    // which kernel takes which rows: as the plain attention part chooses (tiles of 128 queries on
    // the matrix cores for bfloat16 heads of 32, 64 or 128; single rows through registers where a
    // key is 64, 128 or 256 bytes; the general tile and row kernels otherwise)
    if (head_dim > ROW_KERNEL_MAX_HEAD_DIM) {
      if (attn_tile(o.p, qkg.p, qkg.ld, o.ld, kv.k, kv.v, kv.page_stride, kv.block_table, kv.max_blocks, kv.token_req,
                    kv.positions, all_tiles, n_all_tiles, n_heads, n_kv_heads, head_dim, kv.page_size, window, 1.f,
                    ctx->dtype, head_scale, slopes, gate, qkg.ld, keep_first, ctx->stream))
        return host->fail("%s", attn_error());
      host->launched(ctx);
    } else {
      if (n_tiles && bf16 && (head_dim == 32 || head_dim == 64 || head_dim == 128)) {
        if (prefill_kernel()) return 1;
        if (attn_prefill(o.p, qkg.p, qkg.ld, o.ld, kv.k, kv.v, kv.page_stride, kv.block_table, kv.max_blocks,
                         kv.token_req, kv.positions, big_tiles, n_big_tiles, n_heads, n_kv_heads, head_dim, kv.page_size,
                         window, 1.f, head_scale, slopes, gate, qkg.ld, keep_first, ctx->stream))
          return host->fail("%s", prefill_error());
        host->launched(ctx);
      } else if (n_tiles) {
        if (attn_tile(o.p, qkg.p, qkg.ld, o.ld, kv.k, kv.v, kv.page_stride, kv.block_table, kv.max_blocks, kv.token_req,
                      kv.positions, tiles, n_tiles, n_heads, n_kv_heads, head_dim, kv.page_size, window, 1.f, ctx->dtype,
                      head_scale, slopes, gate, qkg.ld, keep_first, ctx->stream))
          return host->fail("%s", attn_error());
        host->launched(ctx);
      }
      if (n_rows) {
        const int key_bytes = head_dim * (bf16 ? 2 : 4);
        const bool fast = (key_bytes == 64 || key_bytes == 128 || key_bytes == 256) && kv.page_size % (1024 / key_bytes) == 0;
        int n_splits = 1, n_waves = 4, key_tile = 32;
        if (fast) {
          long keys = longest;
          if (window > 0 && keys > window + keep_first + 62) keys = window + keep_first + 62;
          attn_decode_row_work(ctx->n_compute_units, n_rows, n_heads, head_dim, keys, &n_splits, &n_waves, &key_tile);
        } else {
          n_splits = row_splits(ctx, n_rows, longest);
        }
        if (ctx->stats && n_splits > ctx->stats->key_splits_most) ctx->stats->key_splits_most = n_splits;
        EngMat part_o = {}, part_ml = {};
        if (n_splits > 1) {
          const long n = (long)n_rows * n_heads * n_splits;
          if (host->take(ctx, 1, (int)(n * head_dim), DT_F32, &part_o)) return 1;
          if (host->take(ctx, 1, (int)(n * 2), DT_F32, &part_ml)) return 1;
        }
        if (fast) {
          if (decode_kernel()) return 1;
          if (attn_decode(o.p, qkg.p, qkg.ld, o.ld, kv.k, kv.v, kv.page_stride, kv.block_table, kv.max_blocks, kv.token_req,
                          kv.positions, rows, n_rows, n_heads, n_kv_heads, head_dim, kv.page_size, window, 1.f, n_splits,
                          (float*)part_o.p, (float*)part_ml.p, n_waves, nullptr, 0, 0, rows_are_requests, ctx->dtype,
                          key_tile, 2, head_scale, slopes, gate, qkg.ld, keep_first, ctx->stream))
            return host->fail("%s", decode_error());
        } else {
          if (attn_row(o.p, qkg.p, qkg.ld, o.ld, kv.k, kv.v, kv.page_stride, kv.block_table, kv.max_blocks, kv.token_req,
                       kv.positions, rows, n_rows, n_heads, n_kv_heads, head_dim, kv.page_size, window, 1.f, n_splits,
                       (float*)part_o.p, (float*)part_ml.p, ctx->dtype, head_scale, slopes, gate, qkg.ld, keep_first,
                       ctx->stream))
            return host->fail("%s", attn_error());
        }
        host->launched(ctx);
      }
    }
    EngLinear out = {};
    out.out = y, out.a.m = o, out.a.packed = pack ? 1 : 0, out.w = out_w, out.accumulate = overwrite ? 0 : 1;
    return host->linear(ctx, &out, &ctx->pending);
  }
};

extern "C" EngPart* make_gated_key_attention(const EngHost* h, int width, int n_heads, int n_kv_heads, int head_dim,
                                             int window, int keep_first, float eps, const EngWeight* qkg_w,
                                             const float* qkg_b, const EngWeight* out_w, const float* head_scale,
                                             const float* slopes, int array_base) {
  host = h;
  if (array_base < 0 || array_base + ARR_ROWS_ARE_REQUESTS >= ENG_MAX_ARRAYS) {
    h->fail("make_gated_key_attention: array ids from %d do not fit", array_base);
    return nullptr;
  }
  GatedKeyAttention* a = new GatedKeyAttention();
  a->width = width, a->n_heads = n_heads, a->n_kv_heads = n_kv_heads, a->head_dim = head_dim;
  a->window = window, a->keep_first = keep_first, a->eps = eps;
  a->q_width = n_heads * head_dim, a->kv_width = n_kv_heads * head_dim;
  a->qkg_w = *qkg_w, a->out_w = *out_w, a->qkg_b = qkg_b, a->head_scale = head_scale, a->slopes = slopes;
  a->array_base = array_base;
  a->first_weight = &a->qkg_w;
  return a;
}
