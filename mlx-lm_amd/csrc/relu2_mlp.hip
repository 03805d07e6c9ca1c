// A dense feed-forward with the square of the ReLU between its two products and no biases:
//   out = Wd relu(Wu x)^2
// The activation runs in the first product's epilogue; the second writes (or adds) 32-bit rows.
// No kernels of its own: the native part only.
#include "common.h"
#include "engine_parts.h"

static const EngHost* host = nullptr;

struct Relu2Mlp : FeedForward {
  int width, inner;
  EngWeight up_w, down_w;
  typedef int (*fn_wants_packed)(const EngCtx*, const EngWeight*, int);
  fn_wants_packed wants_packed = nullptr;
  Relu2Mlp() { can_overwrite = true, accepts_packed = true; }
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& y) override {
    const int M = x.m.rows;
    if (M == 0) return 0;
    // both products through the kernel for 17 to 64 rows: the first writes what the second reads in
    // the packed order (tiles of 16 rows x 64 columns)
    if (!wants_packed) wants_packed = (fn_wants_packed)host->kernel("engine", "eng_wants_packed_rows");
    const bool pack = ctx->dtype == DT_BF16 && wants_packed && wants_packed(ctx, &up_w, M) && wants_packed(ctx, &down_w, M);
    EngMat act;
    if (pack) {
      if (host->take(ctx, (M + 15) / 16 * 16, (inner + 63) / 64 * 64, DT_BF16, &act)) return 1;
      act.rows = M, act.cols = inner, act.ld = 0;
    } else if (host->take(ctx, M, inner, ctx->dtype, &act)) {
      return 1;
    }
    EngLinear up = {};
    up.out = act, up.a = x, up.w = up_w, up.gelu = 2;  // (activation code 2: the squared ReLU)
    up.out_packed = pack ? 1 : 0;
    if (host->linear(ctx, &up, nullptr)) return 1;  // (nothing of this product may stay pending)
    EngLinear down = {};
    down.out = y, down.a.m = act, down.a.packed = pack ? 1 : 0, down.w = down_w, down.accumulate = overwrite ? 0 : 1;
    return host->linear(ctx, &down, &ctx->pending);
  }
};

extern "C" EngPart* make_relu2_mlp(const EngHost* h, int width, int inner_padded, const EngWeight* up_w,
                                   const EngWeight* down_w) {
  host = h;
  Relu2Mlp* m = new Relu2Mlp();
  m->width = width, m->inner = inner_padded, m->up_w = *up_w, m->down_w = *down_w;
  m->first_weight = &m->up_w;
  return m;
}
