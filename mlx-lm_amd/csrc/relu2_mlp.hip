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
  Relu2Mlp() { can_overwrite = true; }
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& y) override {
    const int M = x.m.rows;
    if (M == 0) return 0;
    EngMat act;
    if (host->take(ctx, M, inner, ctx->dtype, &act)) return 1;
    EngLinear up = {};
    up.out = act, up.a = x, up.w = up_w, up.gelu = 2;  // (activation code 2: the squared ReLU)
    if (host->linear(ctx, &up, nullptr)) return 1;  // (nothing of this product may stay pending)
    EngLinear down = {};
    down.out = y, down.a.m = act, down.w = down_w, down.accumulate = overwrite ? 0 : 1;
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
