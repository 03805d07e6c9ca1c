"""Ruzolorn, plainly: one function per mechanism, whole sequences, float64, no cache.

Written from the design's equations; shares no code with the engine.  A model is a dict of
tensors under the checkpoint's names and the parsed config.json.  For tokens ``t_p`` at positions
``p = 0, 1, ...`` of one sequence:

    x        = embed[t] * s_e
    layer:     x += m * LNb1(mixer(LN1(x)));  x += m * LNb2(ff(LN2(x)))      (ff may be absent)
    LN(x)    = (x - mean) / sqrt(var + eps) * w
    logits   = head LN_final(x)
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def rotate_half(x, positions, dims, base):
    """``x`` is ``[T, H, d]``; the first ``dims`` columns of a head turn, column ``i`` with
    column ``i + dims/2`` by the angle ``p * base^(-2i/dims)``."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = positions.to(F64)[:, None, None] * f[None, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * a.cos() - v * a.sin(), v * a.cos() + u * a.sin(), x[..., dims:]], -1)


def retention(h, t, p, m, eps):
    """Linear attention with one fixed decay a head, no softmax: ``S = g S + k v^T; o = S^T q``."""
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
    pos = torch.arange(T)
    q = (h @ t[p + "q"].T).view(T, H, d)
    k = (h @ t[p + "k"].T).view(T, H, d)
    v = (h @ t[p + "v"].T).view(T, H, dv)
    rot = m.get("rot")
    if rot:
        q, k = rotate_half(q, pos, rot["dims"], rot["base"]), rotate_half(k, pos, rot["dims"], rot["base"])
    k = k * d ** -0.5
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for i in range(T):
            S = m["decay"][hd] * S + torch.outer(k[i, hd], v[i, hd])
            out[i, hd] = S.T @ q[i, hd]
    out = unit_rms(out, eps).reshape(T, H * dv)
    return (out * silu(h @ t[p + "g"].T)) @ t[p + "o"].T


def window_mask(T, size):
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return (i - j >= 0) & ((i - j < size) if size else (i >= j))


def window_attention(h, t, p, m, eps):
    """Softmax attention over the last ``mask.size`` tokens, grouped key heads, RMS-normed queries and
    keys with a weight shared by the heads, values of their own width, no positions."""
    T, H, G, d, dv = h.shape[0], m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = unit_rms((h @ t[p + "q"].T).view(T, H, d), eps) * t[p + "q.norm"]
    k = unit_rms((h @ t[p + "k"].T).view(T, G, d), eps) * t[p + "k.norm"]
    v = (h @ t[p + "v"].T).view(T, G, dv)
    seen = window_mask(T, int((m.get("mask") or {}).get("size", 0)))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m.get("scale", d ** -0.5)
        s = s.masked_fill(~seen, -math.inf)
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(T, H * dv) @ t[p + "o"].T


def causal_conv(x, w, b):
    """``y[t, c] = b[c] + sum_j w[c, taps-1-j] x[t-j, c]``: the last column is the current token's."""
    T, taps = x.shape[0], w.shape[1]
    y = b.expand(T, -1).clone()
    for j in range(taps):
        y[j:] += x[: T - j] * w[:, taps - 1 - j]
    return y


def state_space(h, t, p, m, eps):
    """The selective state space with a scalar decay a head: ``S = exp(-exp(A) dt) S + dt B x^T``,
    ``y = S^T C + D x``, gated by ``silu(z)`` and then RMS-normed in equal parts."""
    T, H, dv, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * dv
    u = h @ t[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner : 2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N :]
    xbc = silu(causal_conv(xbc, t[p + "conv"], t[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner : inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N :].view(T, G, N)
    dt = softplus(dt + t[p + "dt_bias"])
    y = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, dv, dtype=F64)
        a = torch.exp(t[p + "A_log"][hd])
        for i in range(T):
            S = torch.exp(-a * dt[i, hd]) * S + dt[i, hd] * torch.outer(B[i, g], x[i, hd])
            y[i, hd] = S.T @ C[i, g] + t[p + "D"][hd] * x[i, hd]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * t[p + "norm"]
    return y @ t[p + "o"].T


def parallel(h, t, p, m, eps):
    left = window_attention(h, t, p + "left.", m["left"], eps)
    right = state_space(h, t, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def gated_expert(h, t, p):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def router_choice(h, t, p, r):
    """``(chosen experts [T, top], their weights [T, top])``: softmax over all router outputs; the
    choice adds the correction, the weights do not."""
    s = torch.softmax(h @ t[p + "router"].T, -1)
    choice = s + t[p + "correction"] if (p + "correction") in t else s
    idx = torch.topk(choice, r["top"], -1).indices
    return idx, torch.gather(s, 1, idx)


def mixture(h, t, p, mlp):
    r = mlp["router"]
    n_real = r["experts"]
    idx, w = router_choice(h, t, p, r)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, we in zip(idx[i].tolist(), w[i]):
            if e >= n_real:  # an identity expert gives its input back
                out[i] += we * h[i]
            else:
                out[i] += we * gated_expert(h[i : i + 1], t, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_expert(h, t, p + "shared.")
    return out


MIXERS = {"retention": retention, "parallel": parallel}


def layer(x, t, i, entry, cfg):
    eps, mult, p = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0), f"l{i}."
    y = MIXERS[entry["type"]](layer_norm(x, t[p + "norm1"], eps), t, p + "mix.", entry["mixer"], eps)
    x = x + mult * layer_norm(y, t[p + "norm1b"], eps)
    if entry.get("mlp") is not None:
        y = mixture(layer_norm(x, t[p + "norm2"], eps), t, p + "mlp.", entry["mlp"])
        x = x + mult * layer_norm(y, t[p + "norm2b"], eps)
    return x


def model(tensors, cfg, tokens, streams=None):
    """Logits ``[T, vocab]`` of one sequence; ``streams`` (a list) receives the stream after each layer."""
    t = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in tensors.items()}
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"].get("scale", 1.0)
    for i, entry in enumerate(cfg["layers"]):
        x = layer(x, t, i, entry, cfg)
        if streams is not None:
            streams.append(x)
    return layer_norm(x, t["final.norm"], cfg["norm"]["eps"]) @ t["head"].T


def random_weights(cfg, seed, sharp=1.0):
    """Float32 tensors under the checkpoint's names, every vector drawn (no ones, no zeros).
    ``sharp`` scales the attention's query and key weights, so that its softmax is peaked and a
    key on the wrong side of the window's edge shows."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=g) * std + mean

    t = {"embed": normal((cfg["vocab"], D), 1.0), "final.norm": normal((D,), 0.1, 1.0),
         "head": normal((cfg["vocab"], D), D ** -0.5)}
    for i, entry in enumerate(cfg["layers"]):
        p, m = f"l{i}.", entry["mixer"]
        t[p + "norm1"], t[p + "norm1b"] = normal((D,), 0.1, 1.0), normal((D,), 0.1, 1.0)
        if entry["type"] == "retention":
            H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
            for name, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                t[p + "mix." + name] = normal((n, D), D ** -0.5)
            t[p + "mix.o"] = normal((D, H * dv), (H * dv) ** -0.5)
        else:
            a, b = m["left"], m["right"]
            H, G, d, dv = a["heads"], a.get("kv_heads", a["heads"]), a["dim"], a.get("vdim", a["dim"])
            q = p + "mix.left."
            t[q + "q"], t[q + "k"] = normal((H * d, D), D ** -0.5) * sharp, normal((G * d, D), D ** -0.5) * sharp
            t[q + "v"], t[q + "o"] = normal((G * dv, D), D ** -0.5), normal((D, H * dv), (H * dv) ** -0.5)
            t[q + "q.norm"], t[q + "k.norm"] = normal((d,), 0.2, 1.0) * sharp, normal((d,), 0.2, 1.0) * sharp
            r = p + "mix.right."
            Hs, P, N, Gs, taps = b["heads"], b["vdim"], b["state"], b["groups"], b["conv"]
            inner, C = Hs * P, Hs * P + 2 * Gs * N
            t[r + "in"] = normal((2 * inner + 2 * Gs * N + Hs, D), D ** -0.5)
            t[r + "conv"], t[r + "conv.b"] = normal((C, taps), 0.5), normal((C,), 0.2)
            t[r + "dt_bias"], t[r + "A_log"] = normal((Hs,), 0.5), normal((Hs,), 0.5, -1.5)
            t[r + "D"], t[r + "norm"] = normal((Hs,), 0.3, 1.0), normal((inner,), 0.1, 1.0)
            t[r + "o"] = normal((D, inner), inner ** -0.5)
        mlp = entry.get("mlp")
        if mlp is not None:
            q, r = p + "mlp.", mlp["router"]
            t[p + "norm2"], t[p + "norm2b"] = normal((D,), 0.1, 1.0), normal((D,), 0.1, 1.0)
            F = (mlp.get("expert") or {}).get("ff", 0)
            for e in range(r["experts"]):
                t[f"{q}e{e}.gate"], t[f"{q}e{e}.up"] = normal((F, D), D ** -0.5), normal((F, D), D ** -0.5)
                t[f"{q}e{e}.down"] = normal((D, F), F ** -0.5)
            n_out = r["experts"] + r.get("identity", 0)
            t[q + "router"], t[q + "correction"] = normal((n_out, D), 1.5 * D ** -0.5), normal((n_out,), 0.05)
            Fs = (mlp.get("shared") or {}).get("ff", 0)
            if Fs:
                t[q + "shared.gate"], t[q + "shared.up"] = normal((Fs, D), D ** -0.5), normal((Fs, D), D ** -0.5)
                t[q + "shared.down"] = normal((D, Fs), Fs ** -0.5)
    return t
