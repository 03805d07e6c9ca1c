"""Plain, slow Pafutar: whole sequences, no cache, one function for each mechanism.

Written from the design's equations, in float64 on the CPU unless asked otherwise.  It shares
no code with the engine: tests import the engine on one side and this file on the other.

The design, for a sequence of tokens ``t_0 .. t_{n-1}`` at positions ``0 .. n-1``:

    x_p      = embed[t_p] * s_e + pos[p]
    layer:     u = shift(x);  x = N1(a x + ls1 * mixer(u));  x = N2(a x + ls2 * ff(x))
    shift:     u_p = x_p + (x_{p-1} - x_p) * mu,  x_{-1} = 0
    N(x)     = x / sqrt(mean(x^2) + eps) * w
    mixer:     q = Wq u + bq, k = Wk u + bk, v = k;  q, k <- unit RMS over a head
               s_ij = (q_i . k_j) * c * temp_h - 2^(-8(h+1)/H) * (i - j)
               j visible from i  <=>  j <= i and (i - j < W or j < F)
               o = softmax(s) v;  out = Wo (o * sigmoid(Wg u))
    ff:        Wd relu(Wu x)^2
    logits   = head N(x)

Weights are a dict of torch tensors under the checkpoint's names (``l<i>.mix.q`` and so on,
linear weights ``[out, in]``).  A layer with ``weights_of: j`` reads layer ``j``'s tensors.
"""

import torch


def embed(weights, tokens, scale, offset=0):
    """Token rows times ``scale`` plus the position rows (not scaled)."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(ids)) + offset
    return weights["embed"].index_select(0, ids) * scale + weights["pos"].index_select(0, pos)


def rms_norm(x, w, eps):
    """``x / sqrt(mean(x^2) + eps) * w`` over the last axis; ``w=None``: no weight."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def token_shift(x, mu, before=None):
    """``x_p + (x_{p-1} - x_p) * mu``; the row before the first is ``before`` (zeros if none)."""
    first = torch.zeros_like(x[:1]) if before is None else before.reshape(1, -1)
    prev = torch.cat([first, x[:-1]], dim=0)
    return x + (prev - x) * mu


def visible(n_q, offset, window, keep_first):
    """Boolean ``[n_q, offset + n_q]``: query at position ``offset + a`` sees key ``j``."""
    i = (torch.arange(n_q) + offset).unsqueeze(1)
    j = torch.arange(offset + n_q).unsqueeze(0)
    return (j <= i) & ((i - j < window) | (j < keep_first))


def head_slopes(n_heads, dtype=torch.float64):
    """``2^(-8 (h+1) / H)`` for head ``h``."""
    h = torch.arange(1, n_heads + 1, dtype=dtype)
    return torch.pow(torch.tensor(2.0, dtype=dtype), -8.0 * h / n_heads)


def attention_scores(q, k, scale, temp, offset=0):
    """``[H, n_q, n_k]`` scores of unit-RMS queries ``[n_q, H, d]`` and keys ``[n_k, G, d]``:
    dot product times ``scale`` times the head's temperature, minus slope times distance."""
    H, G = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)  # query head h reads key head h // (H / G)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale * temp.reshape(H, 1, 1)
    i = (torch.arange(q.shape[0]) + offset).reshape(1, -1, 1)
    j = torch.arange(k.shape[0]).reshape(1, 1, -1)
    return s - head_slopes(H, q.dtype).reshape(H, 1, 1) * (i - j)


def attention(u, w, prefix, mixer, eps):
    """The mixer on whole sequences: ``u`` is ``[n, width]``, the (shifted) input."""
    H, G, d = mixer["heads"], mixer["kv_heads"], mixer["dim"]
    n = u.shape[0]
    q = (u @ w[prefix + "q"].t() + w[prefix + "q.b"]).reshape(n, H, d)
    k = (u @ w[prefix + "k"].t() + w[prefix + "k.b"]).reshape(n, G, d)
    v = k  # the values are the keys as projected, before the norm
    qn, kn = rms_norm(q, None, eps), rms_norm(k, None, eps)
    s = attention_scores(qn, kn, mixer["scale"], w[prefix + "temp"].to(u.dtype))
    mask = mixer.get("mask") or {}
    see = visible(n, 0, mask.get("size", n + 1), mask.get("keep_first", 0))
    s = s.masked_fill(~see.unsqueeze(0), float("-inf"))
    p = torch.softmax(s, dim=-1)
    vv = v.repeat_interleave(H // G, dim=1)
    o = torch.einsum("hij,jhd->ihd", p, vv).reshape(n, H * d)
    gate = torch.sigmoid(u @ w[prefix + "g"].t())
    return (o * gate) @ w[prefix + "o"].t()


def relu_squared_ff(x, w, prefix):
    """``Wd relu(Wu x)^2``."""
    a = torch.relu(x @ w[prefix + "up"].t())
    return (a * a) @ w[prefix + "down"].t()


def layer(x, w, config, index):
    """One layer run; returns the stream after it."""
    entry = config["layers"][index]
    src = index
    while config["layers"][src].get("weights_of") is not None:  # (a run may name a run that names a layer)
        src = config["layers"][src]["weights_of"]
    p = f"l{src}."
    eps, alpha = config["norm"]["eps"], config["postln_alpha"]
    if entry["type"] != "attention":
        raise ValueError(f"unknown mixer type {entry['type']!r}")
    u = token_shift(x, w[p + "shift"])
    x = rms_norm(alpha * x + w[p + "ls1"] * attention(u, w, p + "mix.", entry["mixer"], eps), w[p + "norm1"], eps)
    if entry.get("mlp") is not None:
        if entry["mlp"]["kind"] != "dense":
            raise ValueError(f"unknown feed-forward kind {entry['mlp']['kind']!r}")
        x = rms_norm(alpha * x + w[p + "ls2"] * relu_squared_ff(x, w, p + "mlp."), w[p + "norm2"], eps)
    return x


def forward(weights, config, tokens, dtype=torch.float64, streams=None):
    """Logits ``[n, vocab]`` at every position of one sequence.  ``streams``: a list that gets
    the residual stream after every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    x = embed(w, tokens, config["embedding"]["scale"])
    for i in range(len(config["layers"])):
        x = layer(x, w, config, i)
        if streams is not None:
            streams.append(x.clone())
    x = rms_norm(x, w["final.norm"], config["norm"]["eps"])
    return x @ w["head"].t()


# -- random weights for tests ------------------------------------------------------


def random_weights(config, seed, sharp=1.0):
    """Seeded float32 tensors under the checkpoint's names, every vector drawn (so that none is
    0 or 1 by accident).  ``sharp`` scales the temperatures, which peaks the attention."""
    g = torch.Generator().manual_seed(int(seed))
    D, V = config["width"], config["vocab"]

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=g, dtype=torch.float32) * std + mean

    t = {"embed": normal((V, D), 0.05), "pos": normal((config["max_positions"], D), 0.3)}
    for i, entry in enumerate(config["layers"]):
        if entry.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", entry["mixer"]
        qw, kw = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
        t[p + "norm1"] = normal((D,), 0.2, 1.0)
        t[p + "mix.q"], t[p + "mix.q.b"] = normal((qw, D), D**-0.5), normal((qw,), 0.3)
        t[p + "mix.k"], t[p + "mix.k.b"] = normal((kw, D), D**-0.5), normal((kw,), 0.3)
        t[p + "mix.temp"] = (normal((m["heads"],), 0.2, 1.0).abs() + 0.3) * sharp
        t[p + "mix.g"] = normal((qw, D), D**-0.5)
        t[p + "mix.o"] = normal((D, qw), qw**-0.5)
        t[p + "ls1"] = normal((D,), 0.3, 1.0)
        t[p + "shift"] = torch.rand((D,), generator=g)
        if entry.get("mlp") is not None:
            F = entry["mlp"]["ff"]
            t[p + "norm2"] = normal((D,), 0.2, 1.0)
            t[p + "mlp.up"], t[p + "mlp.down"] = normal((F, D), D**-0.5), normal((D, F), F**-0.5)
            t[p + "ls2"] = normal((D,), 0.3, 1.0)
    t["final.norm"] = normal((D,), 0.2, 1.0)
    t["head"] = normal((V, D), D**-0.5)
    return t
