"""Ruzolorn in the engine against the plain implementation (plain_ruzolorn.py): each mechanism's
kernels, whole prompts, decoding, portions, mixed batches, reused pages and state rows, the
window's edges, far tokens, generation through the entry points."""

import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_ruzolorn as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# max |engine - plain| over max |plain logits|: float32 sums where the plain side has float64;
# bfloat16 rounds activations between the products (the plain side gets the rounded matrices)
TOL = {"float32": 5e-5, "bfloat16": 5e-2}


def _retention(heads, dim, vdim, decay, rot_dims=None, base=10000.0):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    return {"type": "retention", "mixer": m}


def _parallel(heads, kv_heads, dim, vdim, window, s_heads, s_vdim, state, groups, taps, norm_groups, scale=None,
              left_scale=1.0, right_scale=1.0):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if window is not None:
        left["mask"] = {"size": window}
    right = {"heads": s_heads, "vdim": s_vdim, "state": state, "groups": groups, "conv": taps, "norm_groups": norm_groups}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def _moe(entry, experts, identity, top, ff, shared=None):
    entry = dict(entry)
    entry["mlp"] = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top},
                    "shared": {"ff": shared} if shared else None}
    return entry


def _config(width, vocab, layers, mult=1.0, scale=1.0, eps=1e-5):
    for entry in layers:
        entry.setdefault("mlp", None)
    return {"architecture": "Ruzolorn", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}


CONFIGS = {
    # the parallel layer first; values wider than keys; three key heads; a window off the pages' borders
    "A": _config(64, 130, [
        _moe(_parallel(6, 3, 16, 24, 21, 4, 16, 8, 2, 4, 2, scale=0.4, left_scale=0.8, right_scale=1.3), 5, 1, 2, 24, shared=40),
        _moe(_retention(2, 24, 16, [0.9, 0.995], rot_dims=16, base=500.0), 4, 2, 3, 16),
        _retention(4, 8, 8, [0.5, 0.8, 0.97, 1.0], rot_dims=8)], mult=0.6, scale=2.0),
    # corners: one head, no rotation, no window at all, one group, one norm group, two taps, one
    # tap, top 1, no identity experts, no shared expert, sizes that are no powers of two
    "B": _config(72, 97, [
        _moe(_retention(1, 40, 48, [0.99]), 3, 0, 1, 20),
        _parallel(2, 2, 12, 12, None, 3, 24, 5, 1, 2, 1),
        _moe(_parallel(3, 1, 40, 8, 64, 2, 12, 16, 2, 1, 3, left_scale=0.3), 2, 3, 2, 10, shared=12),
        _moe(_parallel(2, 1, 32, 32, 1, 1, 8, 4, 1, 3, 1), 0, 2, 1, 0, shared=8)], mult=1.0, scale=0.7, eps=1e-3),
    # every token uses every expert: nothing is chosen, so bfloat16 rounding cannot change a choice
    "C": _config(128, 300, [
        _moe(_retention(2, 64, 64, [0.98, 0.999], rot_dims=64, base=1e6), 3, 1, 4, 32, shared=64),
        _moe(_parallel(4, 2, 64, 64, 70, 4, 32, 32, 2, 4, 2, scale=0.2), 3, 1, 4, 32, shared=64)], mult=0.7, scale=3.0),
}
SEEDS = {"A": 3, "B": 4, "C": 5}
STRICT_BF16 = {"C"}


def _folder(path, config, weights):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    json.dump(config, open(os.path.join(path, "config.json"), "w"))
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        weights = plain.random_weights(config, SEEDS[name], sharp=2.0)
        out[name] = (_folder(str(tmp_path_factory.mktemp("ruz" + name)), config, weights), config, weights)
    return out


def _engine(folder, dtype, n_pages, page_size=16, max_requests=4, **kw):
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.utils import load_model

    model, _ = load_model(folder, dtype=dtype)
    return Engine(model, dtype=dtype, page_size=page_size, n_pages=n_pages, max_requests=max_requests, **kw)


def _plain(weights, config, tokens, dtype):
    w = helpers.round_matrices_to_bf16(weights) if dtype == "bfloat16" else weights
    return plain.model(w, config, tokens)


def _close(got, want, dtype, what="", strict=True):
    """Every position within the tolerance.  Not ``strict`` (bfloat16 where experts are chosen): a
    choice between two experts of nearly equal score may fall the other way after rounding, so
    nine positions in ten have to be within it and none may be far off."""
    scale = want.abs().max().item()
    err = (got.double().cpu() - want).abs().amax(-1) / scale
    if strict or dtype == "float32":
        assert err.max().item() <= TOL[dtype], f"{what}: max error {err.max().item():.3e} of the scale"
    else:
        assert (err <= TOL[dtype]).double().mean().item() >= 0.9 and err.max().item() < 0.7, \
            f"{what}: {(err > TOL[dtype]).sum().item()} of {err.numel()} positions beyond the tolerance, worst {err.max().item():.3e}"


def _run(engine, rid, tokens, cuts):
    from mlx_lm_amd.engine import StepEntry

    engine.add_request(rid)
    rows, i = [], 0
    for n in cuts:
        part = tokens[i : i + n]
        rows.append(engine.step([StepEntry(rid, part, list(range(len(part))))]).clone())
        i += n
    assert i == len(tokens)
    engine.end_request(rid)
    return torch.cat(rows)


def _ints(values):
    return torch.tensor(values, dtype=torch.int32).cuda()


# -- each mechanism's kernels alone -------------------------------------------------------


@pytest.mark.parametrize("width,rows", [(64, 7), (100, 7), (1000, 7), (1000, 70), (2500, 3), (300, 65)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_sum_between_two_norms(width, rows, dtype):
    """Few rows: a wave a row with the row in registers; many rows or wide ones: a block a row."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(width)
    h, y = (torch.randn(rows, width, generator=g) * 3).cuda(), (torch.randn(rows, width, generator=g) * 5 + 1).cuda()
    w1, w2 = (1 + 0.3 * torch.randn(width, generator=g)).cuda(), (1 + 0.3 * torch.randn(width, generator=g)).cuda()
    want_h = h.double().cpu() + 0.7 * plain.layer_norm(y.double().cpu(), w1.double().cpu(), 1e-3)
    out = torch.empty(rows, width, dtype=dtype, device="cuda")
    h1, h2 = h.clone(), h.clone()
    kernels.add_normed(h1, y, w1, 0.7, 1e-3)
    kernels.add_normed(h2, y, w1, 0.7, 1e-3, w2, out)
    assert torch.equal(h1, h2) and (h1.double().cpu() - want_h).abs().max() <= 1e-5
    want = plain.layer_norm(want_h, w2.double().cpu(), 1e-3)
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_heads_normed_one_by_one(dtype):
    """Heads of 20 columns that lie 32 apart: the padding is neither read nor written."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 3 * 32 + 8, generator=g).to(dtype).cuda()
    w = (1 + 0.3 * torch.randn(20, generator=g)).cuda()
    before = x.clone()
    kernels.head_rmsnorm(x[:, 8:], 3, 32, 20, w, 1e-4)
    heads = before[:, 8:].double().cpu().view(5, 3, 32)
    want = plain.unit_rms(heads[..., :20], 1e-4) * w.double().cpu()
    got = x[:, 8:].double().cpu().view(5, 3, 32)
    assert (got[..., :20] - want).abs().max() <= (1e-5 if dtype == torch.float32 else 3e-2)
    assert torch.equal(got[..., 20:], heads[..., 20:]) and torch.equal(x[:, :8], before[:, :8])


def _scan_plainly(q, k, v, a, S):
    """``S = a_t S + k_t v_t^T; o_t = S^T q_t`` for one head, float64."""
    out = []
    for t in range(q.shape[0]):
        S = a[t] * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out), S


@pytest.mark.parametrize("chunked", [False, True, "spans"])
@pytest.mark.parametrize("N,P,H,Hk", [(8, 8, 4, 4), (24, 16, 2, 1), (5, 24, 3, 1), (64, 64, 2, 2), (40, 48, 1, 1), (128, 128, 1, 1),
                                      (6, 10, 2, 2), (200, 100, 1, 1)])
def test_the_decaying_state_in_portions_of_two_requests(N, P, H, Hk, chunked):
    """Two requests side by side, three steps: the state rows are read at a portion's start and
    written at its end, each request's own (rows 2 and 0 of four; the others stay as they are).
    Token by token, and with the kernel that takes a chunk of tokens at a time (portions longer
    than a chunk, of a chunk and a token, and of one token)."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(N + P)
    lens = [[5, 2], [1, 9], [2, 1]] if not chunked else [[70, 2], [1, 129], [65, 1]]
    n = [sum(x[0] for x in lens), sum(x[1] for x in lens)]
    q = [torch.randn(m, Hk, N, generator=g).double() for m in n]
    k = [torch.randn(m, Hk, N, generator=g).double() * N ** -0.5 for m in n]
    v = [torch.randn(m, H, P, generator=g).double() for m in n]
    log_a = [-torch.rand(m, H, generator=g).double() * (0.1 if chunked else 1.0) for m in n]
    ksc = [torch.rand(m, H, generator=g).double() + 0.5 for m in n]
    skip = torch.randn(H, generator=g)
    state = torch.full((4, 7 + H * N * P), 3.0).cuda()
    state[[2, 0], 7:] = 0
    want = []
    for r in range(2):
        heads = []
        for h in range(H):
            o, _ = _scan_plainly(q[r][:, h // (H // Hk)], k[r][:, h // (H // Hk)] * ksc[r][:, h, None], v[r][:, h],
                                 log_a[r][:, h].exp(), torch.zeros(N, P, dtype=torch.float64))
            heads.append(o + skip[h].double() * v[r][:, h])
        want.append(torch.stack(heads, 1))
    at, got = [0, 0], [[], []]
    for step in lens:
        rows = lambda xs: torch.cat([xs[r][at[r] : at[r] + step[r]].flatten(1) for r in range(2)]).float().cuda()  # noqa: E731
        out = torch.empty(sum(step), H * P, device="cuda")
        spans = None
        if chunked == "spans":  # spans of 64 tokens side by side: (tokens, spans, their requests, their starts, a request's first)
            req, first, lo = [], [], []
            for r_, m_ in enumerate(step):
                first.append(len(req))
                req += [r_] * ((m_ + 63) // 64)
                lo += list(range(0, m_, 64))
            spans = (64, len(req), _ints(req), _ints(lo), _ints(first), lambda shape, dt: torch.empty(shape, dtype=dt, device="cuda"))
        kernels.state_scan(out, rows(q), rows(k), rows(v), state, 7, _ints([0, step[0]]), _ints(step), _ints([2, 0]), 2, H, Hk, N, P,
                           log_a=rows(log_a), k_scale=rows(ksc), skip=skip.cuda(), chunked=bool(chunked), spans=spans)
        got[0].append(out[: step[0]].cpu()), got[1].append(out[step[0] :].cpu())
        at = [at[0] + step[0], at[1] + step[1]]
    for r in range(2):
        w = want[r].flatten(1)
        assert (torch.cat(got[r]).double() - w).abs().max() <= 3e-5 * w.abs().max()
    assert (state[[1, 3]] == 3.0).all() and (state[:, :7] == 3.0).all()


def test_a_token_far_back_in_the_decaying_state():
    """A decay close to one: the query of the last of 1,500 tokens equals, scaled, the key of token
    3, and the output is near that token's value.  Rotation on: the angle of 1,496 positions."""
    from mlx_lm_amd.ops import kernels

    n, N, P = 1500, 16, 8
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(n, N, generator=g) * 0.1, torch.randn(n, N, generator=g) * 0.01, torch.randn(n, P, generator=g)
    k[3] = torch.randn(N, generator=g) * 3.0
    inv_freq = torch.tensor([100.0 ** (-2.0 * i / N) for i in range(N // 2)])
    pos = torch.arange(n)
    # the query that, rotated to position n - 1, meets the key as rotated at position 3
    turned = plain.rotate_half(k[3].double()[None, None], pos[3:4], N, 100.0)
    q[n - 1] = plain.rotate_half(turned, -pos[n - 1 :], N, 100.0)[0, 0].float() * 4.0
    qr = plain.rotate_half(q.double()[:, None], pos, N, 100.0)[:, 0]
    kr = plain.rotate_half(k.double()[:, None], pos, N, 100.0)[:, 0] * 0.25
    decay = 1.0 - 1.0 / 4096
    want, S = _scan_plainly(qr, kr, v.double(), torch.full((n,), decay, dtype=torch.float64), torch.zeros(N, P, dtype=torch.float64))
    lean = (qr[n - 1] @ kr[3]) * decay ** (n - 4)
    assert lean > 10 * (want[n - 1] - lean * v[3].double()).abs().max()  # the far token is what the output is made of
    state = torch.zeros(1, N * P).cuda()
    out = torch.empty(n, P, device="cuda")
    cut = 1490
    for a, b in ((0, cut), (cut, n - 1), (n - 1, n)):
        kernels.state_scan(out[a:b], q[a:b].cuda(), k[a:b].cuda(), v[a:b].cuda(), state, 0, _ints([0]), _ints([b - a]), _ints([0]),
                           1, 1, 1, N, P, decay=torch.tensor([decay]).cuda(), k_mult=0.25, rot_dims=N, inv_freq=inv_freq.cuda(),
                           positions=pos[a:b].to(torch.int32).cuda(), chunked=b - a > 8)
    assert (out.double().cpu() - want).abs().max() <= 1e-4 * want.abs().max()
    assert (state.double().cpu().view(N, P) - S).abs().max() <= 1e-4 * S.abs().max()


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_the_convolution_across_portions(taps):
    """Portions of 2, 1, 1, 6 and 3 tokens (shorter than the taps, so old inputs stay in the state)
    beside a second request; the first tokens of a request see zeros."""
    from mlx_lm_amd.ops import kernels

    C, H, pad = 11, 3, 5
    g = torch.Generator().manual_seed(taps)
    n = 13
    u = [torch.randn(n, pad + C + H, generator=g) for _ in range(2)]
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    dt_bias, a_log = torch.randn(H, generator=g), torch.randn(H, generator=g) * 0.3
    state = torch.zeros(3, 4 + (taps - 1) * C).cuda()
    want = [plain.silu(plain.causal_conv(x[:, pad : pad + C].double(), w.double(), b.double())) for x in u]
    at, got, got_dt, got_a = 0, [[], []], [], []
    for m in (2, 1, 1, 6, 3):
        rows = torch.cat([u[0][at : at + m], u[1][at : at + m]]).cuda()
        xbc, dt, la = torch.empty(2 * m, C, device="cuda"), torch.empty(2 * m, H, device="cuda"), torch.empty(2 * m, H, device="cuda")
        req = _ints([0] * m + [1] * m)
        kernels.ssm_prepare(xbc, dt, la, rows, pad, pad + C, w.cuda(), b.cuda(), dt_bias.cuda(), a_log.cuda(), state, 4, req,
                            _ints([0, m]), _ints([2, 1]), single_tokens=m == 1)  # (one token each: the kernel keeps the state itself)
        if m > 1:
            kernels.conv_state_update(rows, pad, taps, C, state, 4, _ints([0, m]), _ints([m, m]), _ints([2, 1]), 2)
        got[0].append(xbc[:m].cpu()), got[1].append(xbc[m:].cpu())
        got_dt.append(dt[:m].cpu()), got_a.append(la[:m].cpu())
        at += m
    for r in range(2):
        assert (torch.cat(got[r]).double() - want[r]).abs().max() <= 1e-5
    want_dt = plain.softplus(u[0][:, pad + C :].double() + dt_bias.double())
    assert (torch.cat(got_dt).double() - want_dt).abs().max() <= 1e-5
    assert (torch.cat(got_a).double() + a_log.double().exp() * want_dt).abs().max() <= 1e-5
    assert (state[0] == 0).all() and (state[:, :4] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_gate_comes_before_the_norm_in_parts(dtype):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(3)
    y, z, w = torch.randn(6, 40, generator=g) * 4, torch.randn(6, 48, generator=g), 1 + 0.2 * torch.randn(40, generator=g)
    out = torch.empty(6, 40, dtype=dtype, device="cuda")
    kernels.gated_group_rmsnorm(out, y.cuda(), z.cuda()[:, 8:], w.cuda(), 5, 1e-4)
    gated = y.double() * plain.silu(z[:, 8:].double())
    want = plain.unit_rms(gated.view(6, 5, 8), 1e-4).reshape(6, 40) * w.double()
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 3e-2)
    other = plain.unit_rms(y.double().view(6, 5, 8), 1e-4).reshape(6, 40) * w.double() * plain.silu(z[:, 8:].double())
    assert (other - want).abs().max() > 0.1  # (the other order is another function)


@pytest.mark.parametrize("n_out,top", [(14, 4), (3, 3), (5, 1), (70, 8)])
def test_the_routers_choice(n_out, top):
    """The choice adds the correction, the weights do not; corrections large enough to change the
    order of nearly every token's experts."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(n_out)
    z = torch.randn(50, n_out, generator=g) * 2
    corr = torch.randn(n_out, generator=g) * 0.1
    idx, w = torch.empty(50, top, dtype=torch.int32, device="cuda"), torch.empty(50, top, device="cuda")
    kernels.router_choice(idx, w, z.cuda(), corr.cuda(), top)
    s = torch.softmax(z.double(), -1)
    want = torch.topk(s + corr.double(), top, -1).indices
    assert torch.equal(idx.cpu().long(), want)
    assert (w.double().cpu() - torch.gather(s, 1, want)).abs().max() <= 1e-6
    if top < n_out:
        assert not torch.equal(torch.topk(s, top, -1).indices, want)
    kernels.router_choice(idx, w, z.cuda(), None, top)
    assert torch.equal(idx.cpu().long(), torch.topk(s, top, -1).indices)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_choice_and_gate_in_one_launch(dtype):
    """For steps of few tokens one product gives [router | gate | up] and one kernel chooses the
    experts and makes silu(gate) * up."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(7)
    T, n_out, top, F = 5, 11, 3, 40
    zu = torch.randn(T, n_out + 2 * F, generator=g) * 2
    corr = torch.randn(n_out, generator=g) * 0.1
    idx, w = torch.empty(T, top, dtype=torch.int32, device="cuda"), torch.empty(T, top, device="cuda")
    act = torch.empty(T, F, dtype=dtype, device="cuda")
    kernels.route_and_gate(idx, w, act, zu.cuda(), corr.cuda(), top, n_out)
    s = torch.softmax(zu[:, :n_out].double(), -1)
    want = torch.topk(s + corr.double(), top, -1).indices
    assert torch.equal(idx.cpu().long(), want) and (w.double().cpu() - torch.gather(s, 1, want)).abs().max() <= 1e-6
    gated = plain.silu(zu[:, n_out : n_out + F].double()) * zu[:, n_out + F :].double()
    assert (act.double().cpu() - gated).abs().max() <= (1e-5 if dtype == torch.float32 else 3e-2) * gated.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,width,F", [(1, 64, 24), (9, 72, 10), (40, 256, 64), (300, 72, 40), (70, 104, 8)])
def test_chosen_experts_and_identity_experts(dtype, T, width, F):
    from mlx_lm_amd.ops import kernels

    E, n_id, top = 5, 2, 3
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, width, generator=g).to(dtype)
    wg, wu = (torch.randn(E, F, width, generator=g) * width ** -0.5).to(dtype), (torch.randn(E, F, width, generator=g) * width ** -0.5).to(dtype)
    wd = (torch.randn(E, width, F, generator=g) * F ** -0.5).to(dtype)
    idx = torch.stack([torch.randperm(E + n_id, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wt = torch.rand(T, top, generator=g)
    y0 = torch.randn(T, width, generator=g)
    want = y0.double().clone()
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            xe = x[t].double()
            out = xe if e >= E else wd[e].double() @ (plain.silu(wg[e].double() @ xe) * (wu[e].double() @ xe))
            want[t] += wt[t, j].double() * out
    y = y0.clone().cuda()
    act = torch.empty(T * top, F, dtype=dtype, device="cuda")
    kernels.expert_rows(y, x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), idx.cuda(), wt.cuda(), top, act, accumulate=True)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert (y.double().cpu() - want).abs().max() <= tol * want.abs().max()
    kernels.expert_rows(y, x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), idx.cuda(), wt.cuda(), top, act, accumulate=False)
    assert (y.double().cpu() - (want - y0.double())).abs().max() <= tol * want.abs().max()
    if kernels.expert_tiles_takes(F, width, dtype):
        # the same through the sorted tiles (an expert that no token picked, tiles of fewer than 64 picks)
        def alloc(shape, dt):
            return torch.empty(shape, dtype=dt, device="cuda")

        for accumulate in (True, False):
            y = y0.clone().cuda()
            kernels.expert_tiles(y, x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), idx.cuda(), wt.cuda(), top, alloc, accumulate=accumulate)
            assert (y.double().cpu() - (want if accumulate else want - y0.double())).abs().max() <= tol * want.abs().max()


# -- the tests' weights show what they are meant to show ---------------------------------


def test_the_plain_side_notices_what_the_comparisons_are_for(models):
    """With these weights a window one token off, identity experts left out, a dropped correction,
    a norm in one part instead of two, fewer turning columns or the scales of the two mixers
    swapped move the logits by far more than the float32 tolerance."""
    _, config, weights = models["A"]
    tokens = helpers.random_tokens(90, config["vocab"], seed=1)
    base = plain.model(weights, config, tokens)
    scale = base.abs().max().item()

    def moved(change):
        c, w = copy.deepcopy(config), dict(weights)
        change(c, w)
        return (plain.model(w, c, tokens) - base)[40:].abs().max().item() / scale

    def window(c, w):
        c["layers"][0]["mixer"]["left"]["mask"]["size"] += 1

    def correction(c, w):
        w["l0.mlp.correction"] = torch.zeros_like(w["l0.mlp.correction"])

    def identity(c, w):  # an identity expert that gives nothing back
        r = c["layers"][1]["mlp"]["router"]
        r["experts"], r["identity"] = r["experts"] + r["identity"], 0
        for e in range(r["experts"] - 2, r["experts"]):
            w[f"l1.mlp.e{e}.gate"], w[f"l1.mlp.e{e}.up"] = torch.zeros(16, 64), torch.zeros(16, 64)
            w[f"l1.mlp.e{e}.down"] = torch.zeros(64, 16)

    def norm_groups(c, w):
        c["layers"][0]["mixer"]["right"]["norm_groups"] = 1

    def rotation(c, w):
        c["layers"][1]["mixer"]["rot"]["dims"] = 8

    def scales(c, w):
        m = c["layers"][0]["mixer"]
        m["left_scale"], m["right_scale"] = m["right_scale"], m["left_scale"]

    for change in (window, correction, identity, norm_groups, rotation, scales):
        assert moved(change) > 100 * TOL["float32"], change.__name__


# -- whole, decoded, portions ----------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n", [("A", 150), ("B", 130), ("C", 200)])
def test_whole_decoded_and_portions(models, dtype, name, n):
    folder, config, weights = models[name]
    strict = name in STRICT_BF16
    tokens = helpers.random_tokens(n, config["vocab"], seed=n)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=(n + 15) // 16 + 2)
    _close(_run(eng, "whole", tokens, [n]), want, dtype, "whole", strict)
    # most of it at once, then token by token until the windows have passed over decoded tokens
    _close(_run(eng, "decoded", tokens, [n - 90] + [1] * 90), want, dtype, "last 90 one by one", strict)
    _close(_run(eng, "portions", tokens, helpers.cuts_changing(n)), want, dtype, "portions of changing size", strict)
    _close(_run(eng, "twos", tokens[:64], [2] * 32), want[:64], dtype, "portions of two tokens", strict)
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


def test_portions_give_what_the_whole_prompt_gives(models):
    """However a prompt is cut, the logits agree with the uncut prompt's to rounding (float32: the
    engine against itself, much tighter than against the plain side)."""
    folder, config, _ = models["A"]
    tokens = helpers.random_tokens(140, config["vocab"], seed=8)
    eng = _engine(folder, "float32", n_pages=12)
    whole = _run(eng, "w", tokens, [140])
    for cuts in (helpers.cuts_changing(140), [1] * 140, [20, 1, 21, 22, 2, 74], [137, 3]):
        got = _run(eng, "c", tokens, cuts)
        assert (got - whole).abs().max().item() <= 2e-5 * whole.abs().max().item(), cuts[:6]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decode(models, dtype):
    """Every token one by one from the first: 400 of them, recorded decode steps replayed, the window
    passing page borders, the state carried 400 times."""
    folder, config, weights = models["C"]
    n = 400
    tokens = helpers.random_tokens(n, config["vocab"], seed=77)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=n // 16 + 1)
    got = _run(eng, "r", tokens, [1] * n)
    _close(got[:8], want[:8], dtype, "first tokens")
    _close(got, want, dtype, "decoding every token")


def test_a_pool_smaller_than_the_sequence(models):
    """The window's passed pages are used again, and what freed pages hold is never read."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models["A"]
    n = 250
    tokens = helpers.random_tokens(n, config["vocab"], seed=5)
    want = _plain(weights, config, tokens, "float32")
    eng = _engine(folder, "float32", n_pages=6)  # 96 tokens' worth for a window of 21
    eng.add_request("r")
    rows, i = [], 0
    for c in [30, 2, 17] + [1] * 60 + [9, 20, 11] + [1] * 101:
        rows.append(eng.step([StepEntry("r", tokens[i : i + c], list(range(c)))]).clone())
        i += c
        eng.cache.poison_free_pages()
    assert i == n
    _close(torch.cat(rows), want, "float32", "a pool smaller than the sequence")
    eng.end_request("r")
    eng.cache.check()


# -- batches -------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_equal_each_request_alone(models, dtype, name):
    """Up to four live requests of unequal lengths, portions beside single tokens, requests that
    sit a step out; state rows and pages of finished requests are used again by later ones (a
    state row that was not cleared, or another request's, would show at once)."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models[name]
    lengths = [70, 9, 131, 40, 3, 97, 55]
    tokens, steps = helpers.mixed_trace({"vocab_size": config["vocab"]}, 21, lengths, n_live=4)
    eng = _engine(folder, dtype, n_pages=helpers.held(lengths, 4) // 16, max_requests=4)
    got = {rid: [] for rid in tokens}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if not eng.has_request(e["id"]):
                eng.add_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = eng.step(entries).clone()
        at = 0
        for e in entries:
            got[e.request_id].append(logits[at : at + len(e.want)])
            at += len(e.want)
        for rid in s["end"]:
            eng.end_request(rid)
        eng.cache.poison_free_pages()
    for rid, toks in tokens.items():
        _close(torch.cat(got[rid]), _plain(weights, config, toks, dtype), dtype, f"request {rid} in mixed batches",
               name in STRICT_BF16)
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_twenty_requests_decode_together(models, dtype):
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models["C"]
    lengths = [5 + 7 * i for i in range(20)]
    tokens = [helpers.random_tokens(n + 12, config["vocab"], seed=200 + n) for n in lengths]
    eng = _engine(folder, dtype, n_pages=sum((n + 12 + 15) // 16 for n in lengths), max_requests=20)
    for i, (n, toks) in enumerate(zip(lengths, tokens)):
        eng.add_request(i)
        eng.step([StepEntry(i, toks[:n], [])])
    got = [[] for _ in lengths]
    for step in range(12):
        logits = eng.step([StepEntry(i, [tokens[i][n + step]], [0]) for i, n in enumerate(lengths)]).clone()
        for i in range(len(lengths)):
            got[i].append(logits[i])
    for i, n in enumerate(lengths):
        _close(torch.stack(got[i]), _plain(weights, config, tokens[i], dtype)[n:], dtype, f"request {i} among twenty")


def test_models_without_pages_and_without_state(tmp_path):
    """Only retention layers (no cache group at all), and only a parallel layer without a window."""
    # (also: value columns and an inner size that are no multiples of 8, whose output products get zero columns)
    for name, layers in (("r", [_moe(_retention(2, 16, 16, [0.9, 0.99], rot_dims=8), 3, 1, 2, 16), _retention(1, 8, 24, [0.7]),
                                _retention(3, 6, 20, [0.8, 0.9, 0.95], rot_dims=6), _parallel(1, 1, 8, 8, 5, 3, 4, 6, 3, 2, 1)]),
                         ("p", [_moe(_parallel(2, 1, 16, 16, None, 2, 8, 8, 1, 3, 1), 2, 0, 1, 8)])):
        config = _config(48, 61, layers, mult=0.9)
        weights = plain.random_weights(config, 12, sharp=2.0)
        folder = _folder(str(tmp_path / name), config, weights)
        tokens = helpers.random_tokens(70, 61, seed=3)
        eng = _engine(folder, "float32", n_pages=8)
        want = plain.model(weights, config, tokens)
        _close(_run(eng, "a", tokens, [70]), want, "float32", name + " whole")
        _close(_run(eng, "b", tokens, [33, 2, 1, 1, 30, 3]), want, "float32", name + " in portions")


def _drawn_config(seed):
    g = torch.Generator().manual_seed(seed)

    def pick(options):
        return options[int(torch.randint(0, len(options), (), generator=g))]

    layers = []
    for _ in range(pick([1, 2, 3, 4])):
        if pick([0, 1]):
            heads, dim = pick([1, 2, 4]), pick([8, 16, 24, 32, 64])
            vdim = pick([8, 16, 32, 40])
            if (heads * vdim) % 8:
                vdim *= 2
            decay = [pick([0.5, 0.9, 0.99, 0.999, 1.0]) for _ in range(heads)]
            entry = _retention(heads, dim, vdim, decay, rot_dims=pick([None, dim, dim // 2 // 2 * 2]), base=pick([100.0, 1e4, 1e6]))
        else:
            kv = pick([1, 2, 3])
            groups = pick([1, 2])
            s_heads, s_vdim = groups * pick([1, 2, 3]), pick([8, 16, 24, 32])
            norm_groups = pick([g_ for g_ in (1, 2, 3, 4) if (s_heads * s_vdim) % g_ == 0])
            entry = _parallel(kv * pick([1, 2, 4]), kv, pick([8, 12, 16, 32, 40, 64, 96]), pick([8, 16, 24, 48, 80]),
                              pick([None, 1, 7, 16, 33, 64, 100, 1000]), s_heads, s_vdim, pick([4, 8, 16, 32, 64]), groups,
                              pick([1, 2, 3, 4, 5]), norm_groups, scale=pick([None, 0.05, 0.4]), left_scale=pick([0.5, 1.0, 1.2]),
                              right_scale=pick([0.5, 1.0, 2.0]))
        if pick([0, 1, 1]):
            experts, identity = pick([1, 2, 5, 9]), pick([0, 1, 3])
            entry = _moe(entry, experts, identity, pick(list(range(1, min(4, experts + identity) + 1))), pick([4, 8, 20, 64]),
                         shared=pick([None, 8, 20, 64]))
        layers.append(entry)
    return _config(pick([16, 40, 64, 104, 256]), pick([17, 100, 257, 1000]), layers, mult=pick([0.5, 0.7, 1.0, 1.4]),
                   scale=pick([1.0, 8.0, 0.3]), eps=pick([1e-6, 1e-5, 1e-2]))


@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations(tmp_path, seed):
    """Every size, the layers' order, windows and constants drawn: whole, in portions, and two
    requests side by side, in float32."""
    from mlx_lm_amd.engine import StepEntry

    config = _drawn_config(seed)
    weights = plain.random_weights(config, 100 + seed, sharp=2.0)
    folder = _folder(str(tmp_path / "m"), config, weights)
    a, b = helpers.random_tokens(120, config["vocab"], seed=seed), helpers.random_tokens(75, config["vocab"], seed=50 + seed)
    wa, wb = plain.model(weights, config, a), plain.model(weights, config, b)
    eng = _engine(folder, "float32", n_pages=16)
    _close(_run(eng, "whole", a, [120]), wa, "float32", f"seed {seed} whole: {json.dumps(config)}")
    eng.add_request("a"), eng.add_request("b")
    ga, gb, ia, ib = [], [], 0, 0
    for ca, cb in ((50, 2), (1, 40), (1, 1), (38, 1), (2, 30), (28, 1)):
        out = eng.step([StepEntry("a", a[ia : ia + ca], list(range(ca))), StepEntry("b", b[ib : ib + cb], list(range(cb)))]).clone()
        ga.append(out[:ca]), gb.append(out[ca:])
        ia, ib = ia + ca, ib + cb
    _close(torch.cat(ga), wa, "float32", f"seed {seed}, first of two")
    _close(torch.cat(gb), wb, "float32", f"seed {seed}, second of two")


def test_recorded_steps_equal_eager_steps(models):
    """Decode steps replayed from recorded graphs against the same steps run eagerly, bit for bit
    (a state row is read and written once a step either way)."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, _ = models["A"]
    seqs = {"a": helpers.random_tokens(60, config["vocab"], 1), "b": helpers.random_tokens(45, config["vocab"], 2)}
    results = {}
    for use_graphs in (True, False):
        eng = _engine(folder, "bfloat16", n_pages=10, use_graphs=use_graphs)
        assert eng.use_graphs == use_graphs  # every part launches kernels only
        for r in seqs:
            eng.add_request(r)
        out = [eng.step([StepEntry("a", seqs["a"][:20], [19]), StepEntry("b", seqs["b"][:5], [4])]).clone()]
        for i in range(40):
            out.append(eng.step([StepEntry("a", [seqs["a"][20 + i]], [0]), StepEntry("b", [seqs["b"][5 + i]], [0])]).clone())
        if use_graphs:
            assert helpers.decode_graphs(eng, 2)[0].graph is not None
        results[use_graphs] = torch.cat(out)
    assert torch.equal(results[True], results[False])


# -- generation through the entry points -----------------------------------------------------


def _greedy(weights, config, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(plain.model(weights, config, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_scheduler(models):
    from mlx_lm_amd import batch_generate, load, stream_generate

    folder, config, weights = models["A"]
    model, tok = load(folder, dtype="float32")
    prompts = [helpers.random_tokens(n, config["vocab"], seed=n) for n in (23, 5, 61)]
    want = [_greedy(weights, config, p, 10) for p in prompts]
    got = [r.token for r in stream_generate(model, tok, prompts[0], max_tokens=10, prefill_step_size=7)]
    assert got == want[0]
    batch = batch_generate(model, tok, prompts, max_tokens=10)
    assert [[int(t) for t in text.split()] for text in batch.texts] == want


def test_command_line_and_trace_replay(tmp_path, models):
    """``python -m mlx_lm_amd generate`` on a folder of this design, and the replay program on a
    configuration with seeded random weights."""
    folder, config, weights = models["B"]
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]
    want = _greedy(weights, config, prompt, 25)
    env = dict(os.environ, PYTHONPATH=ROOT)
    out = subprocess.run(
        [sys.executable, "-m", "mlx_lm_amd", "generate", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)),
         "--max-tokens", "25", "--dtype", "float32", "--verbose", "F", "--num-pages", "8", "--prefill-step-size", "3"],
        capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip() == " ".join(map(str, want))
    json.dump(config, open(tmp_path / "config.json", "w"))
    tokens = helpers.random_tokens(50, config["vocab"], seed=9)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:31], "want": [30]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": tokens[31:], "want": "all"}], "end": ["x"]}]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--config", str(tmp_path / "config.json"),
                           "--seed", "4", "--dtype", "float32", "--out", str(tmp_path / "out"), "--max-tokens", "64"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    from mlx_lm_amd.config.registry import get_model_classes

    model_cls, args_cls = get_model_classes(config)
    drawn = model_cls.random_weights(args_cls.from_dict(config), 4, "b")
    got = np.fromfile(tmp_path / "out" / "1.f32", dtype="<f4").reshape(-1, config["vocab"])
    _close(torch.from_numpy(got), plain.model(drawn, config, tokens)[31:], "float32", "the replay's second step")
