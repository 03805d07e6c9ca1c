"""Pafutar in the engine against the plain implementation (plain_pafutar.py): each mechanism,
whole prompts, decoding, portions, mixed batches, reused pages, window and kept-first edges,
generation through the entry points."""

import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_pafutar as plain  # noqa: E402

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# max |engine - plain| over max |plain logits|: float32 sums where the plain side has float64;
# bfloat16 rounds activations between the products (the plain side gets the rounded matrices)
TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def _mixer(heads, kv_heads, dim, window=None, keep_first=0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale or dim**-0.5}
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return m


def _layer(mixer, ff=None, weights_of=None):
    e = {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        e["weights_of"] = weights_of
    return e


def _config(width, vocab, layers, max_positions=256, alpha=1.0, scale=1.0, eps=1e-6):
    return {"architecture": "Pafutar", "vocab": vocab, "width": width, "max_positions": max_positions,
            "embedding": {"scale": scale}, "norm": {"eps": eps}, "postln_alpha": alpha, "layers": layers}


_A0 = _mixer(4, 2, 16, window=24, keep_first=5, scale=0.3)
_A1 = _mixer(2, 1, 32, window=40, keep_first=0)
_B0 = _mixer(3, 3, 48)  # no mask at all
_B2 = _mixer(2, 2, 24, window=17, keep_first=3)  # a head size that is a multiple of 8 only; edges off the pages' borders
CONFIGS = {
    # a layer run twice (with a cache and shift state of its own each), a layer without feed-forward
    "A": _config(64, 130, [_layer(_A0, 72), _layer(_A1), _layer(_A0, 72, weights_of=0)], alpha=1.7, scale=3.0, eps=1e-5),
    # no window, an inner size that is no multiple of 8, alpha 1 (the plain sum), kept tokens beyond a page
    "B": _config(96, 211, [_layer(_B0, 100), _layer(_B2, 52), _layer(_B0, 100, weights_of=0),
                           _layer(_mixer(4, 1, 16, window=33, keep_first=18), 40)], alpha=1.0, scale=9.5),
    # head sizes of 64 and 128 (the kernels that stream keys through registers and the matrix cores)
    "F": _config(128, 300, [_layer(_mixer(2, 1, 64, window=70, keep_first=9), 256), _layer(_mixer(2, 2, 128, window=50, keep_first=33), 128),
                            _layer(_mixer(4, 2, 32), 64)], max_positions=512, alpha=2.0, scale=11.0),
}
# the corners: one head, a head size beyond what the row kernels take, small ones (8; 20 and 12,
# multiples of four only), a window
# of one token, more kept tokens than the window is long, a window and kept tokens that no sequence
# here outgrows, a width that is no multiple of 64, a layer that runs three times
CONFIGS["X"] = _config(72, 97, [_layer(_mixer(1, 1, 160, window=1, keep_first=0), 24), _layer(_mixer(3, 1, 8, window=5, keep_first=40)),
                                _layer(_mixer(1, 1, 160, window=1, keep_first=0), 24, weights_of=0),
                                _layer(_mixer(2, 2, 40, window=250, keep_first=300), 80),
                                _layer(_mixer(2, 1, 20, window=30, keep_first=4), 16), _layer(_mixer(2, 2, 12)),
                                _layer(_mixer(1, 1, 160, window=1, keep_first=0), 24, weights_of=2)],
                       max_positions=330, alpha=0.7, scale=0.5, eps=1e-3)
SEEDS = {"A": 3, "B": 4, "F": 5, "X": 6}
# how peaked the attention is: with seven layers as peaked as the others', bfloat16 rounding alone
# moves a logit of X by 6 % now and then (any six of its layers: 2 to 3 %)
SHARP = {"A": 4.0, "B": 4.0, "F": 4.0, "X": 1.5}


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
        weights = plain.random_weights(config, SEEDS[name], sharp=SHARP[name])
        out[name] = (_folder(str(tmp_path_factory.mktemp("paf" + name)), config, weights), config, weights)
    return out


def _engine(folder, dtype, n_pages, page_size=16, max_requests=4, **kw):
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.utils import load_model

    model, _ = load_model(folder, dtype=dtype)
    return Engine(model, dtype=dtype, page_size=page_size, n_pages=n_pages, max_requests=max_requests, **kw)


def _plain(weights, config, tokens, dtype):
    w = helpers.round_matrices_to_bf16(weights) if dtype == "bfloat16" else weights
    return plain.forward(w, config, tokens)


def _close(got, want, dtype, what=""):
    scale = want.abs().max().item()
    err = (got.double().cpu() - want).abs().max().item()
    assert err <= TOL[dtype] * scale, f"{what}: max error {err:.3e} against scale {scale:.3e}"


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


# -- each mechanism alone ------------------------------------------------------------


def _ctypes_lib(name):
    from mlx_lm_amd.ops import build

    return build.load(name)


def _stream():
    from mlx_lm_amd.ops import kernels

    return kernels._stream()


@pytest.mark.parametrize("width", [64, 100, 333])
def test_rmsnorm_kernel(width):
    import ctypes

    L = _ctypes_lib("rmsnorm")
    g = torch.Generator().manual_seed(width)
    x = (torch.randn(9, width, generator=g) * 3).cuda()
    gamma = (1 + 0.3 * torch.randn(width, generator=g)).cuda()
    rows = torch.tensor([7, 0, 3], dtype=torch.int32).cuda()
    for dtype, code, tol in ((torch.float32, 0, 1e-6), (torch.bfloat16, 1, 1e-2)):
        out = torch.empty(3, width, dtype=dtype, device="cuda")
        rc = L.rmsnorm(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(x.data_ptr()), width, ctypes.c_void_p(rows.data_ptr()),
                       ctypes.c_void_p(gamma.data_ptr()), ctypes.c_float(1e-3), 3, width, code, _stream())
        assert rc == 0, L.mlxlm_last_error()
        want = plain.rms_norm(x.double().cpu()[[7, 0, 3]], gamma.double().cpu(), 1e-3)
        assert (out.double().cpu() - want).abs().max() <= tol * want.abs().max()


@pytest.mark.parametrize("W", [72, 70, 1280])  # (70: no multiple of four, the kernels for any width)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_shift_and_the_sum_that_is_normed(dtype, W):
    """Two requests' rows side by side: the shift reads the row before (the state for a portion's
    first row), the fused sum-and-norm keeps each request's last old row in the state."""
    import ctypes

    L = _ctypes_lib("post_norm_block")
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
    g = torch.Generator().manual_seed(1)
    h = torch.randn(7, W, generator=g).cuda()
    mu, s, gamma = (torch.rand(W, generator=g).cuda() for _ in range(3))
    state = torch.randn(4, W, generator=g).cuda()
    slot_ids = torch.tensor([2, 0], dtype=torch.int32).cuda()
    token_req = torch.tensor([0, 0, 0, 1, 1, 1, 1], dtype=torch.int32).cuda()
    code = 0 if dtype == torch.float32 else 1
    out = torch.empty(7, W, dtype=dtype, device="cuda")
    assert L.token_shift(P(out), P(h), W, P(mu), P(state), ctypes.c_size_t(W), P(slot_ids), P(token_req), 7, W, code, 0, _stream()) == 0
    hc, sc = h.double().cpu(), state.double().cpu()
    want = torch.cat([plain.token_shift(hc[:3], mu.double().cpu(), sc[2]), plain.token_shift(hc[3:], mu.double().cpu(), sc[0])])
    assert (out.double().cpu() - want).abs().max() <= (1e-6 if code == 0 else 2e-2)
    y = torch.randn(7, W, generator=g).cuda()
    copy_ = torch.empty(7, W, dtype=dtype, device="cuda")
    h2 = h.clone()
    assert L.residual_rmsnorm(P(h2), W, P(y), W, None, 0, ctypes.c_float(1.5), P(s), P(gamma), ctypes.c_float(1e-4), P(state),
                              ctypes.c_size_t(W), P(slot_ids), P(token_req), P(copy_), code, 0, 7, W, _stream()) == 0
    want = plain.rms_norm(1.5 * hc + s.double().cpu() * y.double().cpu(), gamma.double().cpu(), 1e-4)
    assert (h2.double().cpu() - want).abs().max() <= 2e-6
    # the sublayer's output still in parts (a product that split its inner size), with and without rows beside them
    parts = torch.randn(5, 7, W, generator=g).cuda()
    for rows in (y, None):
        h3 = h.clone()
        assert L.residual_rmsnorm(P(h3), W, P(rows), W, P(parts), 5, ctypes.c_float(1.5), P(s), P(gamma), ctypes.c_float(1e-4),
                                  None, ctypes.c_size_t(0), None, None, None, 0, 0, 7, W, _stream()) == 0
        total = parts.double().cpu().sum(0) + (y.double().cpu() if rows is not None else 0)
        want3 = plain.rms_norm(1.5 * hc + s.double().cpu() * total, gamma.double().cpu(), 1e-4)
        assert (h3.double().cpu() - want3).abs().max() <= 4e-6
    assert (copy_.double().cpu() - want).abs().max() <= (2e-6 if code == 0 else 2e-2)
    assert torch.equal(state[2], h[2]) and torch.equal(state[0], h[6])  # the old rows, not the normed ones
    if code == 1 and W % 4 == 0:
        # the same rows in the order in which the product of 17 to 64 rows reads them fastest
        from mlx_lm_amd.ops.kernels import PackedRows

        packed = PackedRows.empty(7, W, "cuda")
        assert L.token_shift(P(packed), P(h), W, P(mu), P(sc.float().cuda()), ctypes.c_size_t(W), P(slot_ids), P(token_req), 7, W,
                             1, 1, _stream()) == 0
        assert torch.equal(packed.rows(), out)
        packed, h4 = PackedRows.empty(7, W, "cuda"), h.clone()
        assert L.residual_rmsnorm(P(h4), W, P(y), W, None, 0, ctypes.c_float(1.5), P(s), P(gamma), ctypes.c_float(1e-4), None,
                                  ctypes.c_size_t(0), None, None, P(packed), 1, 1, 7, W, _stream()) == 0
        assert torch.equal(packed.rows(), copy_)
    assert torch.equal(state[1].cpu(), sc[1].float()) and torch.equal(state[3].cpu(), sc[3].float())


@pytest.mark.parametrize("rows", [3, 40, 200])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_squared_relu_in_the_products_epilogue(rows, dtype):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(rows)
    a = torch.randn(rows, 96, generator=g).to(dtype).cuda()
    w = (torch.randn(136, 96, generator=g) * 0.2).to(dtype).cuda()
    out = torch.empty(rows, 136, dtype=dtype, device="cuda")
    kernels.linear(out, a, kernels.for_decode(w), activation="relu2")
    want = torch.relu(a.double().cpu() @ w.double().cpu().t()) ** 2
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    with pytest.raises(ValueError, match="activation"):
        kernels.linear(out, a, w, activation="swish")


def test_the_mixer_alone_and_the_feed_forward_alone(tmp_path):
    """One layer without feed-forward (the mixer with shift, scale and norm), and the same with
    one: the difference is the feed-forward's half."""
    for ff in (None, 48):
        config = _config(64, 90, [_layer(_mixer(2, 1, 32, window=12, keep_first=2), ff)], alpha=0.5, scale=2.0)
        weights = plain.random_weights(config, 11, sharp=3.0)
        folder = _folder(str(tmp_path / f"ff{ff}"), config, weights)
        tokens = helpers.random_tokens(60, 90, seed=2)
        got = _run(_engine(folder, "float32", 8), "r", tokens, [60])
        _close(got, plain.forward(weights, config, tokens), "float32", f"one layer, ff={ff}")


# -- the tests' weights show what they are meant to show ---------------------------------


@pytest.mark.parametrize("name", ["A", "B", "F"])
def test_the_plain_side_notices_a_window_a_kept_token_and_a_shift(models, name):
    """With these weights a window one token off, a kept token left out or a missing shift move
    the logits by hundreds of times the float32 tolerance: the comparisons below would show them."""
    _, config, weights = models[name]
    tokens = helpers.random_tokens(120, config["vocab"], seed=1)
    base = plain.forward(weights, config, tokens)
    scale = base.abs().max().item()

    def moved(change):
        c, w = copy.deepcopy(config), dict(weights)
        change(c, w)
        return (plain.forward(w, c, tokens) - base)[60:].abs().max().item() / scale

    def window(c, w):
        for entry in c["layers"]:
            if "mask" in entry["mixer"]:
                entry["mixer"]["mask"]["size"] += 1

    def kept(c, w):
        for entry in c["layers"]:
            if entry["mixer"].get("mask", {}).get("keep_first", 0) > 0:
                entry["mixer"]["mask"]["keep_first"] -= 1

    def shift(c, w):
        w["l0.shift"] = torch.zeros_like(w["l0.shift"])

    for change in (window, kept, shift):
        assert moved(change) > 300 * TOL["float32"], change.__name__


# -- whole, decoded, portions ----------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n", [("A", 200), ("B", 150), ("F", 300), ("X", 310)])
def test_whole_decoded_and_portions(models, dtype, name, n):
    folder, config, weights = models[name]
    tokens = helpers.random_tokens(n, config["vocab"], seed=n)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=(n + 15) // 16 + 2)
    _close(_run(eng, "whole", tokens, [n]), want, dtype, "whole")
    # most of it at once, then token by token until every window has passed over decoded tokens
    _close(_run(eng, "decoded", tokens, [n - 90] + [1] * 90), want, dtype, "last 90 one by one")
    _close(_run(eng, "portions", tokens, helpers.cuts_changing(n)), want, dtype, "portions of changing size")
    _close(_run(eng, "twos", tokens[:64], [2] * 32), want[:64], dtype, "portions of two tokens")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decode(models, dtype):
    """Every token one by one from the first, up to the model's last position (recorded decode
    steps replayed, the window and the kept first tokens passing page borders)."""
    folder, config, weights = models["A"]
    n = config["max_positions"]
    tokens = helpers.random_tokens(n, config["vocab"], seed=77)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=n // 16)
    got = _run(eng, "r", tokens, [1] * n)
    _close(got[:8], want[:8], dtype, "first tokens")
    _close(got, want, dtype, "decoding every token")


@pytest.mark.parametrize("page_size", [16, 32])
def test_windows_give_pages_back_and_stale_pages_do_not_matter(models, page_size):
    """A pool too small for the whole sequence: the windows' passed pages are used again (the kept
    first tokens' never), and what freed pages hold is never read."""
    folder, config, weights = models["A"]
    n = 250
    tokens = helpers.random_tokens(n, config["vocab"], seed=5)
    want = _plain(weights, config, tokens, "float32")
    # the widest window is 40 and 5 tokens are kept: far fewer pages than 250 tokens' worth
    eng = _engine(folder, "float32", n_pages=8 * 16 // page_size, page_size=page_size)
    from mlx_lm_amd.engine import StepEntry

    eng.add_request("r")
    rows, i = [], 0
    for c in [30, 2, 17] + [1] * 60 + [9, 20, 11] + [1] * 101:
        rows.append(eng.step([StepEntry("r", tokens[i : i + c], list(range(c)))]).clone())
        i += c
        eng.cache.poison_free_pages()
    assert i == n
    _close(torch.cat(rows), want, "float32", "a pool smaller than the sequence")
    rc = eng.cache.requests["r"]
    for gi, g in enumerate(eng.cache.groups):
        kept_blocks = (g.need.keep_first + page_size - 1) // page_size
        assert all(p >= 0 for p in rc.blocks[gi][:kept_blocks])
        assert any(p < 0 for p in rc.blocks[gi])
    eng.end_request("r")
    eng.cache.check()


# -- batches -------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "F", "X"])
def test_mixed_batches_equal_each_request_alone(models, dtype, name):
    """Up to four live requests of unequal lengths, portions beside single tokens, requests that
    sit a step out; slots and pages of finished requests are used again by later ones."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models[name]
    lengths = [70, 9, 131, 40, 3, 97, 55]
    cfg = {"vocab_size": config["vocab"]}
    tokens, steps = helpers.mixed_trace(cfg, 21, lengths, n_live=4)
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
        _close(torch.cat(got[rid]), _plain(weights, config, toks, dtype), dtype, f"request {rid} in mixed batches")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "F"])
def test_twenty_requests_decode_together(models, dtype, name):
    """Twenty requests of unequal lengths, each read alone, then decoded together for a dozen steps
    (between 17 and 64 rows a step: the products' rows travel in the packed order in bfloat16)."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models[name]
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


def _drawn_config(seed):
    """A configuration drawn from the seed: every size, the layers' order, windows and constants."""
    g = torch.Generator().manual_seed(seed)

    def pick(options):
        return options[int(torch.randint(0, len(options), (), generator=g))]

    own = []
    for _ in range(pick([1, 2, 3])):
        kv_heads = pick([1, 2, 3])
        heads = kv_heads * pick([1, 2, 4])
        dim = pick([4, 8, 12, 16, 24, 32, 40, 64, 72, 128, 160])
        if (heads * dim) % 8:
            dim *= 2
        window = pick([None, 1, 7, 16, 33, 64, 100, 1000])
        keep = pick([0, 0, 1, 5, 16, 17, 50]) if window else 0
        own.append(_layer(_mixer(heads, kv_heads, dim, window, keep, scale=pick([None, 0.05, 0.4])), pick([None, 8, 44, 96, 200])))
    layers = list(own)
    for _ in range(pick([0, 1, 3])):
        j = pick(list(range(len(own))))
        layers.insert(pick(list(range(len(own), len(layers) + 1))), dict(copy.deepcopy(own[j]), weights_of=j))
    return _config(pick([16, 40, 64, 104, 256]), pick([17, 100, 257, 1000]), layers, max_positions=pick([160, 200, 512]),
                   alpha=pick([0.5, 1.0, 2.5, 4.0]), scale=pick([1.0, 8.0, 0.3]), eps=pick([1e-6, 1e-5, 1e-2]))


@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed):
    """Ten drawn configurations (layers of several shapes in one model, so several cache groups;
    layers run again with a cache of their own) in mixed batches with few pages, against each
    request alone on the plain side: float32 all, bfloat16 every other one."""
    from mlx_lm_amd.engine import StepEntry

    config = _drawn_config(seed)
    weights = plain.random_weights(config, 50 + seed, sharp=2.0)
    folder = _folder(str(tmp_path / "m"), config, weights)
    lengths = [n for n in [70, 9, 131, 40, 3, 97] if n <= config["max_positions"]]
    tokens, steps = helpers.mixed_trace({"vocab_size": config["vocab"]}, seed, lengths, n_live=3)
    for dtype in ["float32"] + (["bfloat16"] if seed % 2 == 0 else []):
        eng = _engine(folder, dtype, n_pages=helpers.held(lengths, 3) // 16, max_requests=3)
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
            _close(torch.cat(got[rid]), _plain(weights, config, toks, dtype), dtype, f"seed {seed}: request {rid} ({config['layers']})")
        eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_thousands_of_keys(tmp_path, dtype):
    """A prompt of 3,300 tokens in two portions, then 40 decoded tokens beside a short request:
    layers without a window (a decoded row's keys are split over blocks, in the kernel that
    streams keys through registers and in the general one), a window of 1,500 that keeps 40, and
    a short window far from the start.  (That a single far key counts is the kernels' own test.)"""
    from mlx_lm_amd.engine import StepEntry

    config = _config(64, 120, [_layer(_mixer(2, 1, 64), 48), _layer(_mixer(4, 2, 24, window=1500, keep_first=40)),
                               _layer(_mixer(2, 2, 48)), _layer(_mixer(2, 1, 64, window=70, keep_first=130), 48)],
                     max_positions=3400, alpha=1.3, scale=4.0)
    weights = plain.random_weights(config, 31, sharp=3.0)
    folder = _folder(str(tmp_path / "long"), config, weights)
    n, n_prompt = 3340, 3300
    tokens = helpers.random_tokens(n, config["vocab"], seed=31)
    short = helpers.random_tokens(60, config["vocab"], seed=32)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=(n + 15) // 16 + 6)
    eng.add_request("long")
    eng.add_request("short")
    rows = [eng.step([StepEntry("long", tokens[:2000], [1999])]).clone(),
            eng.step([StepEntry("long", tokens[2000:n_prompt], [n_prompt - 2001]), StepEntry("short", short[:20], [])])[:1].clone()]
    _close(torch.cat(rows), want[[1999, n_prompt - 1]], dtype, "the prompt's portions")
    got, got_short = [], []
    for i in range(n - n_prompt):
        logits = eng.step([StepEntry("long", [tokens[n_prompt + i]], [0]), StepEntry("short", [short[20 + i]], [0])]).clone()
        got.append(logits[0])
        got_short.append(logits[1])
    _close(torch.stack(got), want[n_prompt:], dtype, "decoding at 3,300 keys")
    _close(torch.stack(got_short), _plain(weights, config, short, dtype)[20:], dtype, "the short request beside it")
    assert eng.stats.key_splits_most > 1  # a row's keys did go over several blocks


def test_recorded_steps_equal_eager_steps(models):
    """Decode steps replayed from recorded graphs against the same steps run eagerly, bit for bit
    (the shift's state is read and written once a step either way)."""
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
        tokens.append(int(plain.forward(weights, config, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_scheduler(models):
    from mlx_lm_amd import batch_generate, load, stream_generate

    folder, config, weights = models["B"]
    model, tok = load(folder, dtype="float32")
    prompts = [helpers.random_tokens(n, config["vocab"], seed=n) for n in (23, 5, 61)]
    want = [_greedy(weights, config, p, 10) for p in prompts]
    got = [r.token for r in stream_generate(model, tok, prompts[0], max_tokens=10, prefill_step_size=7)]
    assert got == want[0]
    batch = batch_generate(model, tok, prompts, max_tokens=10)
    assert [[int(t) for t in text.split()] for text in batch.texts] == want


def test_command_line(models):
    """``python -m mlx_lm_amd generate`` on a Pafutar folder: the tokens the plain side generates,
    also with a small pool of pages that the windows free as they pass."""
    folder, config, weights = models["A"]
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]
    want = _greedy(weights, config, prompt, 40)
    env = dict(os.environ, PYTHONPATH=ROOT)
    for extra in ([], ["--num-pages", "6", "--prefill-step-size", "3"]):
        out = subprocess.run(
            [sys.executable, "-m", "mlx_lm_amd", "generate", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)),
             "--max-tokens", "40", "--dtype", "float32", "--verbose", "F"] + extra,
            capture_output=True, text=True, env=env, timeout=300)
        assert out.returncode == 0, out.stderr[-2000:]
        assert out.stdout.strip() == " ".join(map(str, want))


def test_trace_replay_of_a_random_model(tmp_path, models):
    """The replay program on a configuration with seeded random weights: logits files per step."""
    _, config, _ = models["A"]
    json.dump(config, open(tmp_path / "config.json", "w"))
    tokens = helpers.random_tokens(50, config["vocab"], seed=9)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:31], "want": [30]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": tokens[31:], "want": "all"}], "end": ["x"]}]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--config", str(tmp_path / "config.json"),
                           "--seed", "4", "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "done 0" in proc.stdout and "done 1" in proc.stdout
    from mlx_lm_amd.config.registry import get_model_classes

    model_cls, args_cls = get_model_classes(config)
    weights = model_cls.random_weights(args_cls.from_dict(config), 4, "b")
    want = plain.forward(weights, config, tokens)
    got = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, config["vocab"])
    _close(torch.from_numpy(got), want[31:], "float32", "the replay's second step")


# -- the attention kernels with the optional score terms, each against the plain formulas ------


def _paged(keys, values, page_size, dtype, seed):
    """Keys and values ``[n, G, d]`` in pages handed out in a shuffled order; the rest holds NaN."""
    from mlx_lm_amd.ops.kernels import PagedKV

    n, G, d = keys.shape
    n_blocks = (n + page_size - 1) // page_size
    order = torch.randperm(n_blocks + 3, generator=torch.Generator().manual_seed(seed))[:n_blocks]
    both = torch.full((n_blocks + 3, 2, G, page_size, d), float("nan"), dtype=dtype, device="cuda")
    for b in range(n_blocks):
        rows = slice(b * page_size, min(n, (b + 1) * page_size))
        m = rows.stop - rows.start
        both[order[b], 0, :, :m] = keys[rows].permute(1, 0, 2).to(dtype)
        both[order[b], 1, :, :m] = values[rows].permute(1, 0, 2).to(dtype)
        both[order[b], :, :, m:] = 0  # (rows of a page that are not written yet hold numbers)
    return PagedKV(both[:, 0], both[:, 1]), order.to(torch.int32).cuda()[None].contiguous()


@pytest.mark.parametrize("kernel,dtype,d", [("tile", torch.float32, 48), ("tile", torch.bfloat16, 24), ("row", torch.float32, 40),
                                            ("row", torch.bfloat16, 80), ("prefill", torch.bfloat16, 64),
                                            ("prefill", torch.bfloat16, 128), ("prefill", torch.bfloat16, 32),
                                            ("decode", torch.bfloat16, 64), ("decode", torch.float32, 64),
                                            ("decode", torch.bfloat16, 128)])
@pytest.mark.parametrize("window,keep_first", [(0, 0), (50, 0), (50, 7), (37, 70), (300, 21)])
def test_attention_kernels_with_score_terms(kernel, dtype, d, window, keep_first):
    """Queries at positions 530 .. of a request that holds 530 + n keys: temperatures, distance
    slopes, a window with kept first keys (more of them than a page or a tile, or fewer than the
    window leaves behind) and the gate, against softmax((q.k) c_h - m_h (i - j)) v * sigmoid(g)."""
    from mlx_lm_amd.ops import kernels

    H, G, offset = 4, 2, 530
    n_q = {"tile": 16, "row": 3, "prefill": 150, "decode": 3}[kernel]
    n = offset + n_q
    g = torch.Generator().manual_seed(d + window + keep_first)
    q = torch.randn(n_q, H, d, generator=g).to(dtype)
    k = torch.randn(n, G, d, generator=g).to(dtype)
    v = torch.randn(n, G, d, generator=g).to(dtype)
    gate = torch.randn(n_q, H * d, generator=g).to(dtype)
    temp = torch.rand(H, generator=g) * 2.0 / d**0.5 + 0.5 / d**0.5  # scores with a spread of a few units
    # Keys that stand out for the first query's last head (the one with the gentlest slope): the
    # last kept key and the one after it, the key just inside the window and the one just outside.
    # Taken for the wrong side of its edge, any of them moves the output by about its value.
    if window:
        edges = [(offset - window, 1.2), (offset - window + 1, 1.2)]
        edges += [(keep_first - 1, 1.8), (keep_first, 1.8)] if keep_first else []  # (far away: the slope takes more off)
        for j, factor in edges:
            if 0 <= j < n:
                k[j, G - 1] = (q[0, H - 1].float() * factor).to(dtype)
    else:
        k[2, G - 1] = (q[0, H - 1].float() * 1.8).to(dtype)  # one key far back, among hundreds
    slopes = plain.head_slopes(H).float()
    # the plain side: scores with scale 1 and the heads' temperatures, the mask, the gate
    s = plain.attention_scores(q.double(), k.double(), 1.0, temp.double(), offset)
    see = plain.visible(n_q, offset, window if window else n + 1, keep_first)[:, :n]
    p = torch.softmax(s.masked_fill(~see.unsqueeze(0), float("-inf")), dim=-1)
    want = torch.einsum("hij,jhd->ihd", p, v.double().repeat_interleave(H // G, dim=1)).reshape(n_q, H * d)
    want = want * torch.sigmoid(gate.double())
    if window and keep_first:
        assert p[H - 1, 0, keep_first - 1] > 0.1  # the first query leans on the last kept key
    if not window:
        assert p[H - 1, 0, 2] > 0.1  # and on the far key

    kv, table = _paged(k, v, 16, dtype, seed=d)
    qd = q.reshape(n_q, H * d).cuda()
    out = torch.empty_like(qd)
    zeros = torch.zeros(n_q, dtype=torch.int32, device="cuda")
    positions = (torch.arange(n_q, dtype=torch.int32) + offset).cuda()
    terms = kernels.ScoreTerms(temp.cuda(), slopes.cuda(), gate.cuda(), keep_first)
    rows = torch.arange(n_q, dtype=torch.int32).cuda()
    if kernel == "tile":
        tiles = torch.tensor([[0, n_q]], dtype=torch.int32).cuda()
        kernels.attn_tile(out, qd, kv, table, zeros, positions, tiles, 1, H, 1.0, window, terms)
    elif kernel == "prefill":
        tiles = torch.tensor([[128, n_q - 128], [0, 128]], dtype=torch.int32).cuda()
        kernels.attn_prefill(out, qd, kv, table, zeros, positions, tiles, 2, H, 1.0, window, terms)
    else:
        n_splits = 3
        part_o = torch.empty(n_q * H * n_splits * d, device="cuda")
        part_ml = torch.empty(n_q * H * n_splits * 2, device="cuda")
        if kernel == "row":
            kernels.attn_row(out, qd, kv, table, zeros, positions, rows, n_q, H, 1.0, window, n_splits, part_o, part_ml, terms)
        else:
            kernels.attn_decode(out, qd, kv, table, zeros, positions, rows, n_q, H, 1.0, window, n_splits, part_o, part_ml,
                                n_waves=4, join_in_kernel=2, terms=terms)
    err = (out.double().cpu() - want).abs().max().item()
    assert err <= (2e-5 if dtype == torch.float32 else 2.5e-2) * want.abs().max().item(), err
