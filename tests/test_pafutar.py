"""Pafutar without a GPU: the registry, the arguments and the plan, the pages of kept first tokens,
and the plain implementation's own mask."""

import pytest
import torch

import plain_pafutar as plain
from mlx_lm_amd.cache import CacheManager
from mlx_lm_amd.config import CacheNeed, StateNeed, get_model_classes


def _config(layers, **kw):
    c = {"architecture": "Pafutar", "vocab": 50, "width": 32, "max_positions": 128, "embedding": {"scale": 2.0},
         "norm": {"eps": 1e-5}, "postln_alpha": 1.5, "layers": layers}
    c.update(kw)
    return c


def _layer(window=None, keep_first=0, ff=40, **kw):
    m = {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25}
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return dict({"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}, **kw)


def test_the_design_is_found_by_its_architecture_key_and_planned_run_by_run():
    config = _config([_layer(20, 3), _layer(ff=None), _layer(20, 3, weights_of=0), _layer(200)])
    model_cls, args_cls = get_model_classes(config)
    model = model_cls(args_cls.from_dict(config))
    dec = model.decoder
    assert len(dec.layers) == 3 and [r.layer for r in dec.schedule] == [0, 1, 0, 2]
    assert [r.cache for r in dec.schedule] == [0, 1, 2, 3] and [r.state for r in dec.schedule] == [4, 5, 6, 7]
    needs = dec.cache_needs()
    assert needs[0] == needs[2] == CacheNeed(1, 16, 20, 0, 3)
    assert needs[1] == CacheNeed(1, 16, 0, 0, 0)
    assert needs[3] == CacheNeed(1, 16, 0, 0, 0)  # a window as long as the model's positions is none
    assert needs[4:] == [StateNeed((32,), "float32")] * 4
    names = set(dec.expected_tensors())
    assert {"embed", "pos", "head", "final.norm", "l0.mix.q.b", "l0.mix.temp", "l0.ls2", "l0.shift", "l3.mlp.down"} <= names
    assert not any(n.startswith("l2.") for n in names)  # the second run of layer 0 has no tensors
    assert "l1.norm2" not in names and "l1.ls2" not in names and "l1.mlp.up" not in names
    weights = model_cls.random_weights(args_cls.from_dict(config), 1, "b")
    assert set(weights) == names and all(tuple(weights[n].shape) == tuple(s.shape) for n, s in dec.expected_tensors().items())


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="recurrent"), "mixer type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "feed-forward kind"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][1].update(weights_of=1), "weights_of"),
    (lambda c: c.update(norm={}), "eps"),
    (lambda c: c.update(width=0), "width"),
])
def test_what_cannot_run_is_refused(change, message):
    config = _config([_layer(20, 3), _layer(20, 3, weights_of=0)])
    change(config)
    model_cls, args_cls = get_model_classes(config)
    with pytest.raises(ValueError, match=message):
        model_cls(args_cls.from_dict(config))


def test_pages_of_the_kept_first_tokens_stay_while_the_window_gives_pages_back():
    cm = CacheManager([CacheNeed(1, 16, 24, 0, 20), CacheNeed(1, 16, 24, 0, 0)], page_size=16, n_pages=12, max_requests=2)
    assert len(cm.groups) == 2
    cm.add("r")
    for n in (50, 1, 1, 30, 1, 40, 1):
        cm.reserve("r", n)
        cm.commit("r", n)
        cm.check()
    kept, plain_window = cm.requests["r"].blocks
    length = cm.requests["r"].length
    first_needed = (length - 24 + 1) // 16
    assert all(p >= 0 for p in kept[:2]) and all(p < 0 for p in kept[2:first_needed]) and all(p >= 0 for p in kept[first_needed:])
    assert all(p < 0 for p in plain_window[:first_needed]) and all(p >= 0 for p in plain_window[first_needed:])
    cm.release("r")
    cm.check()
    assert cm.free_pages() == 12


def test_the_plain_mask():
    see = plain.visible(4, 10, window=3, keep_first=2)
    assert see.shape == (4, 14)
    for a in range(4):
        i = 10 + a
        assert [j for j in range(14) if see[a, j]] == [0, 1] + list(range(i - 2, i + 1))
    assert plain.visible(3, 0, window=100, keep_first=0).tolist() == torch.tril(torch.ones(3, 3)).bool().tolist()
    assert torch.allclose(plain.head_slopes(4), torch.tensor([0.25, 0.0625, 0.015625, 0.00390625], dtype=torch.float64))


def test_the_plain_side_token_by_token_equals_whole_sequences():
    """The plain implementation's mechanisms are causal: the logits at a position do not change
    when later tokens are added (what lets the engine's portions be compared with whole runs)."""
    config = _config([_layer(9, 2), _layer(ff=None), _layer(9, 2, weights_of=0)])
    weights = plain.random_weights(config, 2)
    tokens = torch.randint(0, 50, (40,), generator=torch.Generator().manual_seed(0)).tolist()
    whole = plain.forward(weights, config, tokens)
    assert torch.allclose(plain.forward(weights, config, tokens[:23])[-1], whole[22], atol=1e-10)
