"""Ruzolorn without a GPU: the registry, the plan layer by layer, refusals, and the plain side."""

import copy

import pytest
import torch

import plain_ruzolorn as plain
from mlx_lm_amd.config import CacheNeed, StateNeed
from mlx_lm_amd.config.registry import get_model_classes

CONFIG = {
    "architecture": "Ruzolorn", "vocab": 90, "width": 48, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
    "residual_mult": 0.5,
    "layers": [
        {"type": "parallel", "mixer": {
            "left": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 20, "scale": 0.3, "mask": {"size": 9}},
            "right": {"heads": 2, "vdim": 8, "state": 4, "groups": 1, "conv": 3, "norm_groups": 2},
            "left_scale": 1.1, "right_scale": 0.4},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "identity": 1, "top": 2}, "shared": {"ff": 12}}},
        {"type": "retention", "mixer": {"heads": 2, "dim": 8, "vdim": 16, "decay": [0.9, 0.99], "rot": {"dims": 4, "base": 100.0}},
         "mlp": None},
    ],
}


def _model(config):
    model_cls, args_cls = get_model_classes(config)
    return model_cls(args_cls.from_dict(config)), model_cls, args_cls


def test_the_registry_knows_the_design_by_its_architecture():
    model, _, _ = _model(CONFIG)
    assert model.model_type == "ruzolorn" and len(model.layers) == 2


def test_the_plan_layer_by_layer():
    model, _, _ = _model(CONFIG)
    dec = model.decoder
    needs = dec.cache_needs()
    # the parallel layer: pages for its attention (heads padded to the wider of keys and values,
    # a multiple of 16) and a state row (two convolution inputs of 24 channels, two heads of 4 x 8)
    assert needs[0] == CacheNeed(2, 32, 9) and needs[1] == StateNeed((2 * 24 + 2 * 4 * 8,), "float32")
    assert needs[2] == StateNeed((2 * 8 * 16,), "float32")
    assert [(r.layer, r.cache, r.state) for r in dec.schedule] == [(0, 0, 1), (1, 2, None)]
    first, second = dec.layers
    assert first.residual_mult == 0.5 and first.ffn is not None and second.ffn is None
    assert first.mixer.left.window == 9 and first.mixer.left.scale == 0.3 and first.mixer.left_scale == 1.1
    assert first.ffn.n_experts == 3 and first.ffn.n_identity == 1 and first.ffn.top == 2 and first.ffn.shared_inner == 12
    assert second.mixer.rot_dims == 4 and second.mixer.key_scale == 8 ** -0.5
    want = dec.expected_tensors()
    assert want["l0.mix.left.q"].shape == (48, 48) and want["l0.mix.left.v"].shape == (40, 48)
    assert want["l0.mix.left.q.norm"].shape == (12,) and want["l0.mix.right.in"].shape == (2 * 16 + 2 * 4 + 2, 48)
    assert want["l0.mix.right.conv"].shape == (24, 3) and want["l0.mlp.router"].shape == (4, 48)
    assert "l1.norm2" not in want and "l0.norm2b" in want and "pos" not in want


def test_random_weights_fit_the_plan():
    model, model_cls, args_cls = _model(CONFIG)
    tensors = model_cls.random_weights(args_cls.from_dict(CONFIG), 1, "b")
    want = model.decoder.expected_tensors()
    assert set(tensors) == set(want)
    assert all(tuple(tensors[k].shape) == tuple(v.shape) for k, v in want.items())


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="convolution"), "mixer type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "feed-forward kind"),
    (lambda c: c["norm"].clear(), "norm.eps"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.9]), "decays"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(groups=3), "grouped"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "experts a token"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "turning columns"),
])
def test_what_cannot_run_is_refused_with_a_message(change, message):
    config = copy.deepcopy(CONFIG)
    change(config)
    with pytest.raises(ValueError, match=message):
        _model(config)


def test_the_plain_side_is_causal_and_keeps_its_window():
    weights = plain.random_weights(CONFIG, 3, sharp=2.0)
    g = torch.Generator().manual_seed(0)
    tokens = torch.randint(0, 90, (40,), generator=g).tolist()
    base = plain.model(weights, CONFIG, tokens)
    other = list(tokens)
    other[30] = (other[30] + 1) % 90
    moved = (plain.model(weights, CONFIG, other) - base).abs().amax(-1)
    assert moved[:30].max() == 0 and moved[30] > 1e-3
    assert plain.window_mask(12, 3).sum(-1).tolist() == [1, 2] + [3] * 10
    assert plain.window_mask(5, 0).sum(-1).tolist() == [1, 2, 3, 4, 5]


def test_the_plain_convolution_and_the_state_spaces_two_forms():
    """The recurrence against the same sum written out: y_t = sum_j exp(sum of log decays after j)
    dt_j (C_t . B_j) x_j + D x_t."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 3, generator=g).double()
    w, b = torch.randn(3, 4, generator=g).double(), torch.randn(3, generator=g).double()
    y = plain.causal_conv(x, w, b)
    assert torch.allclose(y[0], b + w[:, 3] * x[0]) and torch.allclose(y[5], b + (w * x[2:6].T).sum(-1))
    m = {"heads": 1, "vdim": 2, "state": 3, "groups": 1, "conv": 1, "norm_groups": 1}
    t = {"in": torch.randn(2 * 2 + 6 + 1, 5, generator=g).double(), "conv": torch.ones(8, 1).double(), "conv.b": torch.zeros(8).double(),
         "dt_bias": torch.zeros(1).double(), "A_log": torch.tensor([-0.5]).double(), "D": torch.tensor([0.7]).double(),
         "norm": torch.ones(2).double(), "o": torch.eye(2).double()}
    h = torch.randn(7, 5, generator=g).double()
    got = plain.state_space(h, t, "", m, 1e-6)
    u = h @ t["in"].T
    z, xbc, dt = u[:, :2], plain.silu(u[:, 2:10]), plain.softplus(u[:, 10])
    xs, B, C = xbc[:, :2], xbc[:, 2:5], xbc[:, 5:8]
    la = -torch.exp(t["A_log"][0]) * dt
    want = []
    for i in range(7):
        acc = 0.7 * xs[i]
        for j in range(i + 1):
            acc = acc + torch.exp(la[j + 1 : i + 1].sum()) * dt[j] * (C[i] @ B[j]) * xs[j]
        want.append(acc)
    want = plain.unit_rms(torch.stack(want) * plain.silu(z), 1e-6)
    assert torch.allclose(got, want, atol=1e-10)
