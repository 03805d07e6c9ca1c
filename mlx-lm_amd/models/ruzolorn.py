"""Ruzolorn: arguments, plan, tensor names, random weights.

A decoder-only design whose layers norm their sublayers on both sides and mix tokens in one of
two ways.  Token embedding times a constant, no position table; layers ``h += m * LN(mixer(LN(h)));
h += m * LN(ff(LN(h)))`` with LayerNorms without bias and a constant ``m``; a final LayerNorm and
an untied head.  Mixers:

* ``retention``: linear attention with a fixed decay per head, rotated queries and keys, a
  unit-RMS output per head and a silu gate (``parts/linear_state.py:Retention``);
* ``parallel``: two mixers on the same input, summed with two constants: softmax attention over a
  sliding window with grouped key heads, RMS-normed queries and keys and values of their own
  width (``attention`` with the ``head_rmsnorm`` hook), beside a selective state space
  (``state_space``).

The feed-forward is a mixture of gated experts chosen per token, with identity experts and a
shared expert (``gated_experts``); a layer may have none.

config.json names the design under ``architecture`` and gives every size and constant: ``vocab``,
``width``, ``embedding.scale``, ``norm.eps``, ``residual_mult`` and ``layers``, a list of ``{"type":
"retention" | "parallel", "mixer": {...}, "mlp": {"kind": "moe", "expert": {ff}, "router":
{experts, identity, top}, "shared": {ff} or null} or null}``; ``max_positions`` is optional (the
design has no table that bounds it).  Tensors: ``embed``, ``l<i>.norm1``, ``norm1b``, ``norm2``,
``norm2b``, ``l<i>.mix.{q,k,v,g,o}`` or ``l<i>.mix.left.{q,k,v,q.norm,k.norm,o}`` and
``l<i>.mix.right.{in,conv,conv.b,dt_bias,A_log,D,norm,o}``, ``l<i>.mlp.e<j>.{gate,up,down}``,
``l<i>.mlp.{router,correction}``, ``l<i>.mlp.shared.{gate,up,down}``, ``final.norm``, ``head``;
linear weights ``[out, in]``.
"""

from dataclasses import dataclass, field
from typing import Any, Dict, List

import torch

from ..config.base import BaseModelArgs
from ..config.plan import LayerSpec, ModelPlan, PartSpec, RunEntry
from ..parts.model import DecoderModel

MIXERS = ("retention", "parallel")
FEED_FORWARDS = ("moe",)
DEFAULT_POSITIONS = 1 << 15  # nothing in the design bounds a sequence; the cache's tables need a bound


def _padded_head(dim, vdim):
    """The head size that the attention kernels and the cache see: the wider of keys and values,
    rounded up to a multiple of 16."""
    return (max(dim, vdim) + 15) // 16 * 16


@dataclass
class ModelArgs(BaseModelArgs):
    """Keys of a Ruzolorn config.json; what the engine cannot run is refused here."""

    architecture: str
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    embedding: Dict[str, Any] = field(default_factory=dict)
    norm: Dict[str, Any] = field(default_factory=dict)
    residual_mult: float = 1.0
    max_positions: int = DEFAULT_POSITIONS

    def __post_init__(self):
        for key in ("vocab", "width", "max_positions"):
            if not isinstance(getattr(self, key), int) or getattr(self, key) <= 0:
                raise ValueError(f"{key} must be a positive integer, got {getattr(self, key)!r}")
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        if "eps" not in self.norm:
            raise ValueError("norm.eps is missing")
        for i, entry in enumerate(self.layers):
            if entry.get("type") not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {entry.get('type')!r} is not implemented (known: {MIXERS})")
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind") not in FEED_FORWARDS:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not implemented (known: {FEED_FORWARDS})")
            m = entry["mixer"]
            if entry["type"] == "parallel":
                left = m["left"]
                if _padded_head(left["dim"], left["vdim"]) > 256:
                    raise ValueError(f"layer {i}: attention heads of {left['dim']} / {left['vdim']} columns (at most 256)")

    @property
    def eps(self):
        return float(self.norm["eps"])

    @property
    def embedding_scale(self):
        return float(self.embedding.get("scale", 1.0))


class Model:
    """The Ruzolorn model: a ``DecoderModel`` built from the plan below."""

    def __init__(self, args: ModelArgs):
        self.args = args
        self.model_type = "ruzolorn"
        self.decoder = DecoderModel(self.plan(args))

    @property
    def layers(self):
        return self.decoder.layers

    @staticmethod
    def mixer_spec(args, entry, p):
        D, eps, m = args.width, args.eps, entry["mixer"]
        if entry["type"] == "retention":
            rot = m.get("rot") or {}
            return PartSpec("retention", {
                "width": D, "n_heads": m["heads"], "key_dim": m["dim"], "value_dim": m.get("vdim", m["dim"]),
                "decay": list(m["decay"]), "eps": eps, "rot_dims": int(rot.get("dims", 0)),
                "rot_base": float(rot.get("base", 10000.0))}, p)
        left, right = m["left"], m["right"]
        dim, vdim = left["dim"], left.get("vdim", left["dim"])
        head = _padded_head(dim, vdim)
        window = int((left.get("mask") or {}).get("size", 0))
        if window >= args.max_positions:
            window = 0  # (every key is inside such a window)
        attention = PartSpec("attention", {
            "width": D, "n_heads": left["heads"], "n_kv_heads": left.get("kv_heads", left["heads"]), "head_dim": head,
            "key_dim": dim, "value_dim": vdim, "scale": left.get("scale", dim ** -0.5), "window": window, "bias": False,
            "split_names": ("q", "k", "v", "o"),
            "position": PartSpec("head_rmsnorm", {"dim": dim, "head_stride": head, "eps": eps}, p + "left.")},
            p + "left.")
        space = PartSpec("state_space", {
            "width": D, "n_heads": right["heads"], "value_dim": right["vdim"], "state": right["state"],
            "groups": right.get("groups", 1), "taps": right["conv"], "norm_groups": right.get("norm_groups", 1),
            "eps": eps}, p + "right.")
        return PartSpec("parallel", {"left": attention, "right": space, "left_scale": m.get("left_scale", 1.0),
                                     "right_scale": m.get("right_scale", 1.0)}, p)

    @staticmethod
    def plan(args: ModelArgs) -> ModelPlan:
        D, eps = args.width, args.eps

        def norm(name):
            return PartSpec("layernorm", {"width": D, "eps": eps, "bias": False, "weight_name": name})

        layers, schedule, slot = [], [], 0
        for i, entry in enumerate(args.layers):
            p = f"l{i}."
            parts = dict(mixer_norm=norm(p + "norm1"), mixer=Model.mixer_spec(args, entry, p + "mix."),
                         mixer_post_norm=norm(p + "norm1b"))
            mlp = entry.get("mlp")
            if mlp is not None:
                router, shared = mlp["router"], mlp.get("shared") or {}
                parts["ffn_norm"], parts["ffn_post_norm"] = norm(p + "norm2"), norm(p + "norm2b")
                parts["ffn"] = PartSpec("gated_experts", {
                    "width": D, "n_experts": router["experts"], "inner": (mlp.get("expert") or {}).get("ff", 0),
                    "top": router["top"], "n_identity": router.get("identity", 0),
                    "shared_inner": shared.get("ff", 0)}, p + "mlp.")
            layers.append(LayerSpec("sandwich", parts, {"residual_mult": args.residual_mult}))
            # a parallel layer keeps pages (its attention) and state (its state space): two slots
            if entry["type"] == "parallel":
                schedule.append(RunEntry(layer=i, cache=slot, state=slot + 1))
                slot += 2
            else:
                schedule.append(RunEntry(layer=i, cache=slot))
                slot += 1
        return ModelPlan(
            width=D, vocab_size=args.vocab, max_positions=args.max_positions,
            embedding=PartSpec("token", {"vocab_size": args.vocab, "width": D, "weight_name": "embed",
                                         "scale": args.embedding_scale}),
            embedding_positions=None, layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("linear", {"vocab_size": args.vocab, "width": D, "weight_name": "head"}))

    def sanitize(self, weights):
        return dict(weights)

    @staticmethod
    def random_weights(args: ModelArgs, seed, scheme="a"):
        """Seeded tensors under the checkpoint's names.  Scheme ``a``: norm weights 1, corrections
        and biases 0, ``D`` 1.  Scheme ``b``: all of them drawn."""
        if scheme not in ("a", "b"):
            raise ValueError(f"unknown random-weight scheme '{scheme}'")
        g = torch.Generator().manual_seed(int(seed))
        D = args.width

        def normal(shape, std, mean=0.0):
            return torch.randn(shape, generator=g, dtype=torch.float32) * std + mean

        def vector(n, mean, std):
            return normal((n,), std, mean) if scheme == "b" else torch.full((n,), float(mean))

        t = {"embed": normal((args.vocab, D), 1.0)}
        for i, entry in enumerate(args.layers):
            p, m = f"l{i}.", entry["mixer"]
            t[p + "norm1"], t[p + "norm1b"] = vector(D, 1.0, 0.1), vector(D, 1.0, 0.1)
            if entry["type"] == "retention":
                qk, vw = m["heads"] * m["dim"], m["heads"] * m.get("vdim", m["dim"])
                for name, n in (("q", qk), ("k", qk), ("v", vw), ("g", vw)):
                    t[p + "mix." + name] = normal((n, D), D ** -0.5)
                t[p + "mix.o"] = normal((D, vw), vw ** -0.5)
            else:
                left, right, q = m["left"], m["right"], p + "mix.left."
                H, G, d, dv = left["heads"], left.get("kv_heads", left["heads"]), left["dim"], left.get("vdim", left["dim"])
                t[q + "q"], t[q + "k"] = normal((H * d, D), D ** -0.5), normal((G * d, D), D ** -0.5)
                t[q + "v"], t[q + "o"] = normal((G * dv, D), D ** -0.5), normal((D, H * dv), (H * dv) ** -0.5)
                t[q + "q.norm"], t[q + "k.norm"] = vector(d, 1.0, 0.1), vector(d, 1.0, 0.1)
                r = p + "mix.right."
                Hs, P, N, Gs = right["heads"], right["vdim"], right["state"], right.get("groups", 1)
                inner, C = Hs * P, Hs * P + 2 * Gs * N
                t[r + "in"] = normal((2 * inner + 2 * Gs * N + Hs, D), D ** -0.5)
                t[r + "conv"], t[r + "conv.b"] = normal((C, right["conv"]), right["conv"] ** -0.5), vector(C, 0.0, 0.1)
                t[r + "dt_bias"], t[r + "A_log"] = vector(Hs, 0.0, 0.5), normal((Hs,), 0.5, -1.0)
                t[r + "D"], t[r + "norm"] = vector(Hs, 1.0, 0.2), vector(inner, 1.0, 0.1)
                t[r + "o"] = normal((D, inner), inner ** -0.5)
            mlp = entry.get("mlp")
            if mlp is not None:
                q, router = p + "mlp.", mlp["router"]
                t[p + "norm2"], t[p + "norm2b"] = vector(D, 1.0, 0.1), vector(D, 1.0, 0.1)
                F = (mlp.get("expert") or {}).get("ff", 0)
                for e in range(router["experts"]):
                    t[f"{q}e{e}.gate"], t[f"{q}e{e}.up"] = normal((F, D), D ** -0.5), normal((F, D), D ** -0.5)
                    t[f"{q}e{e}.down"] = normal((D, F), F ** -0.5)
                n_out = router["experts"] + router.get("identity", 0)
                t[q + "router"], t[q + "correction"] = normal((n_out, D), D ** -0.5), vector(n_out, 0.0, 0.02)
                Fs = (mlp.get("shared") or {}).get("ff", 0)
                if Fs:
                    t[q + "shared.gate"], t[q + "shared.up"] = normal((Fs, D), D ** -0.5), normal((Fs, D), D ** -0.5)
                    t[q + "shared.down"] = normal((D, Fs), Fs ** -0.5)
        t["final.norm"] = vector(D, 1.0, 0.1)
        t["head"] = normal((args.vocab, D), D ** -0.5)
        return t
