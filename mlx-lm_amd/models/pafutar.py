"""Pafutar: arguments, plan, tensor names, random weights.

A decoder-only design of post-norm layers.  Token embedding times a constant plus a learned
position row; layers ``h = N(a h + ls1 * mixer(shift(h))); h = N(a h + ls2 * ff(h))`` with RMS
norms, per-column layer scales and a token shift ahead of the mixer; the mixer is
``gated_key_attention`` (values are the keys, unit-RMS queries and keys, a temperature per head, a
bias that grows with distance, a sliding window that keeps the first tokens, a sigmoid output
gate); the feed-forward is dense with a squared ReLU; a final RMS norm and an untied head.  A layer
may run with another layer's weights and a cache and state of its own.

config.json names the design under ``architecture`` and gives every size and constant:
``vocab``, ``width``, ``max_positions``, ``embedding.scale``, ``norm.eps``, ``postln_alpha`` and
``layers``, a list of ``{"type": "attention", "mixer": {heads, kv_heads, dim, vdim, scale,
mask: {size, keep_first}}, "mlp": {"kind": "dense", "ff": n} or null, "weights_of": j (optional)}``.
Tensors: ``embed``, ``pos``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.ls1``, ``l<i>.ls2``,
``l<i>.shift``, ``l<i>.mix.{q,q.b,k,k.b,temp,g,o}``, ``l<i>.mlp.{up,down}``, ``final.norm``, ``head``;
linear weights ``[out, in]``.
"""

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch

from ..config.base import BaseModelArgs
from ..config.plan import LayerSpec, ModelPlan, PartSpec, RunEntry
from ..parts.model import DecoderModel

MIXERS = ("attention",)
FEED_FORWARDS = ("dense",)


@dataclass
class ModelArgs(BaseModelArgs):
    """Keys of a Pafutar config.json; what the engine cannot run is refused here."""

    architecture: str
    vocab: int
    width: int
    max_positions: int
    layers: List[Dict[str, Any]]
    embedding: Dict[str, Any] = field(default_factory=dict)
    norm: Dict[str, Any] = field(default_factory=dict)
    postln_alpha: float = 1.0

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
            if m.get("vdim", m["dim"]) != m["dim"]:
                raise ValueError(f"layer {i}: the values are the keys, so vdim {m['vdim']} must equal dim {m['dim']}")
            if entry.get("weights_of") is not None:
                j = self.weights_layer(i)
                other = self.layers[j]
                if any(entry.get(k) != other.get(k) for k in ("type", "mixer", "mlp")):
                    raise ValueError(f"layer {i} runs with layer {j}'s weights but is described differently")

    def weights_layer(self, i):
        """The layer whose tensors layer ``i`` runs with: itself, or where its ``weights_of`` leads."""
        seen = set()
        while self.layers[i].get("weights_of") is not None:
            j = self.layers[i]["weights_of"]
            if not (isinstance(j, int) and 0 <= j < len(self.layers)) or i in seen:
                raise ValueError(f"layer {i}: weights_of {j!r} must lead to a layer that has weights of its own")
            seen.add(i)
            i = j
        return i

    @property
    def eps(self):
        return float(self.norm["eps"])

    @property
    def embedding_scale(self):
        return float(self.embedding.get("scale", 1.0))


class Model:
    """The Pafutar model: a ``DecoderModel`` built from the plan below."""

    def __init__(self, args: ModelArgs):
        self.args = args
        self.model_type = "pafutar"
        self.decoder = DecoderModel(self.plan(args))

    @property
    def layers(self):
        return self.decoder.layers

    @staticmethod
    def plan(args: ModelArgs) -> ModelPlan:
        D, eps = args.width, args.eps

        def norm(name):
            return PartSpec("rmsnorm", {"width": D, "eps": eps, "weight_name": name})

        own = [i for i, e in enumerate(args.layers) if e.get("weights_of") is None]  # the layers with tensors
        index = {i: n for n, i in enumerate(own)}
        layers = []
        for i in own:
            entry, p = args.layers[i], f"l{i}."
            m, mask = entry["mixer"], entry["mixer"].get("mask") or {}
            window = int(mask.get("size", 0))
            if window >= args.max_positions:
                window = 0  # (every key is inside such a window)
            parts = dict(
                mixer=PartSpec("gated_key_attention", {
                    "width": D, "n_heads": m["heads"], "n_kv_heads": m.get("kv_heads", m["heads"]),
                    "head_dim": m["dim"], "scale": m.get("scale", m["dim"] ** -0.5), "window": window,
                    "keep_first": int(mask.get("keep_first", 0)), "eps": eps}, p + "mix."),
                mixer_norm=norm(p + "norm1"))
            if entry.get("mlp") is not None:
                parts["ffn"] = PartSpec("relu2_mlp", {"width": D, "inner": entry["mlp"]["ff"]}, p + "mlp.")
                parts["ffn_norm"] = norm(p + "norm2")
            layers.append(LayerSpec("post_norm", parts, {"alpha": args.postln_alpha, "layer_scale": True,
                                                         "token_shift": True, "prefix": p}))
        # every entry of the config is a run, with a cache and a shift state of its own; a run with
        # ``weights_of`` is a second run of that layer
        n = len(args.layers)
        schedule = [RunEntry(layer=index[args.weights_layer(i)], cache=i, state=n + i) for i in range(n)]
        return ModelPlan(
            width=D, vocab_size=args.vocab, max_positions=args.max_positions,
            embedding=PartSpec("token", {"vocab_size": args.vocab, "width": D, "weight_name": "embed",
                                         "scale": args.embedding_scale}),
            embedding_positions=PartSpec("learned", {"max_positions": args.max_positions, "width": D,
                                                     "weight_name": "pos"}),
            layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("linear", {"vocab_size": args.vocab, "width": D, "weight_name": "head"}))

    def sanitize(self, weights):
        return dict(weights)

    @staticmethod
    def random_weights(args: ModelArgs, seed, scheme="a"):
        """Seeded tensors under the checkpoint's names.  Scheme ``a``: norm weights, layer scales
        and temperatures 1, biases 0, shifts 0.5.  Scheme ``b``: all of them drawn."""
        if scheme not in ("a", "b"):
            raise ValueError(f"unknown random-weight scheme '{scheme}'")
        g = torch.Generator().manual_seed(int(seed))
        D = args.width

        def normal(shape, std, mean=0.0):
            return torch.randn(shape, generator=g, dtype=torch.float32) * std + mean

        def vector(n, mean, std):
            return normal((n,), std, mean) if scheme == "b" else torch.full((n,), float(mean))

        t = {"embed": normal((args.vocab, D), 0.02), "pos": normal((args.max_positions, D), 0.02 * args.embedding_scale)}
        for i, entry in enumerate(args.layers):
            if entry.get("weights_of") is not None:
                continue
            p, m = f"l{i}.", entry["mixer"]
            qw, kw = m["heads"] * m["dim"], m.get("kv_heads", m["heads"]) * m["dim"]
            t[p + "norm1"] = vector(D, 1.0, 0.1)
            t[p + "mix.q"], t[p + "mix.q.b"] = normal((qw, D), D**-0.5), vector(qw, 0.0, 0.1)
            t[p + "mix.k"], t[p + "mix.k.b"] = normal((kw, D), D**-0.5), vector(kw, 0.0, 0.1)
            t[p + "mix.temp"] = vector(m["heads"], 1.0, 0.1)
            t[p + "mix.g"], t[p + "mix.o"] = normal((qw, D), D**-0.5), normal((D, qw), qw**-0.5)
            t[p + "ls1"], t[p + "shift"] = vector(D, 1.0, 0.1), vector(D, 0.5, 0.2).clamp(0.0, 1.0)
            if entry.get("mlp") is not None:
                F = entry["mlp"]["ff"]
                t[p + "norm2"], t[p + "ls2"] = vector(D, 1.0, 0.1), vector(D, 1.0, 0.1)
                t[p + "mlp.up"], t[p + "mlp.down"] = normal((F, D), D**-0.5), normal((D, F), F**-0.5)
        t["final.norm"] = vector(D, 1.0, 0.1)
        t["head"] = normal((args.vocab, D), D**-0.5)
        return t
