"""Attention whose values are its keys, with normed queries and keys, biased by distance, gated."""

import ctypes

import torch

from ..config.plan import CacheNeed
from ..ops import kernels, native
from .attention import CausalSelfAttention
from .base import Mixer, TensorSpec, register_mixer, value_of


class GatedKeyAttention(Mixer):
    """``out = Wo (softmax(s) k * sigmoid(Wg x))`` over the paged cache, where

    * ``q = Wq x + bq`` and ``k = Wk x + bk``; the values are the keys as projected (no value
      projection), head ``h`` of ``n_heads`` reading key head ``h // (n_heads / n_kv_heads)``;
    * queries and keys are divided by their root mean square over a head (``eps`` inside the root);
    * ``s_ij = (q_i . k_j) * scale * temp[h] - slope_h * (i - j)`` with a learned temperature per
      head and ``slope_h = 2 ** (-slope_bits * (h + 1) / n_heads)``;
    * with ``window > 0`` position ``i`` sees ``j <= i`` where ``i - j < window`` or ``j <
      keep_first`` (the first tokens stay visible at their own positions); ``window = 0``: all.

    One product gives queries, keys and the gate's input; the cache keeps the normed keys in the
    key half of a page and the projected ones in the value half (csrc/gated_key_attention.hip).
    Norms, scores and the softmax are float32.  In an arrangement that sums its output itself
    (``post_norm``) the output projection writes float32 rows instead of adding to the stream.
    No counterpart in mlx_lm/models/gpt2.py, whose attention (:44-68) has neither.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, width, n_heads, head_dim, n_kv_heads=None, scale=None, window=0, keep_first=0, eps=1e-6,
                 slope_bits=8.0, names=("q", "k", "g", "o", "temp"), prefix=""):
        super().__init__(prefix)
        n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads cannot be grouped over {n_kv_heads} key heads")
        if head_dim % 4 or not (4 <= head_dim <= 256):
            raise ValueError(f"head_dim {head_dim} must be a multiple of 4 between 4 and 256")
        if width % 8 or (n_heads * head_dim) % 8:
            raise ValueError(f"width {width} and the heads' columns {n_heads * head_dim} must be multiples of 8")
        if window < 0 or keep_first < 0:
            raise ValueError(f"window {window} and keep_first {keep_first} must not be negative")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.scale = float(scale) if scale is not None else head_dim**-0.5
        self.window, self.keep_first = int(window), int(keep_first) if window else 0
        self.eps, self.slope_bits = float(eps), float(slope_bits)
        self.q_width, self.kv_width = n_heads * head_dim, n_kv_heads * head_dim
        self.names = dict(zip(("q", "k", "g", "o", "temp"), (self._name(n) for n in names)))
        self.qkg_w = self.qkg_b = self.out_w = self.head_scale = self.slopes = None

    def cache_need(self):
        return CacheNeed(self.n_kv_heads, self.head_dim, self.window, 0, self.keep_first)

    def tensors(self):
        n = self.names
        return {
            n["q"]: TensorSpec((self.q_width, self.width), "matrix"),
            n["q"] + ".b": TensorSpec((self.q_width,), "vector"),
            n["k"]: TensorSpec((self.kv_width, self.width), "matrix"),
            n["k"] + ".b": TensorSpec((self.kv_width,), "vector"),
            n["g"]: TensorSpec((self.q_width, self.width), "matrix"),
            n["o"]: TensorSpec((self.width, self.q_width), "matrix"),
            n["temp"]: TensorSpec((self.n_heads,), "vector"),
        }

    def load(self, tensors):
        n = self.names
        q_b, k_b = tensors[n["q"] + ".b"], tensors[n["k"] + ".b"]
        # one product for queries, keys and the gate's input: [q | k | g], the gate without a bias
        qkg = torch.cat([tensors[n["q"]], tensors[n["k"]], tensors[n["g"]]]).contiguous()
        self.qkg_b = torch.cat([q_b, k_b, q_b.new_zeros(self.q_width)]).contiguous()
        self.qkg_w, self.out_w = kernels.for_decode(qkg), kernels.for_decode(tensors[n["o"]])
        self.first_weight = self.qkg_w
        self.head_scale = (tensors[n["temp"]].double() * self.scale).float().contiguous()
        h = torch.arange(1, self.n_heads + 1, dtype=torch.float64)
        self.slopes = torch.pow(2.0, -self.slope_bits * h / self.n_heads).float().to(q_b.device).contiguous()

    # the work lists are the attention part's own: which rows go to which kernel
    step_arrays_key = CausalSelfAttention.step_arrays_key
    step_array_names = CausalSelfAttention.step_array_names
    step_arrays = staticmethod(CausalSelfAttention.step_arrays)
    length_class = staticmethod(CausalSelfAttention.length_class)

    def make_native(self):
        W, P, I, F = ctypes.POINTER(native.EngWeight), ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L = native.part_library("gated_key_attention",
                                {"make_gated_key_attention": [I, I, I, I, I, I, F, W, P, W, P, P, I]})
        base = native.array_ids(self.step_arrays_key, self.step_array_names)
        qkg_w, out_w = kernels.weight_struct(self.qkg_w), kernels.weight_struct(self.out_w)
        return native.made(L.make_gated_key_attention(
            native.host(), self.width, self.n_heads, self.n_kv_heads, self.head_dim, self.window, self.keep_first,
            self.eps, ctypes.byref(qkg_w), native.ptr(self.qkg_b), ctypes.byref(out_w), native.ptr(self.head_scale),
            native.ptr(self.slopes), base), "gated key attention")

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        v, r = value_of(x), native.mat(residual)
        with ctx.enter():
            rc = native.lib().eng_mixer_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(v),
                                                ctypes.byref(r), cache.slot, int(bool(writes_cache)))
        native.check(rc, "gated key attention")


register_mixer("gated_key_attention", GatedKeyAttention)
