"""Position encodings."""

from ..ops import native
from .base import PositionEncoding, TensorSpec, register_position_encoding


class NoPositions(PositionEncoding):
    """Nothing is added and nothing is rotated."""

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, prefix=""):
        super().__init__(prefix)

    def make_native(self):
        return None  # no part at all


class LearnedPositions(PositionEncoding):
    """A learned table indexed by absolute position, added to the token embedding.

    ``h += wpe[arange(L) + offset]`` (mlx_lm/models/gpt2.py:121,137-144); the
    step's ``positions`` array already holds ``offset + i`` for every token.
    A position at or beyond the table's end is refused by the engine before
    anything runs (the reference does not check it).
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, max_positions, width, weight_name="weight", prefix=""):
        super().__init__(prefix)
        if max_positions <= 0:
            raise ValueError(f"max_positions must be positive, got {max_positions}")
        self.max_positions, self.width = max_positions, width
        self.weight_name = self._name(weight_name)
        self.table = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.max_positions, self.width), "matrix")}

    def load(self, tensors):
        self.table = tensors[self.weight_name]

    def reads_rows_of(self):
        """Tensors of which a step reads a row per token, not all."""
        return (self.weight_name,)

    def make_native(self):
        return native.made(native.lib().eng_make_learned_positions(
            self.table.data_ptr(), self.max_positions, self.width, native.DT[self.table.dtype]), "learned positions")

    def embedding_term(self, ctx):
        return self.table, ctx.positions


class HeadRMSNorm(PositionEncoding):
    """Queries and keys divided by their root mean square over a head and multiplied by a weight
    of ``dim`` values that all heads share (one for queries, one for keys), in place, ahead of the
    cache write: the hook that the attention part offers for what happens to queries and keys
    between their projection and the scores.  Positions do not enter.  Heads may lie
    ``head_stride`` columns apart (padded beyond ``dim``).  32-bit inside (csrc/head_norm.hip).
    No counterpart in mlx_lm/models/gpt2.py, whose attention (:44-68) norms neither.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, dim, eps, head_stride=None, q_name="q.norm", k_name="k.norm", prefix=""):
        super().__init__(prefix)
        self.dim, self.eps = int(dim), float(eps)
        self.head_stride = int(head_stride or dim)
        if not 0 < self.dim <= self.head_stride:
            raise ValueError(f"a head of {self.dim} columns does not fit a stride of {self.head_stride}")
        self.q_name, self.k_name = self._name(q_name), self._name(k_name)
        self.q_weight = self.k_weight = None

    def tensors(self):
        return {self.q_name: TensorSpec((self.dim,), "vector"), self.k_name: TensorSpec((self.dim,), "vector")}

    def load(self, tensors):
        self.q_weight, self.k_weight = tensors[self.q_name], tensors[self.k_name]

    def rotate(self, ctx, q, k):
        from ..ops import kernels

        kernels.head_rmsnorm(q, q.shape[1] // self.head_stride, self.head_stride, self.dim, self.q_weight, self.eps)
        kernels.head_rmsnorm(k, k.shape[1] // self.head_stride, self.head_stride, self.dim, self.k_weight, self.eps)


register_position_encoding("none", NoPositions)
register_position_encoding("head_rmsnorm", HeadRMSNorm)
register_position_encoding("learned", LearnedPositions)
