"""Geometry of a grouped n:m tensor.

A dense N-D tensor is cut into tiles of ``c*g`` indices of the *group dim* times ``m`` indices of
the *sparse dim* (``c = C(m, n)``).  Inside a tile every group-dim index ("column") keeps ``n`` of
its ``m`` values according to one of the ``c`` patterns, and exactly ``g`` columns use each
pattern.  Tiles are numbered (remaining dims..., group-dim chunk, sparse-dim block), chunk slower
than block.  The compressed tensor is ``val [outer, c, g, n]`` plus ``idx [outer, c, g, 1]``
(int16 position of the column inside its chunk).

This is the layout of the reference's ``compute_nm_strides`` / ``dense_to_grouped_n_m``
(src/sten/grouped_nm/grouped_nm_tensor.py:71-217, :701-710); the kernels here read the strided
dense tensor directly instead of materialising the padded, permuted ``[outer, c, g, m]`` copy.
"""
import math
from dataclasses import dataclass

from . import native


@dataclass(frozen=True)
class NMGLayout:
    dense_shape: tuple
    n: int
    m: int
    group_size: int
    sparse_dim: int
    group_dim: int

    def __post_init__(self):
        nd = len(self.dense_shape)
        if nd < 2:
            raise ValueError("grouped n:m needs a tensor with at least 2 dims")
        if not (0 <= self.sparse_dim < nd and 0 <= self.group_dim < nd):
            raise ValueError("sparse_dim / group_dim out of range")
        if self.sparse_dim == self.group_dim:
            raise ValueError("sparse_dim and group_dim must differ")
        if not (0 <= self.n <= self.m and self.m >= 1 and self.group_size >= 1):
            raise ValueError(f"invalid n:m:g = {self.n}:{self.m}:{self.group_size}")
        if self.chunk_size * self.group_size >= 2 ** 15:
            # grouped_nm_tensor.py:229 -- column positions are stored as int16
            raise ValueError("chunk_size * group_size must be < 2**15")

    # ---- sizes -------------------------------------------------------------------------
    @property
    def chunk_size(self):
        return math.comb(self.m, self.n)

    @property
    def cols(self):
        return self.chunk_size * self.group_size

    @property
    def num_chunks(self):
        return -(-self.dense_shape[self.group_dim] // self.cols)

    @property
    def num_blocks(self):
        return -(-self.dense_shape[self.sparse_dim] // self.m)

    @property
    def other_dims(self):
        return [d for d in range(len(self.dense_shape)) if d not in (self.sparse_dim, self.group_dim)]

    @property
    def batch(self):
        return math.prod(self.dense_shape[d] for d in self.other_dims)

    @property
    def outer(self):
        return self.batch * self.num_chunks * self.num_blocks

    @property
    def G(self):
        return self.dense_shape[self.group_dim]

    @property
    def S(self):
        return self.dense_shape[self.sparse_dim]

    @property
    def val_shape(self):
        return (self.outer, self.chunk_size, self.group_size, self.n)

    @property
    def idx_shape(self):
        return (self.outer, self.chunk_size, self.group_size, 1)

    @property
    def merged_shape(self):
        return (self.outer, self.chunk_size, self.group_size, self.m)

    @property
    def padded_dense_shape(self):
        s = list(self.dense_shape)
        s[self.sparse_dim] = self.num_blocks * self.m
        s[self.group_dim] = self.num_chunks * self.cols
        return tuple(s)

    @property
    def order(self):
        return native.order_table(self.n, self.m)

    def transposed(self):
        """Layout of the 2-D transpose (same tiles, dims swapped)."""
        assert len(self.dense_shape) == 2
        return NMGLayout(tuple(reversed(self.dense_shape)), self.n, self.m, self.group_size,
                         1 - self.sparse_dim, 1 - self.group_dim)

    def as_nm_strides(self):
        """The subset of the reference's ``nm_strides`` dict that its callers read
        (sten_impls.py:55-63,156; grouped_nm_tensor.py:173-217)."""
        return {
            "n": self.n,
            "m": self.m,
            "sparse_dim": self.sparse_dim,
            "group_dim": self.group_dim,
            "group_size": self.group_size,
            "dense_shape": tuple(self.dense_shape),
            "padded_dense_shape": self.padded_dense_shape,
            "chunk_size": self.chunk_size,
            "num_chunks": self.num_chunks,
            "num_blocks": self.num_blocks,
            "order": self.order,
            "merged_shape": list(self.merged_shape),
            "padded_sparse_dim": self.num_blocks * self.m,
            "padded_group_dim": self.num_chunks * self.cols,
        }


def bgs_view(t, lay):
    """Return (tensor, NmgView) presenting ``t`` as [batch, G, S] with element strides.

    The returned tensor aliases ``t`` whenever the non-sparse, non-group dims collapse into one
    stride (always for 2-D); otherwise it is a contiguous re-ordered copy."""
    p = t.permute(lay.other_dims + [lay.group_dim, lay.sparse_dim])
    G, S = p.shape[-2], p.shape[-1]
    if p.dim() == 2:
        q = p.unsqueeze(0)
    else:
        try:
            q = p.view(-1, G, S)
        except RuntimeError:
            q = p.reshape(-1, G, S)
    v = native.NmgView(q.shape[0], G, S, q.stride(0) if q.shape[0] > 1 else 0, q.stride(1), q.stride(2))
    return q, v
