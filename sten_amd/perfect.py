"""Ungrouped n:m tensor: every block of m along ``sparse_dim`` keeps its n largest magnitudes,
with no constraint across rows.  The reference uses it as the upper bound of the magnitude a
grouped n:m tensor can preserve (grouped_nm_tensor.py:1010-1065, tests/test_nmg.py:73-83).  Plain
torch ops on whatever device the input lives on; not a matmul operand."""
import math

import torch


class PerfectNMTensor:
    def __init__(self, val, idx, n, m, sparse_dim, sparse_dim_size):
        self.val, self.idx = val, idx
        self.n, self.m = n, m
        self.sparse_dim, self.sparse_dim_size = sparse_dim, sparse_dim_size

    @staticmethod
    def from_dense(dense_tensor, n, m, sparse_dim):
        sparse_dim %= dense_tensor.dim()
        size = dense_tensor.shape[sparse_dim]
        blocks = math.ceil(size / m)
        t = dense_tensor.movedim(sparse_dim, -1)
        t = torch.nn.functional.pad(t, (0, blocks * m - size))
        t = t.reshape(*t.shape[:-1], blocks, m)
        idx = t.abs().topk(n, dim=-1).indices                # [..., blocks, n]
        val = t.gather(-1, idx)
        return PerfectNMTensor(val, idx, n, m, sparse_dim, size)

    def to_dense(self):
        blocks = self.val.shape[-2]
        dense = torch.zeros(*self.val.shape[:-1], self.m, dtype=self.val.dtype, device=self.val.device)
        dense.scatter_(-1, self.idx, self.val)
        dense = dense.reshape(*dense.shape[:-2], blocks * self.m)[..., :self.sparse_dim_size]
        return dense.movedim(-1, self.sparse_dim).contiguous()

    @property
    def shape(self):
        s = list(self.val.shape[:-2])
        s.insert(self.sparse_dim, self.sparse_dim_size)
        return torch.Size(s)

    @property
    def dtype(self):
        return self.val.dtype

    @property
    def device(self):
        return self.val.device


def is_correct_nm(original_dense, sparsified_dense, sparse_dim, n, m):
    """Every entry is kept or zero, and no block of m along sparse_dim keeps more than n
    (the check of grouped_nm_tensor.py:1069-1091)."""
    kept_or_zero = (original_dense == sparsified_dense) | (sparsified_dense == 0)
    if not bool(kept_or_zero.all()):
        return False
    sparse_dim %= original_dense.dim()
    size = original_dense.shape[sparse_dim]
    blocks = math.ceil(size / m)
    t = torch.nn.functional.pad(sparsified_dense.movedim(sparse_dim, -1), (0, blocks * m - size))
    nnz = (t.reshape(*t.shape[:-1], blocks, m) != 0).sum(dim=-1)
    return bool((nnz <= n).all())
