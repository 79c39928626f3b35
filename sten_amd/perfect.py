"""Ungrouped n:m tensor: every block of m along ``sparse_dim`` keeps its n largest magnitudes,
with no constraint across rows.  The reference uses it as the upper bound of the magnitude a
grouped n:m tensor can preserve (grouped_nm_tensor.py:1010-1065, tests/test_nmg.py:73-83).

Shapes follow the reference: the sparse dim of the dense shape is replaced by ``(blocks, n)`` in
``val`` and ``idx`` (``idx`` = position inside the block, int64).  Tensors on the GPU go through
the library (``nmg_perfect_nm``); host tensors are handled with the same torch operators the
reference uses, so the class can be exercised without a GPU.  Kept values are ordered by
descending magnitude, equal magnitudes by position."""
import math

import torch

from . import native


class PerfectNMTensor:
    def __init__(self, val, idx, n, m, sparse_dim, sparse_dim_size):
        self.val, self.idx = val, idx
        self.n, self.m = n, m
        self.sparse_dim, self.sparse_dim_size = sparse_dim, sparse_dim_size

    @staticmethod
    def _geometry(shape, sparse_dim):
        return math.prod(shape[:sparse_dim]), shape[sparse_dim], math.prod(shape[sparse_dim + 1:])

    @staticmethod
    def from_dense(dense_tensor, n, m, sparse_dim):
        sparse_dim %= dense_tensor.dim()
        shape = tuple(dense_tensor.shape)
        size = shape[sparse_dim]
        blocks = math.ceil(size / m)
        out_shape = shape[:sparse_dim] + (blocks, n) + shape[sparse_dim + 1:]
        t = dense_tensor.detach()
        if t.device.type == "cuda":
            t = t.contiguous()
            outer, S, inner = PerfectNMTensor._geometry(shape, sparse_dim)
            val = torch.empty(out_shape, dtype=t.dtype, device=t.device)
            idx = torch.empty(out_shape, dtype=torch.int64, device=t.device)
            with torch.cuda.device(t.device):
                native.check(native.load().nmg_perfect_nm(
                    native.ptr(t), outer, S, inner, native.ptr(val), native.ptr(idx), n, m,
                    native.dtype_code(t.dtype), native.stream_ptr(t.device)))
            return PerfectNMTensor(val, idx, n, m, sparse_dim, size)
        # host tensors: pad, split the sparse dim into (blocks, m), stable descending sort
        t = t.movedim(sparse_dim, -1)
        t = torch.nn.functional.pad(t, (0, blocks * m - size))
        t = t.reshape(*t.shape[:-1], blocks, m)
        order = t.abs().argsort(dim=-1, descending=True, stable=True)[..., :n]
        val = t.gather(-1, order)
        # [..., rest, blocks, n] -> blocks, n at the place of the sparse dim
        nd = val.dim()
        perm = list(range(sparse_dim)) + [nd - 2, nd - 1] + list(range(sparse_dim, nd - 2))
        return PerfectNMTensor(val.permute(perm).contiguous(), order.permute(perm).contiguous(), n, m,
                               sparse_dim, size)

    def to_dense(self):
        sd = self.sparse_dim
        shape = tuple(self.val.shape[:sd]) + (self.sparse_dim_size,) + tuple(self.val.shape[sd + 2:])
        if self.val.device.type == "cuda":
            val, idx = self.val.contiguous(), self.idx.contiguous()
            outer, S, inner = PerfectNMTensor._geometry(shape, sd)
            dense = torch.empty(shape, dtype=val.dtype, device=val.device)
            with torch.cuda.device(val.device):
                native.check(native.load().nmg_perfect_nm_to_dense(
                    native.ptr(val), native.ptr(idx), outer, S, inner, native.ptr(dense), self.n, self.m,
                    native.dtype_code(val.dtype), native.stream_ptr(val.device)))
            return dense
        blocks = self.val.shape[sd]
        full = list(self.val.shape)
        full[sd + 1] = self.m
        dense = torch.zeros(full, dtype=self.val.dtype, device=self.val.device)
        dense.scatter_(sd + 1, self.idx, self.val)
        merged = full[:sd] + [blocks * self.m] + full[sd + 2:]
        return dense.reshape(merged).narrow(sd, 0, self.sparse_dim_size).contiguous()

    @property
    def shape(self):
        sd = self.sparse_dim
        return torch.Size(tuple(self.val.shape[:sd]) + (self.sparse_dim_size,) + tuple(self.val.shape[sd + 2:]))

    @property
    def dtype(self):
        return self.val.dtype

    @property
    def device(self):
        return self.val.device

    def to(self, device=None, dtype=None, non_blocking=False, copy=False, **_):
        return PerfectNMTensor(self.val.to(device=device, dtype=dtype, non_blocking=non_blocking, copy=copy),
                               self.idx.to(device=device, non_blocking=non_blocking, copy=copy),
                               self.n, self.m, self.sparse_dim, self.sparse_dim_size)


class PerfectNMSparsifier:
    """Exact per-block top-n magnitude sparsifier: ``n`` of every ``m`` along ``sparse_dim``."""

    def __init__(self, n, m, sparse_dim=-1):
        self.n, self.m, self.sparse_dim = n, m, sparse_dim


def install(api):
    """Register the sparsifier and the densifying conversion with a STen-style registry."""
    wrap = api.SparseTensorWrapper.wrapped_from_dense

    @api.register_sparsifier_implementation(sparsifier=PerfectNMSparsifier, inp=torch.Tensor, out=PerfectNMTensor)
    def dense_to_perfect_nm(sparsifier, tensor, grad_fmt=None):
        return wrap(PerfectNMTensor.from_dense(tensor, sparsifier.n, sparsifier.m, sparsifier.sparse_dim),
                    tensor, grad_fmt)

    @api.register_sparsifier_implementation(sparsifier=api.KeepAll, inp=PerfectNMTensor, out=api.DenseTensor)
    def perfect_nm_to_dense_tensor(sparsifier, tensor, grad_fmt=None):
        dense = tensor.wrapped_tensor.to_dense()
        return wrap(api.DenseTensor(dense), dense, grad_fmt)

    return {"dense_to_perfect_nm": dense_to_perfect_nm}


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
