"""2:4-pruned, int4-quantised weight for decode-shape linear layers (the benchmark's "sparse-marlin"
configuration).  Mirrors the custom format of the reference's test, which wraps an external
library: ``SparseMarlinSparsifier`` / ``SparseMarlinTensor`` with fields ``B`` (packed values),
``s`` (scales) and ``meta`` (positions), registered for ``F.linear``
(tests/test_sparse_marlin.py:60-114).  Here the weight is really pruned and quantised, and the
product runs in this library's HIP kernel (``nmg_w4_linear``); the packing is this library's own.
"""
import ctypes

import torch

from . import native


class SparseMarlinSparsifier:
    """2:4 magnitude pruning along the last dim + symmetric int4, one fp16 scale per row and
    ``group_size`` positions (only 128 is built)."""

    def __init__(self, group_size=128):
        if group_size != 128:
            raise ValueError("only group_size=128 is supported")
        self.group_size = group_size


class SparseMarlinTensor:
    def __init__(self, B, s, meta, dense_shape):
        self.B, self.s, self.meta = B, s, meta
        self.dense_shape = tuple(dense_shape)

    @classmethod
    def from_dense(cls, w):
        """w: fp16 [out_features, in_features] on the GPU, in_features a multiple of 128."""
        if w.dim() != 2 or w.dtype != torch.float16:
            raise native.NmgError("the int4 format takes a 2-D fp16 weight")
        native.require_gpu(w)
        if w.stride(1) != 1:
            w = w.contiguous()
        lib = native.load()
        M, K = w.shape
        nb, nm, ns = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        native.check(lib.nmg_w4_sizes(M, K, ctypes.byref(nb), ctypes.byref(nm), ctypes.byref(ns)))
        B = torch.empty((nb.value,), dtype=torch.uint8, device=w.device)
        meta = torch.empty((nm.value,), dtype=torch.int32, device=w.device)
        s = torch.empty((ns.value,), dtype=torch.float16, device=w.device)
        with torch.cuda.device(w.device):
            native.check(lib.nmg_w4_pack(native.ptr(w), w.stride(0), M, K, native.ptr(B), native.ptr(meta),
                                         native.ptr(s), native.stream_ptr(w.device)))
        return cls(B, s, meta, (M, K))

    # attributes the dispatch wrapper looks for (avoids a to_dense() round trip)
    @property
    def shape(self):
        return torch.Size(self.dense_shape)

    @property
    def dtype(self):
        return torch.float16

    @property
    def device(self):
        return self.B.device

    def nbytes(self):
        return self.B.numel() + 4 * self.meta.numel() + 2 * self.s.numel()

    def to_dense(self):
        """The dequantised weight (zeros at pruned positions)."""
        M, K = self.dense_shape
        out = torch.empty((M, K), dtype=torch.float16, device=self.B.device)
        with torch.cuda.device(out.device):
            native.check(native.load().nmg_w4_to_dense(
                native.ptr(self.B), native.ptr(self.meta), native.ptr(self.s), M, K, native.ptr(out), K,
                native.stream_ptr(out.device)))
        return out

    def linear(self, x, bias=None):
        """x [..., K] fp16 -> [..., M].  At most 16 token rows go through the int4 kernel; larger
        batches multiply by the dequantised weight (a plain dense GEMM, not the path this format is
        for)."""
        M, K = self.dense_shape
        if x.shape[-1] != K or x.dtype != torch.float16:
            raise native.NmgError(f"activations must be fp16 [..., {K}], got {x.dtype} {tuple(x.shape)}")
        native.require_gpu(x)
        x2 = x.reshape(-1, K)
        T = x2.shape[0]
        if T > 16:
            return torch.nn.functional.linear(x, self.to_dense(), bias)
        if x2.stride(1) != 1 or x2.stride(0) % 8 != 0 or x2.data_ptr() % 16 != 0:
            x2 = x2.contiguous()
        if bias is not None:
            bias = bias.to(torch.float16).contiguous()
        y = torch.empty((T, M), dtype=torch.float16, device=x.device)
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_w4_linear(
                native.ptr(self.B), native.ptr(self.meta), native.ptr(self.s), M, K, native.ptr(x2),
                x2.stride(0) if T > 1 else K, native.ptr(y), M, native.ptr(bias), T,
                native.stream_ptr(x.device)))
        return y.reshape(*x.shape[:-1], M)


def install(api):
    """Registers the sparsifier and the forward of F.linear (arity 2 and 3), as the reference's
    test does for its external kernel (tests/test_sparse_marlin.py:76-114)."""
    wrap = api.SparseTensorWrapper.wrapped_from_dense
    dense_fmt = (api.KeepAll, torch.Tensor)

    @api.register_sparsifier_implementation(
        sparsifier=SparseMarlinSparsifier, inp=torch.Tensor, out=SparseMarlinTensor)
    def marlin_sparsifier_impl(sparsifier, tensor, grad_fmt=None):
        return wrap(SparseMarlinTensor.from_dense(tensor), tensor, grad_fmt)

    def linear_fwd(ctx, inputs, output_sparsifiers):
        x, weight = inputs[0], inputs[1]
        bias = inputs[2] if len(inputs) > 2 else None
        return weight.wrapped_tensor.linear(x, bias)

    api.register_fwd_op_impl(operator=torch.nn.functional.linear,
                             inp=(torch.Tensor, SparseMarlinTensor), out=[dense_fmt])(linear_fwd)
    api.register_fwd_op_impl(operator=torch.nn.functional.linear,
                             inp=(torch.Tensor, SparseMarlinTensor, torch.Tensor), out=[dense_fmt])(linear_fwd)
