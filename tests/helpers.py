"""Shared helpers of the GPU parity tests: run the CPU oracle on torch tensors."""
import numpy as np
import torch

from oracle import nmg_oracle as O


def to_np(t):
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.float().numpy()
    return t.numpy()


def oracle_sparsify(x, n, m, sparse_dim, g, group_dim):
    """(val, idx, layout) of the oracle for a torch tensor; bf16 goes through fp32 (exact)."""
    val, idx, lay = O.sparsify(np.ascontiguousarray(to_np(x)), n, m, sparse_dim, g, group_dim)
    return val, idx, lay


def same_bits(gpu_tensor, ref_np):
    """Bit-exact comparison of a GPU tensor with an oracle array (values compared as raw bits)."""
    got = to_np(gpu_tensor)
    ref = ref_np.astype(got.dtype) if got.dtype != ref_np.dtype else ref_np
    if got.shape != ref.shape:
        return False
    if got.dtype.kind == "f":
        width = {2: np.uint16, 4: np.uint32, 8: np.uint64}[got.dtype.itemsize]
        return np.array_equal(np.ascontiguousarray(got).view(width), np.ascontiguousarray(ref).view(width))
    return np.array_equal(got, ref)


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def seeded(shape, dtype, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)
