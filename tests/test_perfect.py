"""PerfectNMTensor (ungrouped n:m).  Host logic on the CPU (torch operators, like the reference);
on the GPU the HIP kernels, bit-exact against the numpy restatement of
grouped_nm_tensor.py:1010-1065 in oracle/nmg_oracle.py.  The order of equal magnitudes is open in
the reference (unstable argsort) -- parity unpinned for ties; here the lower position comes first."""
import itertools

import numpy as np
import pytest
import torch

import sten_amd as sten
from sten_amd.perfect import PerfectNMSparsifier, PerfectNMTensor, is_correct_nm
from oracle import nmg_oracle as O
from helpers import same_bits, seeded, to_np


def test_round_trip_and_block_structure():
    torch.manual_seed(0)
    for shape in [(3, 17, 5), (8, 8), (1, 13)]:
        x = torch.randn(*shape)
        for sd in range(len(shape)):
            for n, m in [(2, 4), (1, 8), (5, 12)]:
                p = PerfectNMTensor.from_dense(x, n, m, sd)
                # the reference's shapes: the sparse dim becomes (blocks, n)
                blocks = -(-shape[sd] // m)
                assert tuple(p.val.shape) == shape[:sd] + (blocks, n) + shape[sd + 1:] == tuple(p.idx.shape)
                d = p.to_dense()
                assert d.shape == x.shape == p.shape
                assert is_correct_nm(x, d, sd, n, m)
                # each block keeps exactly its n largest magnitudes (padding counts as zeros)
                xs = x.movedim(sd, -1)
                pad = (-xs.shape[-1]) % m
                blk = torch.nn.functional.pad(xs, (0, pad)).reshape(*xs.shape[:-1], -1, m).abs()
                best = blk.topk(n, dim=-1).values.sum()
                assert torch.isclose(d.abs().sum(), best)
                # and matches the numpy restatement bit for bit
                val, idx = O.perfect_nm(x.numpy(), n, m, sd)
                assert np.array_equal(p.val.numpy(), val) and np.array_equal(p.idx.numpy(), idx)
                assert np.array_equal(d.numpy(), O.perfect_nm_to_dense(val, idx, m, sd, shape[sd]))


def test_oracle_hand_worked_blocks():
    # 2:4 along the last dim: block (1, -7, 3, 7) keeps -7 and 7, the lower position first on the
    # tie; block (0, 0, 0, 5) keeps 5 and then the first zero; the ragged tail (2,) is padded
    x = np.array([[1, -7, 3, 7, 0, 0, 0, 5, 2]], dtype=np.float32)
    val, idx = O.perfect_nm(x, 2, 4, 1)
    assert val.tolist() == [[[-7, 7], [5, 0], [2, 0]]]
    assert idx.tolist() == [[[1, 3], [3, 0], [0, 1]]]
    assert O.perfect_nm_to_dense(val, idx, 4, 1, 9).tolist() == [[0, -7, 0, 7, 0, 0, 0, 5, 2]]


def test_is_correct_nm_rejects_violations():
    x = torch.arange(1.0, 9.0).reshape(2, 4)
    assert is_correct_nm(x, x * torch.tensor([1.0, 1.0, 0.0, 0.0]), 1, 2, 4)
    assert not is_correct_nm(x, x, 1, 2, 4)                                   # 4 kept in a block of 4
    assert not is_correct_nm(x, torch.full_like(x, 0.5), 1, 2, 4)             # values changed


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_hip_kernels_match_the_restatement_bit_exactly(dtype):
    dev = "cuda:0"
    for shape, (n, m) in itertools.product([(3, 17, 5), (5, 1, 17), (64, 200), (1, 13), (7, 40, 3, 2)],
                                           [(2, 4), (1, 8), (5, 12), (4, 4), (3, 64)]):
        x = seeded(shape, dtype, seed=sum(shape) + n + m)
        x.view(-1)[::7] = x.view(-1)[3]               # ties, also across block boundaries
        x.view(-1)[::11] = 0
        for sd in range(len(shape)):
            print(f"case perfect nm {dtype} {shape} {n}:{m} sd={sd}", flush=True)
            p = PerfectNMTensor.from_dense(x.to(dev), n, m, sd)
            xn = to_np(x) if dtype != torch.bfloat16 else to_np(x)          # bf16 compared through fp32 (exact)
            val, idx = O.perfect_nm(xn, n, m, sd)
            assert same_bits(p.val, val)
            assert np.array_equal(to_np(p.idx), idx)
            d = p.to_dense()
            assert same_bits(d, O.perfect_nm_to_dense(val, idx, m, sd, shape[sd]))
            assert is_correct_nm(x.to(dev), d, sd, n, m)


@pytest.mark.gpu
def test_registered_sparsifier_and_upper_bound_of_the_grouped_format():
    # the flow of tests/test_nmg.py:12-30 with the ungrouped sparsifier, and its role in
    # tests/test_nmg.py:73-83: no grouped n:m tensor preserves more magnitude
    dev = "cuda:0"
    torch.manual_seed(5)
    lin = torch.nn.Linear(96, 64).to(dev)
    w0 = lin.weight.detach().clone()
    sb = sten.SparsityBuilder()
    sb.set_weight("weight", initial_sparsifier=PerfectNMSparsifier(2, 4, sparse_dim=1), out_format=PerfectNMTensor)
    sp = sb.get_sparse_model(lin)
    p = sp.weight.wrapped_tensor
    assert isinstance(p, PerfectNMTensor) and tuple(p.val.shape) == (64, 24, 2)
    val, idx = O.perfect_nm(to_np(w0), 2, 4, 1)
    assert same_bits(p.val, val) and np.array_equal(to_np(p.idx), idx)
    x = torch.randn(5, 96, device=dev)
    with pytest.warns(sten.DispatchWarning):
        y = sp(x)                                                 # F.linear has no implementation for it: dense fallback
    ref = torch.nn.functional.linear(x, p.to_dense(), lin.bias)
    assert torch.allclose(y, ref, atol=1e-5)
    g = sten.GroupedNMTensor.from_dense(w0, 2, 4, sparse_dim=1, group_size=4, group_dim=0)
    assert float(p.to_dense().abs().sum()) >= float(g.to_dense().abs().sum()) - 1e-5


@pytest.mark.gpu
def test_argument_errors():
    from sten_amd import native
    lib = native.load()
    x = torch.zeros(8, 8, device="cuda:0")
    v = torch.zeros(8, 2, 2, device="cuda:0")
    i = torch.zeros(8, 2, 2, dtype=torch.int64, device="cuda:0")
    assert lib.nmg_perfect_nm(native.ptr(x), 8, 8, 1, native.ptr(v), native.ptr(i), 5, 4, native.NMG_F32, None) == 1
    assert lib.nmg_perfect_nm(native.ptr(x), 8, 8, 1, native.ptr(v), native.ptr(i), 2, 65, native.NMG_F32, None) == 1
    assert lib.nmg_perfect_nm(None, 8, 8, 1, native.ptr(v), native.ptr(i), 2, 4, native.NMG_F32, None) == 1
    assert lib.nmg_perfect_nm(native.ptr(x), 8, 0, 1, native.ptr(v), native.ptr(i), 2, 4, native.NMG_F32, None) == 0
