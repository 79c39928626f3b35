"""GPU parity of the compressor and its element-wise companions against the CPU oracle.
Integer / byte results must be identical; kept values are copies and must match bit for bit."""
import itertools

import numpy as np
import pytest
import torch

import sten_amd as sten
from oracle import nmg_oracle as O
from helpers import oracle_sparsify, same_bits, seeded, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def check_parity(x_cpu, n, m, sd, g, gd):
    print(f"case shape={tuple(x_cpu.shape)} dtype={x_cpu.dtype} n:m:g={n}:{m}:{g} sd={sd} gd={gd}", flush=True)
    val, idx, lay = oracle_sparsify(x_cpu, n, m, sd, g, gd)
    t = sten.GroupedNMTensor.from_dense(x_cpu.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=gd)
    assert tuple(t.val.shape) == val.shape and tuple(t.idx.shape) == idx.shape
    assert np.array_equal(to_np(t.idx), idx), "idx differs from the oracle"
    assert same_bits(t.val, val), "val differs from the oracle"
    dense = t.to_dense()
    assert same_bits(dense, O.to_dense(val, idx, lay)), "to_dense differs from the oracle"
    return t, val, idx, lay


def test_config1_fp32_768_bit_exact():
    # benchmark config 1: fp32 768x768 N(0,1) seed 0, 2:4, group 16, n:m along the reduction dim
    torch.manual_seed(0)
    w = torch.randn(768, 768)
    check_parity(w, 2, 4, 1, 16, 0)
    check_parity(w, 2, 4, 0, 16, 1)  # the reference's default orientation


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,g", [(2, 4, 16), (1, 8, 32), (2, 8, 32), (3, 6, 4)])
def test_dtypes_and_ratios(dtype, n, m, g):
    w = seeded((300, 520), dtype, seed=n * 100 + m, std=0.02)
    check_parity(w, n, m, 1, g, 0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,g", [
    (1, 2, 3),     # 6 columns per tile: one lane per tile
    (2, 4, 4),     # 24 columns
    (1, 4, 16),    # 64 columns: two lanes per tile
    (2, 4, 8),     # 48 columns
    (2, 8, 4),     # 112 columns, 28 patterns: four lanes per tile
    (3, 6, 16),    # 320 columns: sixteen lanes per tile
    (2, 8, 16),    # 448 columns
    (4, 4, 5),     # n == m: one pattern
])
def test_small_tile_team_kernel_sizes(dtype, n, m, g):
    # many ties (few distinct magnitudes) in one input, continuous values in the other
    gen = torch.Generator().manual_seed(n * 1000 + m * 10 + g)
    ties = torch.randint(-3, 4, (150, 200), generator=gen).to(dtype)
    check_parity(ties, n, m, 1, g, 0)
    check_parity(seeded((257, 130), dtype, seed=g, std=0.02), n, m, 0, g, 1)


def test_4_8_32_large_tile():
    w = seeded((2240 + 100, 72), torch.float16, seed=48, std=0.02)
    check_parity(w, 4, 8, 1, 32, 0)


def test_ties_and_zeros():
    g = torch.Generator().manual_seed(7)
    w = torch.randint(-2, 3, (200, 96), generator=g).float()
    check_parity(w, 2, 4, 1, 16, 0)
    check_parity(torch.zeros(100, 40), 2, 4, 0, 4, 1)
    check_parity(w.half(), 1, 4, 0, 8, 1)


@pytest.mark.parametrize("n,m,g,rows", [
    (2, 4, 16, 96 * 2 + 40),     # half a wavefront per tile; 56 padded columns in the last chunk
    (2, 4, 64, 384 + 7),         # 384 columns: two wavefronts per tile, 377 padded columns
    (2, 8, 4, 112 + 30),         # one wavefront per tile (28 patterns)
    (2, 4, 32, 192 + 9),         # one wavefront per tile, four entries per lane
    (2, 8, 32, 896 + 130),       # four wavefronts per tile, 766 padded columns
    (4, 8, 32, 2240 + 33),       # sixteen wavefronts per tile
    (1, 8, 8, 64 * 3 + 1),       # quarter wavefronts; a single real column beside 63 padded ones
    (2, 4, 8, 48 * 2 + 5),       # quarter wavefronts, 43 padded columns
    (3, 6, 4, 80 + 13),          # half wavefronts, 20 patterns
])
def test_zero_columns_beside_zero_padding(n, m, g, rows):
    # Zero padding is placed in closed form after the keys with a positive score; real columns
    # that are zero, wholly or in the positions of some patterns, tie with it and must come out
    # as in the sorted walk: before it when their score is positive, after it when it is zero.
    gen = torch.Generator().manual_seed(rows)
    w = torch.randn(rows, 5 * m, generator=gen) * 0.02
    w[torch.rand(rows, generator=gen) < 0.3] = 0                      # whole columns of every tile
    w[torch.rand(rows, 5 * m, generator=gen) < 0.4] = 0               # scattered zeros
    w[:, m:2 * m] = torch.randint(-1, 2, (rows, m), generator=gen).float() * 0.5   # three magnitudes
    w[:, 2 * m:3 * m] = 0                                             # a block column of zero tiles
    check_parity(w.half(), n, m, 1, g, 0)
    check_parity(w.t().contiguous(), n, m, 0, g, 1)


def test_resparsifying_a_pruned_weight():
    # half of the entries are exact zeros already, so most patterns of a column tie at its best score
    w = seeded((500, 256), torch.float16, seed=21, std=0.02)
    t = sten.GroupedNMTensor.from_dense(w.to(DEV), 2, 4, 1, 16, 0)
    check_parity(t.to_dense().cpu(), 2, 4, 1, 32, 0)
    check_parity(t.to_dense().cpu(), 1, 4, 1, 16, 0)
    check_parity(t.to_dense().cpu(), 2, 8, 1, 8, 0)


def test_reference_test_shapes_5_12_2():
    # tests/test_nmg.py:33-86: shapes (3,a,b), a,b in {17,5,1}, all axis orders, 5:12:2
    torch.manual_seed(123)
    dims = [17, 5, 1]
    for a, b in itertools.product(dims, dims):
        base = torch.rand(3, a, b)
        for perm in itertools.permutations(range(3)):
            x = base.permute(perm).contiguous()
            layout = "".join("abc"[i] for i in perm)
            t, val, idx, lay = check_parity(x, 5, 12, layout.index("c"), 2, layout.index("b"))
            sp = to_np(t.to_dense())
            xn = x.numpy()
            assert ((sp == xn) | (sp == 0)).all()
            assert np.abs(sp).sum() / np.abs(xn).sum() > 5 / 12


def test_non_contiguous_input_and_empty():
    w = seeded((64, 200), torch.float32, seed=3)
    check_parity(w.t(), 2, 4, 0, 4, 1)           # transposed view, read through strides
    t = sten.GroupedNMTensor.from_dense(torch.zeros(0, 8, device=DEV), 2, 4, 1, 4, 0)
    assert t.val.numel() == 0 and tuple(t.to_dense().shape) == (0, 8)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("n,m,g", [(2, 4, 16), (1, 8, 8), (2, 8, 4), (1, 2, 16)])
def test_device_views_with_offsets_and_row_strides(dtype, n, m, g):
    # the compressor reads a column's m values with one aligned load where it can; views whose
    # base or row stride break the alignment, or whose rows are longer than the view, must give
    # the same bits as a contiguous copy
    for width, lo, hi in [(208, 8, 200), (208, 0, 192), (203, 3, 195), (203, 4, 196), (208, 1, 193)]:
        big = seeded((130, width), dtype, seed=width + lo).to(DEV)
        view = big[:, lo:hi]
        print(f"case view of ({130},{width})[:, {lo}:{hi}] dtype={dtype} n:m:g={n}:{m}:{g}", flush=True)
        val, idx, lay = oracle_sparsify(view.cpu().contiguous(), n, m, 1, g, 0)
        t = sten.GroupedNMTensor.from_dense(view, n, m, sparse_dim=1, group_size=g, group_dim=0)
        assert np.array_equal(to_np(t.idx), idx)
        assert same_bits(t.val, val)


def test_clone_layout_matches_oracle_gather():
    w = seeded((100, 72), torch.float32, seed=11)
    t, val, idx, lay = check_parity(w, 2, 4, 1, 4, 0)
    other = seeded((100, 72), torch.float32, seed=12)
    got = t.clone_layout(other.to(DEV))
    want = O.gather_merged(O.merge(other.numpy(), lay), idx, 2)
    assert same_bits(got.val, want)
    assert got.idx.data_ptr() == t.idx.data_ptr()


def test_rejects_cpu_tensor_and_wide_tile():
    with pytest.raises(sten.NmgError):
        sten.GroupedNMTensor.from_dense(torch.zeros(8, 8), 2, 4, 1, 1, 0)
    with pytest.raises(ValueError):
        sten.GroupedNMTensor.from_dense(torch.zeros(8, 8, device=DEV), 5, 12, 1, 42, 0)


def test_full_size_properties_config2():
    # 4096x4096 fp16 N(0,0.02), 2:4:16 along K: size-independent properties + oracle on a slab
    torch.manual_seed(0)
    w = (torch.randn(4096, 4096) * 0.02).half()
    t = sten.GroupedNMTensor.from_dense(w.to(DEV), 2, 4, 1, 16, 0)
    lay = t.layout
    idx = t.idx.view(lay.outer, lay.cols).int()
    assert bool((idx.sort(dim=1).values == torch.arange(lay.cols, device=DEV, dtype=torch.int32)).all())
    dense = t.to_dense()
    wg = w.to(DEV)
    assert bool(((dense == wg) | (dense == 0)).all())
    blocks = (dense.view(4096, 1024, 4) != 0).sum(-1)
    assert int(blocks.max()) <= 2
    again = sten.GroupedNMTensor.from_dense(dense, 2, 4, 1, 16, 0)      # idempotence of the kept mass
    assert float(again.to_dense().abs().sum()) == pytest.approx(float(dense.abs().sum()), rel=1e-6)
    val, idx_o, _ = oracle_sparsify(w[:192], 2, 4, 1, 16, 0)            # first two 96-row chunks
    k = val.shape[0]
    assert np.array_equal(to_np(t.idx[:k]), idx_o) and same_bits(t.val[:k], val)


def test_preserved_magnitude_between_random_and_perfect():
    # tests/test_nmg.py:33-86: shapes (3, a, b) with a, b in {17, 5, 1} in every axis order, 5:12:2;
    # the grouped tensor is a valid n:m tensor, beats n/m of the magnitude and stays below the
    # ungrouped ("perfect") n:m tensor
    torch.manual_seed(123)
    n, m, g = 5, 12, 2
    for a, b in itertools.permutations([17, 5, 1], 2):
        for sparse_dim, group_dim in itertools.permutations(range(3), 2):
            x = torch.rand(3, a, b, device=DEV)
            t = sten.GroupedNMTensor.from_dense(x, n, m, sparse_dim=sparse_dim, group_size=g, group_dim=group_dim)
            d = t.to_dense()
            assert sten.is_correct_nm(x, d, sparse_dim, n, m)
            kept = float(d.abs().sum() / x.abs().sum())
            assert kept > n / m or x.shape[sparse_dim] < m
            p = sten.PerfectNMTensor.from_dense(x, n=n, m=m, sparse_dim=sparse_dim)
            pd = p.to_dense()
            assert pd.shape == x.shape and sten.is_correct_nm(x, pd, sparse_dim, n, m)
            assert float(pd.abs().sum() / x.abs().sum()) >= kept - 1e-5
