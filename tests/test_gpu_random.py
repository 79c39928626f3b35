"""Differential sweep: random shapes, n:m:g patterns, orientations, dtypes and token counts (ragged
extents, tie-heavy inputs, tile-boundary sizes) -- sparsifier and to_dense bit-exact against the CPU
oracle, both matmul directions against the fp64 product of the oracle's dense form, the masked
weight gradient against the oracle's gather, the ungrouped n:m format bit-exact.  Seeds are fixed."""
import math
import random

import numpy as np
import pytest
import torch

import sten_amd as sten
from oracle import nmg_oracle as O
from helpers import oracle_sparsify, rel_l2, same_bits, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# rel-L2 against fp64: fp16 and fp32 as the benchmark contract states them (1e-3 with fp32
# accumulation, 1e-5); it states none for bf16, which has three mantissa bits fewer than fp16: 8 x 1e-3
TOL = {torch.float16: 1e-3, torch.bfloat16: 8e-3, torch.float32: 1e-5}


def one_case(rng, big):
    m = rng.choice([2, 3, 4, 4, 4, 5, 6, 8, 8, 8])
    n = rng.randint(1, m)
    c = math.comb(m, n)
    g = rng.choice([1, 2, 3, 4, 8, 16, 32])
    if c * g > 2600:
        g = max(1, 2600 // c)
    dt = rng.choice([torch.float16, torch.float16, torch.bfloat16, torch.float32])
    sd = rng.choice([0, 1])
    mult = 64 if big else rng.choice([1, 8, 8, 64])
    R = rng.randint(1, 40) * mult + (rng.choice([0, 0, 1, 3]) if mult == 1 else 0)
    C = rng.randint(1, 40) * mult + (rng.choice([0, 0, 1, 5]) if mult == 1 else 0)
    T = rng.choice([16, 17, 120, 256, 257, 300, 520, 1030]) if big else rng.choice([1, 2, 7, 16, 17, 33, 64, 100, 130, 260])
    ties = rng.random() < 0.3
    seed = rng.randint(0, 10 ** 6)
    print(f"case random {R}x{C} {n}:{m}:{g} sd={sd} {dt} T={T} ties={ties} seed={seed}", flush=True)
    gen = torch.Generator().manual_seed(seed)
    W = torch.randn((R, C), generator=gen)
    if ties:
        W = torch.round(W * 2) / 2          # many equal magnitudes and zeros
    W = W.to(dt)
    val, idx, lay = oracle_sparsify(W, n, m, sd, g, 1 - sd)
    w = sten.GroupedNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=1 - sd)
    assert np.array_equal(to_np(w.idx), idx) and same_bits(w.val, val), "sparsify"
    Wd = O.to_dense(val, idx, lay)
    assert same_bits(w.to_dense(), Wd), "to_dense"
    Wd64 = Wd.astype(np.float64)
    for rd in (0, 1):
        X = torch.randn((T, (R, C)[rd]), generator=gen).to(dt)
        b = torch.randn(((C, R)[rd],), generator=gen).to(dt) if rng.random() < 0.5 else None
        y = sten.spmm(w, X.to(DEV), None if b is None else b.to(DEV), reduce_dim=rd)
        ref = to_np(X).astype(np.float64) @ (Wd64.T if rd == 1 else Wd64)
        if b is not None:
            ref = ref + to_np(b).astype(np.float64)
        assert rel_l2(to_np(y), ref) <= TOL[dt], f"spmm reduce_dim={rd}"
    # torch.mm(W, B) and its gradient with respect to B, operands as they lie in memory
    B = torch.randn((C, T), generator=gen).to(dt)
    prod = sten.spmm_tt(w, B.to(DEV))
    assert prod.shape == (R, T)
    assert rel_l2(to_np(prod), Wd64 @ to_np(B).astype(np.float64)) <= TOL[dt], "W @ B"
    G = torch.randn((R, T), generator=gen).to(dt)
    gB = sten.spmm_tt_dense(w, G.to(DEV), reduce_dim=0)
    assert gB.shape == (C, T)
    assert rel_l2(to_np(gB), Wd64.T @ to_np(G).astype(np.float64)) <= TOL[dt], "W^T @ G"
    if dt != torch.float32 and R % 8 == 0 and C % 8 == 0:
        gy = torch.randn((T, R), generator=gen).to(dt)
        x = torch.randn((T, C), generator=gen).to(dt)
        gw = w.masked_product(gy.to(DEV), x.to(DEV))
        full = to_np(gy).astype(np.float64).T @ to_np(x).astype(np.float64)
        ref = O.gather_merged(O.merge(full, lay), idx, lay.n)
        real = O.gather_merged(O.merge(np.ones_like(full), lay), idx, lay.n) != 0
        got = to_np(gw.val).astype(np.float64)
        assert not got[~real].any(), "padded slots of the weight gradient"
        assert rel_l2(got, ref) <= TOL[dt], "masked weight gradient"
    if dt == torch.float32:
        # fp32: dense product on the fp32 matrix cores (both operands reduction-major), then the gather
        from sten_amd.impls import _masked_weight_grad
        gy = torch.randn((T, R), generator=gen).to(dt)
        x = torch.randn((T, C), generator=gen).to(dt)
        gw = _masked_weight_grad(w, gy.to(DEV), x.to(DEV))
        full = to_np(gy).astype(np.float64).T @ to_np(x).astype(np.float64)
        ref = O.gather_merged(O.merge(full, lay), idx, lay.n)
        assert rel_l2(to_np(gw.val).astype(np.float64), ref) <= TOL[dt], "fp32 weight gradient"
    pv, pi = O.perfect_nm(to_np(W), n, m, sd)
    p = sten.PerfectNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd)
    assert same_bits(p.val, pv) and np.array_equal(to_np(p.idx), pi), "ungrouped n:m"


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_small_cases(seed):
    rng = random.Random(seed)
    for _ in range(40):
        one_case(rng, big=False)


def test_random_tile_boundary_cases():
    rng = random.Random(21)
    for _ in range(25):
        one_case(rng, big=True)


def test_random_streamed_few_token_cases():
    """Random shapes, patterns, token counts, row pitches and biases through the two kernels that
    stream the compressed operand for at most 16 tokens (blocks of 8 along the reduction; the
    reduction along the group dim), against the fp64 product of the oracle's dense form."""
    rng = random.Random(31)
    for _ in range(60):
        along_sparse = rng.random() < 0.5
        dt = rng.choice([torch.float16, torch.bfloat16])
        T = rng.choice([1, 2, 3, 5, 8, 9, 13, 16])
        if along_sparse:
            n, m, g = rng.choice([1, 2, 4]), 8, rng.choice([1, 2, 4, 8, 32])
            M, K = rng.choice([8, 40, 96, 200, 512, 1000]), 256 * rng.choice([1, 2, 3, 5, 8, 13])
            sd, kern = 1, "sstream"
        else:
            m, n, g = rng.choice([4, 8]), rng.choice([1, 2]), rng.choice([1, 4, 8, 16])
            M, K = m * rng.choice([1, 3, 17, 64, 65, 190, 520]), 8 * rng.choice([1, 4, 5, 33, 64, 100, 333])
            sd, kern = 0, "gstream"
        seed = rng.randint(0, 10 ** 6)
        print(f"case streamed {kern} {dt} M={M} K={K} {n}:{m}:{g} T={T} seed={seed}", flush=True)
        gen = torch.Generator().manual_seed(seed)
        W = (torch.randn((M, K), generator=gen) * 0.5).to(dt)
        val, idx, lay = oracle_sparsify(W, n, m, sd, g, 1 - sd)
        Wd64 = O.to_dense(val, idx, lay).astype(np.float64)
        w = sten.GroupedNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=1 - sd)
        x = torch.randn((T, K), generator=gen).to(dt)
        b = torch.randn((M,), generator=gen).to(dt) if rng.random() < 0.5 else None
        xs = x.to(DEV)
        if rng.random() < 0.4 and T > 1:        # rows further apart than their length
            xs = torch.zeros((2 * T, K + 8), dtype=dt, device=DEV)[::2, :K]
            xs.copy_(x.to(DEV))
        y = sten.spmm(w, xs, None if b is None else b.to(DEV), reduce_dim=1, kernel=kern)
        ref = to_np(x).astype(np.float64) @ Wd64.T
        if b is not None:
            ref = ref + to_np(b).astype(np.float64)
        assert rel_l2(to_np(y), ref) <= TOL[dt], f"{kern} {M}x{K} {n}:{m}:{g} T={T}"
        if kern == "gstream" and (n, m) == (2, 4):
            # the same product with 16 outputs per workgroup (its lanes hold at most 4 token rows)
            T4 = min(T, 4)
            y4 = sten.spmm(w, xs[:T4], None if b is None else b.to(DEV), reduce_dim=1, kernel="ostream")
            assert rel_l2(to_np(y4), ref[:T4]) <= TOL[dt], f"ostream {M}x{K} T={T4}"
