"""Pins the CPU oracle (oracle/) against hand-worked answers, closed forms, invariants and a
brute-force matcher.  The reference holds no golden vectors for this path (its tests draw random
inputs and check invariants, tests/test_nmg.py:33-86), so these checks are what fixes the oracle."""
import itertools
import math

import numpy as np
import pytest

from oracle import nmg_oracle as O


def tuples(n, m):
    return [tuple(int(x) for x in t) for t in O.order(n, m)]


# ---------------------------------------------------------------- pattern order (make_n_m)

def test_order_hand_traced_tables():
    # traced by hand from the recursion in grouped_nm_tensor.py:37-50
    assert tuples(2, 4) == [(0, 1), (0, 2), (1, 2), (1, 3), (0, 3), (2, 3)]
    assert tuples(1, 8) == [(5,), (3,), (1,), (0,), (2,), (4,), (6,), (7,)]
    assert tuples(1, 4) == [(1,), (0,), (2,), (3,)]
    assert tuples(1, 2) == [(0,), (1,)]
    assert tuples(2, 3) == [(0, 1), (0, 2), (1, 2)]
    assert tuples(1, 3) == [(0,), (1,), (2,)]
    assert tuples(2, 2) == [(0, 1)]
    assert tuples(3, 4) == [(0, 1, 2), (0, 1, 3), (0, 2, 3), (1, 2, 3)]


def test_order_closed_form_n1():
    # T(1) = [0]; T(k) = reversed(T(k-1)) + [k-1]; make_n_m(1, m) = T(m-1) + [m-1]
    def T(k):
        return [0] if k == 1 else list(reversed(T(k - 1))) + [k - 1]

    for m in range(2, 17):
        assert [t[0] for t in tuples(1, m)] == T(m - 1) + [m - 1]


@pytest.mark.parametrize("m", range(1, 13))
def test_order_invariants(m):
    # is_valid_n_m (grouped_nm_tensor.py:24-34)
    for n in range(0, m + 1):
        t = tuples(n, m)
        assert len(t) == math.comb(m, n)
        assert len(set(t)) == len(t)
        for a in t:
            assert all(x < y for x, y in zip(a, a[1:]))
            assert all(0 <= x < m for x in a)
        for a, b in zip(t, t[1:]):
            assert sum(x != y for x, y in zip(a, b)) == 1


def test_order_recursive_structure():
    # the last C(m-1, n-1) entries are exactly the tuples that contain m-1, the others never do
    for n, m in [(2, 8), (4, 8), (3, 6), (5, 12), (2, 6)]:
        t = tuples(n, m)
        c1 = math.comb(m - 1, n)
        assert all(m - 1 not in a for a in t[:c1])
        assert all(a[-1] == m - 1 for a in t[c1:])
        # first part is make_n_m(n, m-1, special=True): for the top-level call it is not reversed,
        # and special only reverses *its* first part -> same set, checked as a set here
        assert set(t[:c1]) == set(itertools.combinations(range(m - 1), n))


# -------------------------------------------------------------------------- sparsifier

def test_sparsify_hand_worked_tiles():
    d = np.array([[[[3, 1]], [[2, 5]]]], dtype=np.float32)  # 1:2, g=1: columns (3,1), (2,5)
    v, i = O.sparsify_merged(d, 1)
    assert i.ravel().tolist() == [0, 1] and v.ravel().tolist() == [3, 5]
    d = np.array([[[[3, 1]], [[4, 0.5]]]], dtype=np.float32)  # capacity conflict
    v, i = O.sparsify_merged(d, 1)
    assert i.ravel().tolist() == [1, 0] and v.ravel().tolist() == [4, 1]
    z = np.zeros((1, 6, 2, 4), dtype=np.float32)  # all-zero 2:4 g=2 tile
    v, i = O.sparsify_merged(z, 2)
    assert i.ravel().tolist() == [1, 0, 3, 2, 5, 4, 7, 6, 9, 8, 11, 10]
    assert not v.any()


@pytest.mark.parametrize("n,m,g", [(2, 4, 3), (1, 8, 2), (3, 6, 1), (2, 8, 2)])
def test_sparsify_all_zero_closed_form(n, m, g):
    c = math.comb(m, n)
    z = np.zeros((2, c, g, m), dtype=np.float32)
    _, idx = O.sparsify_merged(z, n)
    p, s = np.meshgrid(np.arange(c), np.arange(g), indexing="ij")
    want = (c * g - 1) - ((c - 1 - p) * g + s)
    for t in range(2):
        assert np.array_equal(idx[t, :, :, 0], want)


def test_sparsify_n_equals_m_closed_form():
    # c = 1: columns sorted by descending sum |col|, ties -> larger index first
    rng = np.random.default_rng(5)
    g, m = 7, 3
    d = rng.integers(-3, 4, size=(4, 1, g, m)).astype(np.float32)
    val, idx = O.sparsify_merged(d, m)
    for t in range(4):
        score = np.abs(d[t, 0]).sum(axis=1)
        want = sorted(range(g), key=lambda o: (score[o], o), reverse=True)
        assert idx[t, 0, :, 0].tolist() == want
        assert np.array_equal(val[t, 0], d[t, 0][want])


def brute_force_tile(d, n, g):
    """Independent matcher: repeatedly take the best (score, o, p) among the still-valid pairs."""
    c, m = math.comb(d.shape[-1], n), d.shape[-1]
    cols = d.reshape(-1, m)
    order = tuples(n, m)
    score = {}
    for o in range(cols.shape[0]):
        for p in range(c):
            acc = np.float32(0)
            for j in order[p]:
                acc = np.float32(acc + np.float32(abs(cols[o, j])))
            score[(o, p)] = acc
    free, cnt = set(range(cols.shape[0])), [0] * c
    idx = [-1] * (c * g)
    while free:
        best = max(((score[(o, p)], o, p) for o in free for p in range(c) if cnt[p] < g))
        _, o, p = best
        idx[p * g + cnt[p]] = o
        cnt[p] += 1
        free.remove(o)
    return idx


@pytest.mark.parametrize("n,m,g,seed", [(1, 2, 1, 0), (1, 2, 3, 1), (2, 4, 2, 2), (1, 4, 2, 3),
                                        (2, 3, 2, 4), (3, 5, 1, 5), (2, 4, 2, 6)])
def test_sparsify_vs_brute_force(n, m, g, seed):
    rng = np.random.default_rng(seed)
    c = math.comb(m, n)
    # small integers produce many ties, which exercises the tie-breaking order
    d = rng.integers(-2, 3, size=(5, c, g, m)).astype(np.float32)
    d[3] = rng.standard_normal((c, g, m)).astype(np.float32)
    val, idx = O.sparsify_merged(d, n)
    order = tuples(n, m)
    for t in range(d.shape[0]):
        want = brute_force_tile(d[t], n, g)
        assert idx[t].ravel().tolist() == want
        cols = d[t].reshape(-1, m)
        for slot, o in enumerate(want):
            assert val[t].reshape(-1, n)[slot].tolist() == [cols[o, j] for j in order[slot // g]]


def is_correct_nm(orig, sp, sparse_dim, n, m):
    """Restatement of the reference's validity check (grouped_nm_tensor.py:1069-1091)."""
    if not ((orig == sp) | (sp == 0)).all():
        return False
    S = orig.shape[sparse_dim]
    pad = [(0, 0)] * orig.ndim
    pad[sparse_dim] = (0, -(-S // m) * m - S)
    x = np.moveaxis(np.pad(sp, pad), sparse_dim, -1)
    x = x.reshape(*x.shape[:-1], -1, m)
    return bool(((x != 0).sum(-1) <= n).all())


def perfect_nm(x, sparse_dim, n, m):
    S = x.shape[sparse_dim]
    pad = [(0, 0)] * x.ndim
    pad[sparse_dim] = (0, -(-S // m) * m - S)
    y = np.moveaxis(np.pad(x, pad), sparse_dim, -1)
    shp = y.shape
    y = y.reshape(*shp[:-1], -1, m)
    kth = np.sort(np.abs(y), axis=-1)[..., m - n][..., None]
    keep = np.abs(y) >= kth
    return (np.abs(y) * keep).sum()


def test_sparsify_invariants_reference_test_shapes():
    # shapes / n:m:g / seed style of tests/test_nmg.py:33-86 (uniform [0,1) inputs)
    rng = np.random.default_rng(123)
    n, m, g = 5, 12, 2
    dims = [17, 5, 1]
    for a, b in itertools.product(dims, dims):
        base = rng.random((3, a, b), dtype=np.float32)
        for perm in itertools.permutations(range(3)):
            x = np.ascontiguousarray(np.transpose(base, perm))
            layout = "".join("abc"[i] for i in perm)
            sparse_dim, group_dim = layout.index("c"), layout.index("b")
            val, idx, lay = O.sparsify(x, n, m, sparse_dim, g, group_dim)
            cols = lay.c * g
            flat = idx.reshape(lay.outer, cols)
            assert (np.sort(flat, axis=1) == np.arange(cols)).all()
            sp = O.to_dense(val, idx, lay)
            assert sp.shape == x.shape
            assert is_correct_nm(x, sp, sparse_dim, n, m)
            kept = np.abs(sp).sum() / np.abs(x).sum()
            assert kept > n / m
            assert perfect_nm(x, sparse_dim, n, m) / np.abs(x).sum() >= kept - 1e-5


def test_sparsify_fp16_is_upcast_algorithm_downcast():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((32, 48)) * 0.02).astype(np.float16)
    v16, i16, _ = O.sparsify(x, 2, 4, 1, 4, 0)
    v32, i32, _ = O.sparsify(x.astype(np.float32), 2, 4, 1, 4, 0)
    assert np.array_equal(i16, i32)
    assert v16.dtype == np.float16 and np.array_equal(v16.astype(np.float32), v32)


def test_sparsify_rejects_wide_tiles():
    with pytest.raises(ValueError):
        O.sparsify_merged(np.zeros((1, 792, 42, 12), dtype=np.float32), 5)  # 792*42 >= 2**15


# ------------------------------------------------------------------- to_dense / merge

def test_merge_unmerge_roundtrip_all_dim_pairs():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 17, 5)).astype(np.float32)
    for sd, gd in itertools.permutations(range(3), 2):
        lay = O.Layout(x.shape, 2, 4, 2, sd, gd)
        mm = O.merge(x, lay)
        assert mm.shape == (lay.outer, 6, 2, 4)
        assert np.array_equal(O.unmerge(mm, lay), x)


def test_merge_element_formula():
    # tile (kc, mb), column j, row r  ==  Wpad[mb*m + r, kc*c*g + j]   (2-D, sparse dim 0)
    W = np.arange(10 * 30, dtype=np.float32).reshape(10, 30)
    lay = O.Layout(W.shape, 2, 4, 2, 0, 1)
    mm = O.merge(W, lay).reshape(lay.num_chunks, lay.num_blocks, 12, 4)
    Wp = np.pad(W, [(0, 2), (0, 6)])
    for kc, mb, j, r in [(0, 0, 0, 0), (1, 2, 5, 3), (2, 1, 11, 2), (2, 2, 7, 1)]:
        assert mm[kc, mb, j, r] == Wp[mb * 4 + r, kc * 12 + j]


def test_to_dense_scatter_closed_form():
    rng = np.random.default_rng(2)
    n, m, g = 2, 4, 3
    c = 6
    val = rng.standard_normal((2, c, g, n)).astype(np.float32)
    idx = np.stack([rng.permutation(c * g) for _ in range(2)]).reshape(2, c, g, 1).astype(np.int16)
    dense = O.to_dense_merged(val, idx, m).reshape(2, c * g, m)
    order = tuples(n, m)
    want = np.zeros_like(dense)
    for t in range(2):
        for slot in range(c * g):
            for j in range(n):
                want[t, idx.reshape(2, -1)[t, slot], order[slot // g][j]] = val.reshape(2, -1, n)[t, slot, j]
    assert np.array_equal(dense, want)


def test_gather_inverts_to_dense():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((24, 36)).astype(np.float32)
    val, idx, lay = O.sparsify(x, 2, 4, 0, 3, 1)
    again = O.gather_merged(O.merge(O.to_dense(val, idx, lay), lay), idx, 2)
    assert np.array_equal(again, val)


# ------------------------------------------------------------------------------- spmm

@pytest.mark.parametrize("M,K,N,n,m,g", [
    (768, 768, 256, 2, 4, 16),   # benchmark config 1 shape
    (50, 200, 64, 2, 4, 4),      # M and K remainders
    (23, 95, 128, 3, 6, 2),
    (97, 97, 64, 1, 8, 3),       # K one past a tile boundary
    (16, 96, 64, 2, 4, 16),      # exactly one tile
    (16, 95, 64, 2, 4, 16),      # tile boundary - 1
    (33, 130, 192, 4, 8, 1),
])
def test_spmm_equals_dense_equation(M, K, N, n, m, g):
    # the equation the reference asserts: C[:M,:N] == to_dense(A) @ B (dace_gnm_mult.py:1123,1189-1199)
    rng = np.random.default_rng(M + K)
    W = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    val, idx, lay = O.sparsify(W, n, m, 0, g, 1)
    ref = O.to_dense(val, idx, lay).astype(np.float64) @ B.astype(np.float64)
    for fn in (O.spmm, O.simd_spmm):
        C = fn(val, idx, lay, B)
        rel = np.linalg.norm(C - ref) / np.linalg.norm(ref)
        assert rel < 1e-6


def test_simd_spmm_rejects_ragged_n():
    W = np.ones((8, 24), dtype=np.float32)
    val, idx, lay = O.sparsify(W, 2, 4, 0, 1, 1)
    with pytest.raises(ValueError):  # N % (4*v) != 0 (dace_gnm_mult.py:605-606)
        O.simd_spmm(val, idx, lay, np.ones((24, 10), dtype=np.float32))


def test_linear_matches_dense():
    rng = np.random.default_rng(9)
    W = rng.standard_normal((20, 36)).astype(np.float32)
    x = rng.standard_normal((2, 5, 36)).astype(np.float32)
    b = rng.standard_normal(20).astype(np.float32)
    val, idx, lay = O.sparsify(W, 2, 4, 0, 3, 1)
    y = O.linear(x, val, idx, lay, b)
    ref = x @ O.to_dense(val, idx, lay).T + b
    assert np.allclose(y, ref, rtol=1e-5, atol=1e-5)
