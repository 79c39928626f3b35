"""Committed fixtures (tests/golden/): hand-traced known answers of the reference algorithm and
frozen oracle outputs.  The CPU tests hold the oracle to them, the GPU tests the HIP path."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import nmg_oracle as O
from helpers import rel_l2, same_bits, to_np

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
HAND = json.load(open(os.path.join(HERE, "hand_traced.json")))
VEC = np.load(os.path.join(HERE, "regression_vectors.npz"))
CASES = sorted({k.split(".")[0] for k in VEC.files})
TOL = {np.dtype(np.float16): 1e-3, np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-5}


@pytest.mark.parametrize("key", sorted(HAND["orders"]))
def test_oracle_order_tables(key):
    n, m = map(int, key.split(":"))
    assert O.order(n, m).tolist() == HAND["orders"][key]


@pytest.mark.parametrize("i", range(len(HAND["tiles"])))
def test_oracle_hand_worked_tiles(i):
    t = HAND["tiles"][i]
    d = np.array([t["tile"]], dtype=np.float32)
    val, idx = O.sparsify_merged(d, t["n"])
    assert idx.ravel().tolist() == t["idx"]
    assert val.reshape(-1, max(t["n"], 1)).tolist() == t["val"]


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_frozen_vectors(name):
    n, m, g, sd, gd = VEC[name + ".meta"].tolist()
    x = VEC[name + ".x"]
    val, idx, lay = O.sparsify(x, n, m, sd, g, gd)
    assert np.array_equal(idx, VEC[name + ".idx"])
    assert np.array_equal(val.astype(x.dtype), VEC[name + ".val"])
    assert np.array_equal(O.to_dense(val, idx, lay).astype(x.dtype), VEC[name + ".dense"])


# ------------------------------------------------------------------------------------ GPU

@pytest.mark.parametrize("key", sorted(HAND["orders"]))
def test_library_order_tables(key):
    # host-side entry point of the HIP library (nmg_order): no GPU needed
    from sten_amd import native
    n, m = map(int, key.split(":"))
    assert [list(t) for t in native.order_table(n, m)] == HAND["orders"][key]


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(len(HAND["tiles"])))
def test_hip_hand_worked_tiles(i):
    import sten_amd as sten
    t = HAND["tiles"][i]
    n, m, g = t["n"], t["m"], t["g"]
    tile = torch.tensor(t["tile"], dtype=torch.float32)          # [c, g, m]
    c = tile.shape[0]
    # one tile as a 2-D weight: columns of the tile are lines of dim 0, the block of m runs along dim 1
    w = tile.reshape(c * g, m).to("cuda:0")
    s = sten.GroupedNMTensor.from_dense(w, n, m, sparse_dim=1, group_size=g, group_dim=0)
    assert to_np(s.idx).ravel().tolist() == t["idx"]
    assert to_np(s.val).reshape(-1, max(n, 1)).tolist() == t["val"]


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_hip_reproduces_frozen_vectors(name):
    import sten_amd as sten
    n, m, g, sd, gd = VEC[name + ".meta"].tolist()
    x = VEC[name + ".x"]
    xt = torch.from_numpy(x).to("cuda:0")
    s = sten.GroupedNMTensor.from_dense(xt, n, m, sparse_dim=sd, group_size=g, group_dim=gd)
    assert np.array_equal(to_np(s.idx), VEC[name + ".idx"])
    assert same_bits(s.val, VEC[name + ".val"])
    assert same_bits(s.to_dense(), VEC[name + ".dense"])
    if x.dtype != np.float64:
        act = torch.from_numpy(VEC[name + ".act"]).to("cuda:0")
        y = sten.spmm(s, act, reduce_dim=1)
        assert rel_l2(to_np(y), VEC[name + ".y"]) <= TOL[x.dtype]
