"""The one-pass derivation of the matmul operands (nmg_pack_operands) against the two scatter
kernels it replaces (nmg_rowpack, nmg_fragpack): both operands must come out bit for bit."""
import ctypes

import pytest
import torch

import sten_amd as sten
from sten_amd import native
from helpers import seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def two_step(t):
    lay, lib = t.layout, native.load()
    dt, dev = t.val.dtype, t.val.device
    pat_bytes = lib.nmg_rowpack_pat_bytes(lay.n, lay.m)
    pk_val = torch.empty((lay.G, lay.num_blocks, lay.n), dtype=dt, device=dev)
    pk_pat = torch.empty((lay.G, lay.num_blocks), dtype=torch.uint8 if pat_bytes == 1 else torch.int16, device=dev)
    native.check(lib.nmg_rowpack(native.ptr(t.val), native.ptr(t.idx), lay.G, lay.S, native.ptr(pk_val),
                                 native.ptr(pk_pat), lay.n, lay.m, lay.group_size, native.dtype_code(dt),
                                 native.stream_ptr(dev)))
    fp = None
    if dt in (torch.float16, torch.bfloat16) and lib.nmg_fragpack_supported(lay.n, lay.m):
        ve, iw = ctypes.c_int64(), ctypes.c_int64()
        native.check(lib.nmg_fragpack_sizes(lay.G, lay.S, ctypes.byref(ve), ctypes.byref(iw)))
        fp_val = torch.empty(ve.value, dtype=dt, device=dev)
        fp_idx = torch.empty(iw.value, dtype=torch.int32, device=dev)
        native.check(lib.nmg_fragpack(native.ptr(pk_val), native.ptr(pk_pat), lay.G, lay.S, native.ptr(fp_val),
                                      native.ptr(fp_idx), lay.n, lay.m, native.dtype_code(dt),
                                      native.stream_ptr(dev)))
        fp = (fp_val, fp_idx)
    return pk_val, pk_pat, fp


def bits(x):
    return x.view(torch.int16) if x.dtype in (torch.float16, torch.bfloat16) else x.view(torch.int32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("G,S,n,m,g", [
    (4096, 1024, 2, 4, 16),     # whole chunks and fragments
    (300, 520, 2, 4, 16),       # ragged lines; positions not a multiple of 64
    (96 * 3 + 1, 201, 2, 4, 16),  # positions not a multiple of m
    (70, 64, 2, 4, 4),          # 24-line chunks: a workgroup spans four of them
    (500, 256, 1, 4, 8),
    (1000, 192, 1, 8, 32),
    (1900, 136, 2, 8, 32),      # 896-line chunks
    (333, 96, 2, 8, 4),
    (130, 130, 1, 2, 16),
    (2300, 72, 4, 8, 32),       # no sparse-matrix-core operand: rowpack alone
    (200, 90, 3, 6, 4),         # m not a power of two
    (100, 48, 5, 12, 2),        # 792 patterns: 16-bit pattern numbers, scatter kernels
])
def test_one_pass_matches_the_scatter_kernels(dtype, G, S, n, m, g):
    print(f"case pack {dtype} G={G} S={S} {n}:{m}:{g}", flush=True)
    t = sten.GroupedNMTensor.from_dense(seeded((G, S), dtype, seed=G + S, std=0.5).to(DEV), n, m,
                                        sparse_dim=1, group_size=g, group_dim=0)
    pk_val, pk_pat, fp = two_step(t)
    got_val, got_pat = t.rowpack()
    assert torch.equal(bits(got_val), bits(pk_val)) and torch.equal(got_pat, pk_pat)
    got_fp = t.fragpack()
    assert (got_fp is None) == (fp is None)
    if fp is not None:
        assert torch.equal(bits(got_fp[0]), bits(fp[0])), "fragment values"
        assert torch.equal(got_fp[1], fp[1]), "fragment index words"


def test_rejects_fragments_for_an_incompatible_pattern():
    t = sten.GroupedNMTensor.from_dense(seeded((64, 64), torch.float16, seed=1).to(DEV), 4, 8, 1, 2, 0)
    lib = native.load()
    dummy = torch.empty(16, dtype=torch.float16, device=DEV)
    rc = lib.nmg_pack_operands(native.ptr(t.val), native.ptr(t.idx), 64, 64, native.ptr(dummy), native.ptr(dummy),
                               native.ptr(dummy), native.ptr(dummy), 4, 8, 2, native.dtype_code(torch.float16),
                               native.stream_ptr(t.val.device))
    assert rc != 0
