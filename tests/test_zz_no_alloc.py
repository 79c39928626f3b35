"""The split reduction that allocates nothing (nmg_spmm_smfmac_splitk_noalloc), called through the
C ABI and compared bit for bit with nmg_spmm_smfmac_splitk on a caller-owned workspace: two calls
in a row, the second on a smaller input, so that what the first call left in the library's
scratch array must not matter.  Collected last on purpose: a failure here hides no other test."""
import ctypes

import pytest
import torch

import sten_amd as sten
from sten_amd import native
from helpers import seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(lib, w, x, bias, slices, noalloc):
    lay = w.layout
    M, K = lay.dense_shape
    T = x.shape[0]
    fp_val, fp_idx = w.fragpack()
    y = torch.full((T, M), float("nan"), dtype=x.dtype, device=DEV)
    common = (native.ptr(fp_val), native.ptr(fp_idx), M, K, native.ptr(x), x.stride(0), native.ptr(y), M,
              native.ptr(bias), T, native.dtype_code(x.dtype), slices)
    if noalloc:
        rc = lib.nmg_spmm_smfmac_splitk_noalloc(*common, native.stream_ptr(x.device))
    else:
        ws = torch.empty(slices * T * ((M + 255) // 256) * 256, dtype=torch.float32, device=DEV)
        rc = lib.nmg_spmm_smfmac_splitk(*common, native.ptr(ws), ws.numel() * 4, native.stream_ptr(x.device))
    native.check(rc)
    torch.cuda.synchronize()
    return y


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_two_calls_in_a_row_match_the_workspace_entry_point(dtype):
    lib = native.load()
    assert lib.nmg_noalloc_scratch_bytes() == 32 << 20
    native.check(lib.nmg_noalloc_prepare())
    big = sten.GroupedNMTensor.from_dense(seeded((1024, 2048), dtype, seed=1, std=0.05).to(DEV), 2, 4,
                                          sparse_dim=1, group_size=16, group_dim=0)
    small = sten.GroupedNMTensor.from_dense(seeded((300, 512), dtype, seed=2, std=0.05).to(DEV), 2, 4,
                                            sparse_dim=1, group_size=16, group_dim=0)
    cases = [(big, seeded((200, 2048), dtype, seed=3).to(DEV), seeded((1024,), dtype, seed=4).to(DEV), 4),
             (small, seeded((40, 512), dtype, seed=5).to(DEV), None, 2)]
    for w, x, bias, slices in cases:
        print(f"case noalloc {dtype} weight {tuple(w.layout.dense_shape)} tokens {x.shape[0]} slices {slices}", flush=True)
        want = _call(lib, w, x, bias, slices, noalloc=False)
        before = torch.cuda.memory_allocated(DEV)
        got = _call(lib, w, x, bias, slices, noalloc=True)
        assert torch.equal(got, want)
        assert not bool(torch.isnan(got.float()).any())
        # torch's allocator saw the output of the call and nothing else (blocks are rounded to 512 bytes)
        assert torch.cuda.memory_allocated(DEV) - before <= got.numel() * got.element_size() + 512
    # once more in the other order: large after small
    w, x, bias, slices = cases[0]
    assert torch.equal(_call(lib, w, x, bias, slices, noalloc=True), _call(lib, w, x, bias, slices, noalloc=False))


def test_sizes_beyond_the_scratch_are_refused():
    lib = native.load()
    w = sten.GroupedNMTensor.from_dense(seeded((512, 1024), torch.float16, seed=6, std=0.05).to(DEV), 2, 4,
                                        sparse_dim=1, group_size=16, group_dim=0)
    fp_val, fp_idx = w.fragpack()
    T = 20000                                   # 8 slices x 20000 tokens x 512 features x 4 bytes = 328 MB
    x = torch.zeros(T, 1024, dtype=torch.float16, device=DEV)
    y = torch.zeros(T, 512, dtype=torch.float16, device=DEV)
    rc = lib.nmg_spmm_smfmac_splitk_noalloc(native.ptr(fp_val), native.ptr(fp_idx), 512, 1024, native.ptr(x), 1024,
                                            native.ptr(y), 512, None, T, native.NMG_F16, 8, None)
    assert rc == 2 and b"scratch holds" in lib.nmg_last_error()
    # one slice needs no scratch at all and is served whatever the size
    rc = lib.nmg_spmm_smfmac_splitk_noalloc(native.ptr(fp_val), native.ptr(fp_idx), 512, 1024, native.ptr(x), 1024,
                                            native.ptr(y), 512, None, T, native.NMG_F16, 1, None)
    assert rc == 0
    torch.cuda.synchronize()
