"""The C ABI library loads on a machine without a GPU and exports what include/nmg_hip.h declares."""
import ctypes
import os
import re

import pytest

from sten_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "nmg_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nmg_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert "nmg_sparsify" in names and "nmg_spmm" in names
    lib = ctypes.CDLL(native.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), f"{name} declared in nmg_hip.h but not exported"
        assert name in native.SIGNATURES, f"{name} has no ctypes signature in sten_amd.native"
    assert sorted(native.SIGNATURES) == names


def test_order_table_is_served_by_the_library_on_cpu():
    assert native.order_table(2, 4) == [(0, 1), (0, 2), (1, 2), (1, 3), (0, 3), (2, 3)]
    assert [t[0] for t in native.order_table(1, 8)] == [5, 3, 1, 0, 2, 4, 6, 7]
    with pytest.raises(native.NmgError):
        native.order_table(5, 4)


def test_product_order_equals_oracle_order():
    from oracle import nmg_oracle as O
    for m in range(1, 13):
        for n in range(0, m + 1):
            assert native.order_table(n, m) == [tuple(int(x) for x in t) for t in O.order(n, m)]


def test_argument_errors_need_no_gpu():
    lib = native.load()
    view = native.NmgView(1, 8, 8, 0, 8, 1)
    one = ctypes.c_void_p(8)  # never dereferenced: validation fails first
    rc = lib.nmg_sparsify(one, ctypes.byref(view), one, one, 5, 12, 42, native.NMG_F32, None)
    assert rc == 1 and b"2^15" in lib.nmg_last_error()
    rc = lib.nmg_sparsify(one, ctypes.byref(view), one, one, 3, 2, 1, native.NMG_F32, None)
    assert rc == 1
    rc = lib.nmg_spmm(one, one, 8, 8, one, 8, one, 8, None, 4, 1, 2, 4, 9, 0, None)
    assert rc == 1 and b"dtype" in lib.nmg_last_error()
    assert lib.nmg_spmm(one, one, 8, 8, one, 4, one, 8, None, 4, 1, 2, 4, native.NMG_F16, 0, None) == 1


def test_split_reduction_plan_and_argument_errors():
    lib = native.load()
    slices, ws = ctypes.c_int(0), ctypes.c_int64(0)
    plan = lambda M, K, T: (lib.nmg_splitk_plan(M, K, T, ctypes.byref(slices), ctypes.byref(ws)),
                            slices.value, ws.value)
    assert plan(4096, 11008, 64) == (0, 8, 8 * 64 * 4096 * 4)         # 16 tiles -> 8 slices of 22 K steps
    assert plan(4096, 11008, 512) == (0, 4, 4 * 512 * 4096 * 4)
    assert plan(4096, 11008, 16) == (0, 1, 0)                         # decode shapes are not split
    assert plan(4096, 11008, 2048) == (0, 1, 0)                       # enough tiles
    assert plan(4096, 200, 64) == (0, 1, 0)                           # K % 64 != 0
    assert plan(1000, 256, 64)[1] == 1                                # four K steps: too short to cut
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    args = lambda sl, wsb: (one, one, 512, 1152, one, 1152, one, 512, None, 40, native.NMG_F16, sl, one, wsb, None)
    assert lib.nmg_spmm_smfmac_splitk(*args(17, 1 << 30)) == 1 and b"empty" in lib.nmg_last_error()
    assert lib.nmg_spmm_smfmac_splitk(*args(2, 100)) == 1 and b"workspace" in lib.nmg_last_error()


def test_cpu_tensors_are_refused_loudly():
    import torch
    import sten_amd as sten
    with pytest.raises(sten.NmgError):
        sten.GroupedNMTensor.from_dense(torch.zeros(8, 8), 2, 4, 1, 1, 0)
