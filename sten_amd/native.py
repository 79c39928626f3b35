"""ctypes binding of libnmg_hip.so (the C ABI declared in include/nmg_hip.h).

The library is built in-tree by ``sten_amd.build`` and loaded from this directory.  There is
no CPU implementation behind these calls: if the library is missing, or a kernel is asked to
run on a non-GPU tensor, the call raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnmg_hip.so")

NMG_F32, NMG_F16, NMG_BF16, NMG_F64 = 0, 1, 2, 3
KERNEL_AUTO, KERNEL_MFMA, KERNEL_SMFMAC, KERNEL_SKINNY = 0, 1, 2, 3
KERNELS = {"auto": KERNEL_AUTO, "mfma": KERNEL_MFMA, "smfmac": KERNEL_SMFMAC, "skinny": KERNEL_SKINNY,
           "expand": KERNEL_MFMA, "densefrag": KERNEL_MFMA, "gstream": KERNEL_SKINNY, "sstream": KERNEL_SKINNY, "ostream": KERNEL_SKINNY}

DTYPE_CODE = {
    torch.float32: NMG_F32,
    torch.float16: NMG_F16,
    torch.bfloat16: NMG_BF16,
    torch.float64: NMG_F64,
}


class NmgError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


class NmgView(ctypes.Structure):
    _fields_ = [(name, ctypes.c_int64)
                for name in ("batch", "G", "S", "stride_b", "stride_g", "stride_s")]


_P, _I, _I64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
_VP = ctypes.POINTER(NmgView)

# name -> (restype, argtypes); must list every symbol include/nmg_hip.h declares
SIGNATURES = {
    "nmg_version": (_I, []),
    "nmg_last_error": (ctypes.c_char_p, []),
    "nmg_order": (_I64, [_I, _I, _P]),
    "nmg_chunk": (_I64, [_I, _I]),
    "nmg_sparsify": (_I, [_P, _VP, _P, _P, _I, _I, _I, _I, _P]),
    "nmg_to_dense": (_I, [_P, _P, _P, _VP, _I, _I, _I, _I, _P]),
    "nmg_gather": (_I, [_P, _VP, _P, _P, _I, _I, _I, _I, _P]),
    "nmg_rowpack_pat_bytes": (_I64, [_I, _I]),
    "nmg_rowpack": (_I, [_P, _P, _I64, _I64, _P, _P, _I, _I, _I, _I, _P]),
    "nmg_rowpack_expand": (_I, [_P, _P, _I64, _I64, _P, _I64, _I, _I, _I, _I, _P]),
    "nmg_densefrag_supported": (_I, [_I, _I]),
    "nmg_densefrag_elems": (_I, [_I64, _I64, ctypes.POINTER(ctypes.c_int64)]),
    "nmg_densefrag": (_I, [_P, _P, _I64, _I64, _I, _P, _I, _I, _I, _P]),
    "nmg_spmm_densefrag": (_I, [_P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _P]),
    "nmg_spmm_densefrag_splitk": (_I, [_P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _P, _I64, _P]),
    "nmg_spmm_densefrag_tt": (_I, [_P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _P]),
    "nmg_w4_sizes": (_I, [_I64, _I64] + [ctypes.POINTER(ctypes.c_int64)] * 3),
    "nmg_w4_pack": (_I, [_P, _I64, _I64, _I64, _P, _P, _P, _P]),
    "nmg_w4_to_dense": (_I, [_P, _P, _P, _I64, _I64, _P, _I64, _P]),
    "nmg_w4_linear": (_I, [_P, _P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _P]),
    "nmg_spmm": (_I, [_P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _I, _I, _I, _P]),
    "nmg_fragpack_supported": (_I, [_I, _I]),
    "nmg_fragpack_sizes": (_I, [_I64, _I64, ctypes.POINTER(_I64), ctypes.POINTER(_I64)]),
    "nmg_fragpack": (_I, [_P, _P, _I64, _I64, _P, _P, _I, _I, _I, _P]),
    "nmg_pack_operands": (_I, [_P, _P, _I64, _I64, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "nmg_spmm_smfmac": (_I, [_P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _P]),
    "nmg_splitk_plan": (_I, [_I64, _I64, _I64, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64)]),
    "nmg_spmm_smfmac_splitk": (_I, [_P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _P, _I64, _P]),
    "nmg_slotmap": (_I, [_P, _I64, _I64, _P, _I, _I, _I, _P]),
    "nmg_sddmm": (_I, [_P, _I64, _P, _I64, _I64, _P, _I64, _I64, _P, _I, _I, _I, _I, _P]),
    "nmg_sddmm_nt": (_I, [_P, _I64, _P, _I64, _I64, _P, _I64, _I64, _P, _I, _I, _I, _I, _P]),
    "nmg_perfect_nm": (_I, [_P, _I64, _I64, _I64, _P, _P, _I, _I, _I, _P]),
    "nmg_perfect_nm_to_dense": (_I, [_P, _P, _I64, _I64, _I64, _P, _I, _I, _I, _P]),
    "nmg_noalloc_scratch_bytes": (_I64, []),
    "nmg_noalloc_prepare": (_I, []),
    "nmg_spmm_smfmac_splitk_noalloc": (_I, [_P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _P]),
    "nmg_spmm_smfmac_tt": (_I, [_P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _P]),
    "nmg_spmm_gstream_supported": (_I, [_I, _I]),
    "nmg_spmm_gstream_plan": (_I, [_I64, _I64, _I64, _I, _I, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64)]),
    "nmg_gpack_bytes": (_I, [_I64, _I64, _I, _I, ctypes.POINTER(ctypes.c_int64)]),
    "nmg_gpack": (_I, [_P, _P, _I64, _I64, _I, _I, _P, _I, _P]),
    "nmg_spmm_gstream": (_I, [_P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _I, _P, _I64, _P]),
    "nmg_spmm_ostream_supported": (_I, [_I, _I]),
    "nmg_opack_bytes": (_I, [_I64, _I64, _I, _I, ctypes.POINTER(ctypes.c_int64)]),
    "nmg_opack": (_I, [_P, _P, _I64, _I64, _I, _I, _P, _I, _P]),
    "nmg_spmm_ostream": (_I, [_P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _I, _P]),
    "nmg_spmm_sstream_supported": (_I, [_I, _I]),
    "nmg_lanepack8_sizes": (_I, [_I64, _I64, _I, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]),
    "nmg_lanepack8": (_I, [_P, _P, _I64, _I64, _I, _P, _P, _I, _P]),
    "nmg_spmm_sstream": (_I, [_P, _P, _I64, _I64, _P, _I64, _P, _I64, _P, _I64, _I, _I, _I, _P]),
    "nmg_gemm_nt": (_I, [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I, _P]),
    "nmg_gemm_nn": (_I, [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I, _P]),
    "nmg_gemm_tn": (_I, [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I, _P]),
}

_lib = None


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NmgError(
                f"{LIB_PATH} is missing: build it with `python -m sten_amd.build` "
                "(there is no fallback implementation)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise NmgError(f"nmg call failed with status {rc}: {load().nmg_last_error().decode()}")


def dtype_code(dtype):
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise NmgError(f"unsupported dtype {dtype}") from None


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise NmgError(
                f"nmg kernels run on the GPU only; got a tensor on {t.device} "
                "(move the tensor to an MI355X device)")


def stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def order_table(n, m):
    """Pattern order as a list of tuples (host call, no GPU needed)."""
    lib = load()
    c = lib.nmg_chunk(n, m)
    buf = (ctypes.c_int8 * max(1, c * n))()
    got = lib.nmg_order(n, m, buf)
    if got != c:
        raise NmgError(f"invalid n:m = {n}:{m}")
    return [tuple(buf[i * n + j] for j in range(n)) for i in range(c)]
