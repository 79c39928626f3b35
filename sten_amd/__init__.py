"""sten_amd -- the grouped n:m (nmg) sparse path of STen, written for MI355X (gfx950).

The module exposes the STen names that the path touches, so user code written against
``import sten`` runs with ``import sten_amd as sten``.
"""
from . import dispatch
from .dispatch import (DISPATCH_RAISE, DISPATCH_WARN, DenseTensor, DispatchError, DispatchWarning,
                       KeepAll, SameFormatSparsifier, SparseOperatorDispatcher,
                       SparseParameterWrapper, SparseTensorWrapper, SparsityBuilder,
                       get_bwd_op_impl, get_fwd_op_impl, get_sparsifier_implementation,
                       register_bwd_op_impl, register_fwd_op_impl,
                       register_sparsifier_implementation, set_dispatch_failure, sparsified_op,
                       unregister_sparsifier_implementation)
from .impls import GroupedNMSparsifier, install
from .layout import NMGLayout
from .native import NmgError
from . import perfect
from .perfect import PerfectNMSparsifier, PerfectNMTensor, is_correct_nm
from .tensor import GroupedNMTensor, spmm, spmm_tt, spmm_tt_dense
from . import w4
from .w4 import SparseMarlinSparsifier, SparseMarlinTensor

install(dispatch)
w4.install(dispatch)
perfect.install(dispatch)

__all__ = [n for n in dir() if not n.startswith("_")]
