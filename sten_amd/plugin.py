"""Install the MI355X grouped n:m implementations into a real STen installation.

    import sten, sten_amd.plugin
    sten_amd.plugin.register(sten)

replaces STen's CPU/CUDA ``GroupedNMTensor`` sparsifier and ``F.linear`` implementation
(src/sten/grouped_nm/sten_impls.py:20-37, :143-174) with the HIP ones and adds ``torch.mm``, the
backward implementations and the ``SameFormatSparsifier`` entry.  STen refuses a second
registration of a sparsifier key (sten.py:1096-1100), so existing keys are removed first.
"""
import torch

from . import impls, perfect, w4
from .tensor import GroupedNMTensor


def register(sten_module, nm_along_reduction=False):
    """Install the implementations into ``sten_module``.  ``nm_along_reduction=True`` also makes
    ``GroupedNMSparsifier(n, m, g)`` (no dims given) put the n:m blocks along the last dim -- the
    reduction dim of ``F.linear`` -- instead of the reference's dim -2: unchanged user code then
    reaches the sparse matrix cores in forward, at the price of a pattern that differs from the one
    the reference would choose for the same call."""
    impls.GroupedNMSparsifier.default_dims = (-1, -2) if nm_along_reduction else (-2, -1)
    reg = getattr(sten_module, "SPARSIFIER_IMPLEMENTATIONS", None)
    if reg is None and hasattr(sten_module, "sten"):
        reg = sten_module.sten.SPARSIFIER_IMPLEMENTATIONS
    keys = [
        (impls.GroupedNMSparsifier, torch.Tensor, GroupedNMTensor),
        (sten_module.SameFormatSparsifier, torch.Tensor, GroupedNMTensor),
        (sten_module.KeepAll, GroupedNMTensor, sten_module.DenseTensor),
    ]
    for key in keys:
        if reg is not None and key in reg:
            sten_module.unregister_sparsifier_implementation(*key)
    # expose the GPU classes under the names user code already uses
    sten_module.GroupedNMTensor = GroupedNMTensor
    sten_module.GroupedNMSparsifier = impls.GroupedNMSparsifier
    impls.install(sten_module)
    w4_key = (w4.SparseMarlinSparsifier, torch.Tensor, w4.SparseMarlinTensor)
    if reg is None or w4_key not in reg:
        w4.install(sten_module)
    pf_key = (perfect.PerfectNMSparsifier, torch.Tensor, perfect.PerfectNMTensor)
    if reg is None or pf_key not in reg:
        perfect.install(sten_module)
    sten_module.PerfectNMTensor = perfect.PerfectNMTensor
    sten_module.PerfectNMSparsifier = perfect.PerfectNMSparsifier
