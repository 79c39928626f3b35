"""sten_amd.plugin.register against a stand-in for a STen installation: a second, empty instance
of the dispatch module (real STen cannot be imported here: it needs dace and cpuinfo).  Host logic
only -- nothing is computed."""
import importlib.util
import os

import pytest
import torch

import sten_amd
from sten_amd import impls, perfect, plugin, w4
from sten_amd.tensor import GroupedNMTensor


def fresh_registry():
    path = os.path.join(os.path.dirname(sten_amd.__file__), "dispatch.py")
    spec = importlib.util.spec_from_file_location("fake_sten", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_register_installs_every_key_and_can_run_twice():
    sten = fresh_registry()
    assert not sten.SPARSIFIER_IMPLEMENTATIONS
    plugin.register(sten)
    keys = set(sten.SPARSIFIER_IMPLEMENTATIONS)
    for key in [(impls.GroupedNMSparsifier, torch.Tensor, GroupedNMTensor),
                (sten.SameFormatSparsifier, torch.Tensor, GroupedNMTensor),
                (sten.KeepAll, GroupedNMTensor, sten.DenseTensor),
                (w4.SparseMarlinSparsifier, torch.Tensor, w4.SparseMarlinTensor),
                (perfect.PerfectNMSparsifier, torch.Tensor, perfect.PerfectNMTensor)]:
        assert key in keys, key
    # operators: F.linear with and without bias, torch.mm, forward and both backward flavours
    lin = torch.nn.functional.linear
    assert sten.get_fwd_op_impl(lin, (torch.Tensor, GroupedNMTensor), [(sten.KeepAll, torch.Tensor)]) is not None
    assert sten.get_fwd_op_impl(lin, (torch.Tensor, GroupedNMTensor, torch.Tensor),
                                [(sten.KeepAll, torch.Tensor)]) is not None
    assert sten.get_fwd_op_impl(torch.mm, (GroupedNMTensor, torch.Tensor), [(sten.KeepAll, torch.Tensor)]) is not None
    dense, nmg = (sten.KeepAll, torch.Tensor), (sten.KeepAll, GroupedNMTensor)
    for grad_w in (dense, nmg):
        assert sten.get_bwd_op_impl(lin, (torch.Tensor,), (dense, grad_w), (torch.Tensor, GroupedNMTensor)) is not None
        assert sten.get_bwd_op_impl(torch.mm, (torch.Tensor,), (grad_w, dense), (GroupedNMTensor, torch.Tensor)) is not None
    # the names user code uses
    assert sten.GroupedNMTensor is GroupedNMTensor and sten.GroupedNMSparsifier is impls.GroupedNMSparsifier
    assert sten.PerfectNMTensor is perfect.PerfectNMTensor
    # STen refuses a second registration of a sparsifier key (sten.py:1096-1100): register removes
    # what it replaces first, so it can run again
    plugin.register(sten)
    assert set(sten.SPARSIFIER_IMPLEMENTATIONS) == keys
    with pytest.raises(Exception):
        sten.register_sparsifier_implementation(
            sparsifier=impls.GroupedNMSparsifier, inp=torch.Tensor, out=GroupedNMTensor)(lambda *a: None)


def test_orientation_switch_for_unchanged_user_code():
    sten = fresh_registry()
    try:
        plugin.register(sten)
        sp = sten.GroupedNMSparsifier(2, 4, 16)
        assert (sp.sparse_dim, sp.group_dim) == (-2, -1)              # the reference's orientation
        plugin.register(sten, nm_along_reduction=True)
        sp = sten.GroupedNMSparsifier(2, 4, 16)
        assert (sp.sparse_dim, sp.group_dim) == (-1, -2)              # n:m along the reduction of F.linear
        sp = sten.GroupedNMSparsifier(2, 4, 16, sparse_dim=-2, group_dim=-1)
        assert (sp.sparse_dim, sp.group_dim) == (-2, -1)              # explicit dims always win
    finally:
        impls.GroupedNMSparsifier.default_dims = (-2, -1)
