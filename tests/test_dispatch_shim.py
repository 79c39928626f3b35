"""Host-side contract of the STen-compatible dispatch (runs without a GPU, with a toy format).
Patterns restated from the reference's tests/test_api.py:245-413 (custom format + operator
registration), :421-450 and :512-551 (optimizer steps, grad_fmt survival)."""
import copy
import io
import warnings

import pytest
import torch

import sten_amd as sten


class MaskFmt:
    """Dense values + fixed 0/1 mask: the simplest format with a pattern to preserve."""

    def __init__(self, val, mask):
        self.val, self.mask = val, mask

    def to_dense(self):
        return self.val * self.mask

    @property
    def dtype(self):
        return self.val.dtype

    @property
    def device(self):
        return self.val.device

    def add_(self, other, *, alpha=1):
        o = other.wrapped_tensor.to_dense() if hasattr(other, "wrapped_tensor") else other
        self.val.add_(o * self.mask, alpha=alpha)
        return self


class EvenSparsifier:
    pass


def _mask_like(t):
    return (torch.arange(t.numel()).reshape(t.shape) % 2 == 0).to(t.dtype)


@sten.register_sparsifier_implementation(sparsifier=EvenSparsifier, inp=torch.Tensor, out=MaskFmt)
def _to_mask(sp, t, grad_fmt=None):
    mask = _mask_like(t)
    return sten.SparseTensorWrapper.wrapped_from_dense(MaskFmt(t.detach().clone() * mask, mask), t, grad_fmt)


@sten.register_sparsifier_implementation(sparsifier=sten.SameFormatSparsifier, inp=torch.Tensor, out=MaskFmt)
def _same_mask(sp, t, grad_fmt=None):
    ref = sp.ref_sp_ten.wrapped_tensor
    return sten.SparseTensorWrapper.wrapped_from_dense(MaskFmt(t.detach().clone() * ref.mask, ref.mask), t, grad_fmt)


@sten.register_fwd_op_impl(operator=torch.nn.functional.linear,
                           inp=(torch.Tensor, MaskFmt, torch.Tensor), out=[(sten.KeepAll, torch.Tensor)])
def _lin_fwd(ctx, inputs, output_sparsifiers):
    x, w, b = inputs
    ctx.save_for_backward(x, w, b)
    return x @ w.wrapped_tensor.to_dense().t() + b


@sten.register_bwd_op_impl(operator=torch.nn.functional.linear, grad_out=(torch.Tensor,),
                           grad_inp=((sten.KeepAll, torch.Tensor),) * 3,
                           inp=(torch.Tensor, MaskFmt, torch.Tensor))
def _lin_bwd(ctx, grad_outputs, input_sparsifiers):
    x, w, b = ctx.saved_tensors
    [g] = grad_outputs
    return g @ w.wrapped_tensor.to_dense(), g.t() @ x, g.sum(0)


def sparse_linear(seed=0):
    torch.manual_seed(seed)
    model = torch.nn.Linear(6, 4)
    ref = copy.deepcopy(model)
    sb = sten.SparsityBuilder()
    sb.set_weight("weight", initial_sparsifier=EvenSparsifier(), out_format=MaskFmt)
    return model, ref, sb


def test_key_canonicalisation_and_duplicate_registration():
    assert sten.dispatch._canon_formats((torch.Tensor, torch.Tensor)) is None
    assert sten.dispatch._canon_sp_formats([(sten.KeepAll, torch.Tensor)]) is None
    assert sten.dispatch._canon_formats((torch.Tensor, MaskFmt)) == (torch.Tensor, MaskFmt)
    with pytest.raises(Exception, match="second time"):
        sten.register_sparsifier_implementation(sparsifier=EvenSparsifier, inp=torch.Tensor, out=MaskFmt)(_to_mask)

    class Tmp:
        pass

    sten.register_sparsifier_implementation(sparsifier=Tmp, inp=torch.Tensor, out=MaskFmt)(_to_mask)
    sten.unregister_sparsifier_implementation(Tmp, torch.Tensor, MaskFmt)
    with pytest.raises(sten.DispatchError):
        sten.get_sparsifier_implementation(Tmp, torch.Tensor, MaskFmt)


def test_grouped_nm_entries_are_registered():
    F = torch.nn.functional
    G = sten.GroupedNMTensor
    assert (sten.GroupedNMSparsifier, torch.Tensor, G) in sten.dispatch.SPARSIFIER_IMPLEMENTATIONS
    assert (sten.SameFormatSparsifier, torch.Tensor, G) in sten.dispatch.SPARSIFIER_IMPLEMENTATIONS
    sten.get_fwd_op_impl(F.linear, (torch.Tensor, G, torch.Tensor), None)
    sten.get_fwd_op_impl(F.linear, (torch.Tensor, G), None)          # bias=None changes the arity
    sten.get_fwd_op_impl(torch.mm, (G, torch.Tensor), None)
    sten.get_bwd_op_impl(F.linear, None, None, (torch.Tensor, G, torch.Tensor))
    sten.get_bwd_op_impl(F.linear, None, ((sten.KeepAll, torch.Tensor), (sten.KeepAll, G), (sten.KeepAll, torch.Tensor)),
                         (torch.Tensor, G, torch.Tensor))
    sten.get_bwd_op_impl(torch.mm, None, None, (G, torch.Tensor))


def test_builder_forward_backward_match_dense():
    sten.set_dispatch_failure("raise")
    model, ref, sb = sparse_linear()
    model = sb.sparsify_model_inplace(model)
    assert isinstance(model.weight, sten.SparseParameterWrapper) and model.weight.requires_grad
    mask = model.weight.wrapped_tensor.mask
    with torch.no_grad():
        ref.weight.mul_(mask)
    x = torch.randn(3, 6)
    y, yr = model(x), ref(x)
    assert torch.allclose(y, yr)
    y.sum().backward()
    yr.sum().backward()
    assert isinstance(model.weight.grad, sten.SparseTensorWrapper)
    assert isinstance(model.weight.grad.wrapped_tensor, sten.DenseTensor)
    assert torch.allclose(model.weight.grad.wrapped_tensor.to_dense(), ref.weight.grad)
    assert torch.allclose(model.bias.grad, ref.bias.grad)


def test_optimizer_steps_and_grad_fmt_survive():
    model, ref, sb = sparse_linear(1)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9)
    model, opt = sb.sparsify_model_and_optimizer_inplace(model, opt)
    assert any(p is model.weight for g in opt.param_groups for p in g["params"])
    mask = model.weight.wrapped_tensor.mask
    with torch.no_grad():
        ref.weight.mul_(mask)
    ropt = torch.optim.SGD(ref.parameters(), lr=0.1, momentum=0.9)
    fmt0 = model.weight.grad_fmt
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for _ in range(3):
            x = torch.randn(5, 6)
            model(x).sum().backward()
            ref(x).sum().backward()
            with torch.no_grad():
                ref.weight.grad.mul_(mask)
            opt.step(); ropt.step()
            opt.zero_grad(); ropt.zero_grad()
    assert torch.allclose(model.weight.wrapped_tensor.to_dense(), ref.weight * mask, atol=1e-6)
    assert model.weight.grad_fmt[3] is fmt0[3] and model.weight.requires_grad
    adam = torch.optim.AdamW(model.parameters())
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for _ in range(2):
            model(torch.randn(5, 6)).sum().backward()
            adam.step()
            adam.zero_grad()
    dense = model.weight.wrapped_tensor.to_dense()
    assert bool(((dense != 0) <= (mask != 0)).all())


def test_unregistered_operator_falls_back_or_raises():
    w = _to_mask(EvenSparsifier(), torch.randn(4, 4))
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        out = torch.relu(w)                      # warn mode: dense fallback
    assert torch.equal(out, torch.relu(w.wrapped_tensor.to_dense()))
    sten.set_dispatch_failure("raise")
    w2 = _to_mask(EvenSparsifier(), torch.randn(4, 4))   # dispatch decisions are cached per tensor
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        with pytest.raises(sten.DispatchError):
            torch.relu(w2)


def test_wrapper_copy_detach_pickle():
    w = _to_mask(EvenSparsifier(), torch.randn(4, 4).requires_grad_(True))
    d = w.detach()
    assert not d.requires_grad and d.wrapped_tensor is w.wrapped_tensor
    c = w.clone()
    assert c.wrapped_tensor is not w.wrapped_tensor
    assert torch.equal(c.wrapped_tensor.to_dense(), w.wrapped_tensor.to_dense())
    lin = torch.nn.Linear(4, 4)
    lin.weight = sten.SparseParameterWrapper(w)
    buf = io.BytesIO()
    torch.save(lin, buf)
    buf.seek(0)
    back = torch.load(buf, weights_only=False)
    assert isinstance(back.weight, sten.SparseParameterWrapper)
    assert torch.equal(back.weight.wrapped_tensor.to_dense(), w.wrapped_tensor.to_dense())


def test_layout_geometry_matches_oracle_layout():
    from oracle import nmg_oracle as O
    for shape, n, m, g, sd, gd in [((768, 768), 2, 4, 16, 1, 0), ((4096, 4096), 2, 4, 16, 1, 0),
                                   ((8192, 8192), 2, 8, 32, 1, 0), ((3, 17, 5), 5, 12, 2, 2, 1),
                                   ((50, 200), 3, 6, 4, 0, 1)]:
        a = sten.NMGLayout(shape, n, m, g, sd, gd)
        b = O.Layout(shape, n, m, g, sd, gd)
        assert (a.outer, a.num_chunks, a.num_blocks, a.chunk_size) == (b.outer, b.num_chunks, b.num_blocks, b.c)
        assert a.padded_dense_shape == b.padded_shape
    lay = sten.NMGLayout((4096, 4096), 2, 4, 16, 1, 0)
    assert lay.outer == 44032 and lay.padded_dense_shape == (4128, 4096)   # benchmark config 2: 43 chunks of 96 lines x 1024 blocks
    with pytest.raises(ValueError):
        sten.NMGLayout((8, 8), 5, 12, 42, 1, 0)
