"""Sparsifier and operator implementations of the grouped n:m format, registered through the
STen dispatch API (the reference registers its own in src/sten/grouped_nm/sten_impls.py:13-37
and :143-174; it has no ``torch.mm``, no backward and no ``SameFormatSparsifier`` entry -- those
are defined here by dense autograd of the same operators).

``install(api)`` registers everything into any module that exposes the STen registration
functions: this package's own ``dispatch`` module, or a real ``sten``.
"""
import torch

from . import native
from .tensor import GroupedNMTensor, spmm, spmm_tt, spmm_tt_dense


class GroupedNMSparsifier:
    """n:m:g magnitude sparsifier.  Reference signature ``(n, m, g)`` (sten_impls.py:13-17); the
    default orientation is the reference's (n:m blocks along dim -2, grouping along dim -1).
    ``sparse_dim`` / ``group_dim`` select another one, e.g. ``sparse_dim=-1, group_dim=-2`` puts
    the n:m blocks along the reduction dim of ``F.linear``."""

    # orientation used when the caller names none: the reference's.  `plugin.register(sten,
    # nm_along_reduction=True)` switches it to (-1, -2) for unchanged user code that wants the
    # n:m blocks along the reduction dim of F.linear, where the sparse matrix cores can use them.
    default_dims = (-2, -1)

    def __init__(self, n, m, g, sparse_dim=None, group_dim=None):
        self.n, self.m, self.g = n, m, g
        self.sparse_dim = type(self).default_dims[0] if sparse_dim is None else sparse_dim
        self.group_dim = type(self).default_dims[1] if group_dim is None else group_dim


def _masked_weight_grad(weight, lhs_t, rhs):
    """val-layout gradient: the kept positions of ``lhs_t^T @ rhs`` (``lhs_t`` [T, rows of W],
    ``rhs`` [T, columns of W]).  16-bit weights take the fused kernel, which never stores the dense
    product; fp32 (``nmg_gemm_tn``) and extents that are not multiples of 8 go through the dense
    product and the same-pattern gather."""
    if rhs.dtype != weight.dtype:
        rhs = rhs.to(weight.dtype)
    if weight.masked_product_supported(lhs_t, rhs):
        return weight.masked_product(lhs_t, rhs)
    if rhs.dtype == torch.float32 and lhs_t.dtype == torch.float32 and lhs_t.is_cuda and lhs_t.shape[0] > 0:
        # single precision: the dense product on the fp32 matrix cores, operands as they lie
        # (both reduction-major), then the gather
        return weight.clone_layout(_f32_product("tn", lhs_t, rhs))
    return weight.clone_layout(_dense_product("tn", lhs_t, rhs))


def _f32_product(form, x, a):
    """Dense fp32 product on this library's matrix-core GEMM, operands as they lie in memory:
    ``"tn"``: x [K, T], a [K, O] -> x^T @ a;  ``"nt"``: x [T, K], a [O, K] -> x @ a^T."""
    return _dense_product(form, x, a)


def _dense_product(form, x, a):
    """Dense product on this library's matrix-core kernels, operands as they lie in memory:
    ``"tn"``: x [K, T], a [K, O] -> x^T @ a (``nmg_gemm_tn``);  ``"nt"``: x [T, K], a [O, K] -> x @ a^T
    (``nmg_gemm_nt``).  fp32 always; 16-bit types where the kernels take the shape (extents and
    pitches that are multiples of 8, 16-byte aligned bases; ``"nt"``: K a multiple of 64) -- other
    16-bit shapes go through the fp32 kernel (operands widened, result rounded once); only what
    that does not take either (double, more than 2 097 120 tokens) goes to ``torch.mm``."""
    dt = x.dtype
    if form == "tn":
        (K, T), O = x.shape, a.shape[1]
    else:
        (T, K), O = x.shape, a.shape[0]
    ok = x.is_cuda and a.dtype == dt and dt in native.DTYPE_CODE and dt != torch.float64 and T > 0 and O > 0 and K > 0
    if ok:
        x = x if x.stride(1) == 1 else x.contiguous()
        a = a if a.stride(1) == 1 else a.contiguous()
    if ok and dt != torch.float32:
        ok = (x.stride(0) % 8 == 0 and a.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and a.data_ptr() % 16 == 0
              and O % 8 == 0 and max(x.stride(0), a.stride(0)) < 2 ** 24)
        if form == "tn":
            ok = ok and T % 8 == 0
        else:
            ok = ok and K % 64 == 0 and O * a.stride(0) * 2 < 2 ** 31 and T * x.stride(0) * 2 < 2 ** 31
    if ok and dt == torch.float32:
        ok = (T + 31) // 32 <= 65535
    if not ok:
        if (x.is_cuda and a.dtype == dt and dt in (torch.float16, torch.bfloat16) and T > 0 and O > 0 and K > 0
                and (T + 31) // 32 <= 65535):
            return _dense_product(form, x.float(), a.float()).to(dt)
        return torch.mm(x.t(), a) if form == "tn" else torch.mm(x, a.t())
    entry = native.load().nmg_gemm_tn if form == "tn" else native.load().nmg_gemm_nt
    y = torch.empty((T, O), dtype=dt, device=x.device)
    with torch.cuda.device(x.device):
        native.check(entry(native.ptr(a), a.stride(0), native.ptr(x), x.stride(0), native.ptr(y), O,
                           None, O, K, T, native.dtype_code(dt), native.stream_ptr(x.device)))
    return y


def install(api):
    KeepAll, SameFormat = api.KeepAll, api.SameFormatSparsifier
    wrap = api.SparseTensorWrapper.wrapped_from_dense
    dense_fmt = (KeepAll, torch.Tensor)
    nmg_fmt = (KeepAll, GroupedNMTensor)

    # ---- sparsifiers -----------------------------------------------------------------------
    @api.register_sparsifier_implementation(
        sparsifier=GroupedNMSparsifier, inp=torch.Tensor, out=GroupedNMTensor)
    def dense_to_grouped_nm(sparsifier, tensor, grad_fmt=None):
        gnm = GroupedNMTensor.from_dense(
            tensor, sparsifier.n, sparsifier.m,
            sparse_dim=getattr(sparsifier, "sparse_dim", -2) % tensor.dim(),
            group_size=sparsifier.g,
            group_dim=getattr(sparsifier, "group_dim", -1) % tensor.dim())
        return wrap(gnm, tensor, grad_fmt)

    @api.register_sparsifier_implementation(
        sparsifier=SameFormat, inp=torch.Tensor, out=GroupedNMTensor)
    def dense_to_same_grouped_nm(sparsifier, tensor, grad_fmt=None):
        ref = sparsifier.ref_sp_ten
        ref_fmt = ref.wrapped_tensor if hasattr(ref, "wrapped_tensor") else ref
        return wrap(ref_fmt.clone_layout(tensor), tensor,
                    grad_fmt if grad_fmt is not None else getattr(ref, "grad_fmt", None))

    @api.register_sparsifier_implementation(
        sparsifier=KeepAll, inp=GroupedNMTensor, out=api.DenseTensor)
    def grouped_nm_to_dense_tensor(sparsifier, tensor, grad_fmt=None):
        dense = tensor.wrapped_tensor.to_dense()
        return wrap(api.DenseTensor(dense), dense, grad_fmt)

    # ---- F.linear(x, W_nmg[, b]) -----------------------------------------------------------
    def linear_fwd(ctx, inputs, output_sparsifiers):
        x, weight = inputs[0], inputs[1]
        bias = inputs[2] if len(inputs) > 2 else None
        ctx.save_for_backward(*inputs)
        w = weight.wrapped_tensor
        x2 = x.reshape(-1, x.shape[-1])
        y = spmm(w, x2, bias, reduce_dim=1)
        return y.reshape(*x.shape[:-1], y.shape[-1])

    def linear_bwd_common(ctx, grad_outputs, compressed):
        saved = ctx.saved_tensors
        x, weight = saved[0], saved[1]
        [gy] = grad_outputs
        w = weight.wrapped_tensor
        gy2 = gy.reshape(-1, gy.shape[-1])
        x2 = x.reshape(-1, x.shape[-1])
        if gy2.dtype != w.dtype:
            gy2 = gy2.to(w.dtype)
        gx = spmm(w, gy2.contiguous(), reduce_dim=0).reshape(x.shape)
        if compressed:
            gw = wrap(_masked_weight_grad(w, gy2, x2), x2)
        else:
            # the dense weight gradient dY^T X from the operands as they lie (both token-major)
            gw = _dense_product("tn", gy2, x2 if x2.dtype == gy2.dtype else x2.to(gy2.dtype))
        grads = [gx, gw]
        if len(saved) > 2:
            grads.append(gy2.sum(dim=0))
        return tuple(grads)

    for arity in (2, 3):
        fmts = (torch.Tensor, GroupedNMTensor) + (torch.Tensor,) * (arity - 2)
        api.register_fwd_op_impl(operator=torch.nn.functional.linear, inp=fmts, out=[dense_fmt])(linear_fwd)
        api.register_bwd_op_impl(
            operator=torch.nn.functional.linear, grad_out=(torch.Tensor,),
            grad_inp=(dense_fmt,) * arity, inp=fmts,
        )(lambda ctx, g, s: linear_bwd_common(ctx, g, compressed=False))
        api.register_bwd_op_impl(
            operator=torch.nn.functional.linear, grad_out=(torch.Tensor,),
            grad_inp=(dense_fmt, nmg_fmt) + (dense_fmt,) * (arity - 2), inp=fmts,
        )(lambda ctx, g, s: linear_bwd_common(ctx, g, compressed=True))

    # ---- torch.mm(W_nmg, B) -----------------------------------------------------------------
    @api.register_fwd_op_impl(operator=torch.mm, inp=(GroupedNMTensor, torch.Tensor), out=[dense_fmt])
    def mm_fwd(ctx, inputs, output_sparsifiers):
        weight, b = inputs
        ctx.save_for_backward(weight, b)
        return spmm_tt(weight.wrapped_tensor, b)

    def mm_bwd_common(ctx, grad_outputs, compressed):
        weight, b = ctx.saved_tensors
        [gc] = grad_outputs
        w = weight.wrapped_tensor
        gc = gc.to(w.dtype)
        gb = spmm_tt_dense(w, gc, reduce_dim=0)     # W^T @ grad_out, both as they lie in memory
        if compressed:
            # grad_out [R, N] and B [C, N] are reduction-contiguous as they lie: no transposing copies
            if w.masked_product_supported(gc, b, reduction_last=True):
                gw = wrap(w.masked_product(gc, b, reduction_last=True), gc)
            elif gc.dtype == torch.float32 and b.dtype == torch.float32 and gc.shape[1] > 0:
                gw = wrap(w.clone_layout(_f32_product("nt", gc, b)), gc)     # grad_out @ B^T
            else:
                gw = wrap(_masked_weight_grad(w, gc.t(), b.t()), gc)
        else:
            gw = _dense_product("nt", gc, b if b.dtype == gc.dtype else b.to(gc.dtype))     # grad_out @ B^T
        return gw, gb

    api.register_bwd_op_impl(
        operator=torch.mm, grad_out=(torch.Tensor,), grad_inp=(dense_fmt, dense_fmt),
        inp=(GroupedNMTensor, torch.Tensor),
    )(lambda ctx, g, s: mm_bwd_common(ctx, g, compressed=False))
    api.register_bwd_op_impl(
        operator=torch.mm, grad_out=(torch.Tensor,), grad_inp=(nmg_fmt, dense_fmt),
        inp=(GroupedNMTensor, torch.Tensor),
    )(lambda ctx, g, s: mm_bwd_common(ctx, g, compressed=True))

    return {"dense_to_grouped_nm": dense_to_grouped_nm,
            "dense_to_same_grouped_nm": dense_to_same_grouped_nm}
