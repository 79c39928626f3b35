"""A small, protocol-compatible stand-in for STen's sparsifier / operator dispatch.

Only the contract that the grouped n:m path plugs into is provided -- the registries, the
wrapper tensors, the autograd dispatcher and the weight branch of ``SparsityBuilder`` -- with
the same names, key canonicalisation and call signatures as the reference
(src/sten/sten.py:1068-1324 registries, :91-270 wrappers, :1557-1736 dispatcher,
:1809-1928 ``sparsified_op``, :720-1019 builder).  When a real ``sten`` is importable the same
implementations can be installed into it instead (see ``sten_amd.plugin``).

Contract summary
  * sparsifier implementation: ``fn(sparsifier, tensor, grad_fmt=None) -> SparseTensorWrapper``,
    key ``(sparsifier class, input format, output format)``; registering a key twice raises.
  * forward implementation: ``fn(ctx, inputs, output_sparsifiers)``; ``inputs`` are the tensor
    arguments of the call, flattened, positional before keyword.
  * backward implementation: ``fn(ctx, grad_outputs, input_sparsifiers) -> grads`` (one per input).
  * all-dense keys are canonicalised to ``None``.
  * a tensor's ``grad_fmt`` is ``(inline sparsifier, tmp format, external sparsifier, format)``.
"""
import copy
import inspect
import types
import warnings

import torch

DISPATCH_RAISE = "raise"
DISPATCH_WARN = "warn"
_dispatch_failure = [DISPATCH_WARN]


def set_dispatch_failure(action):
    if action not in (DISPATCH_RAISE, DISPATCH_WARN):
        raise ValueError("Unknown action")
    _dispatch_failure[0] = action


class DispatchWarning(Warning):
    pass


class DispatchError(Warning):  # the reference derives it from Warning as well (sten.py:75)
    pass


class DenseTensor:
    """Dense payload inside a wrapper (lets a dense tensor carry a sparse gradient format)."""

    def __init__(self, data):
        self.data = data

    def to_dense(self):
        return self.data


class KeepAll:
    def __eq__(self, other):
        return type(other) == type(self)

    def __hash__(self):
        return hash(KeepAll)


class SameFormatSparsifier:
    """Re-sparsify a dense result into the format (and pattern) of ``ref_sp_ten``."""

    def __init__(self, ref_sp_ten):
        self.ref_sp_ten = ref_sp_ten


# ------------------------------------------------------------------------------- registries

SPARSIFIER_IMPLEMENTATIONS = {}
FWD_OP_IMPLS = {}
BWD_OP_IMPLS = {}


def _canon_formats(fmts):
    if fmts is None or all(f is torch.Tensor for f in fmts):
        return None
    return tuple(fmts)


def _canon_sp_formats(pairs):
    if pairs is None or all((s is KeepAll and f is torch.Tensor) for s, f in pairs):
        return None
    return tuple(tuple(p) for p in pairs)


def register_sparsifier_implementation(sparsifier, inp, out):
    def decorator(func):
        key = (sparsifier, inp, out)
        if key in SPARSIFIER_IMPLEMENTATIONS:
            raise Exception(
                "Trying to register sparsifier implementation second time! "
                "Use unregister_sparsifier_implementation to remove existing implementation.")
        SPARSIFIER_IMPLEMENTATIONS[key] = func
        return func

    return decorator


def unregister_sparsifier_implementation(sparsifier, inp, out):
    del SPARSIFIER_IMPLEMENTATIONS[(sparsifier, inp, out)]


def get_sparsifier_implementation(sparsifier, inp, out):
    if (sparsifier, inp, out) == (type(None), None, None):
        return lambda sp, ten: ten
    if sparsifier == KeepAll and inp == out:
        return lambda sp, ten: ten
    if sparsifier in (KeepAll, SameFormatSparsifier) and inp == torch.Tensor and out == DenseTensor:
        return lambda sp, ten: SparseTensorWrapper.wrapped_from_dense(
            DenseTensor(ten.clone().detach()), ten)
    impl = SPARSIFIER_IMPLEMENTATIONS.get((sparsifier, inp, out))
    if impl is not None:
        return impl
    msg = (f"Sparsifier implementation is not registered: sparsifier={_name(sparsifier)}, "
           f"inp={_name(inp)}, out={_name(out)}")
    if _dispatch_failure[0] == DISPATCH_WARN and inp != torch.Tensor:
        warnings.warn(msg + "; densifying the input first", DispatchWarning)
        via_dense = get_sparsifier_implementation(sparsifier, torch.Tensor, out)
        return lambda sp, ten: via_dense(sp, ten.wrapped_tensor.to_dense())
    raise DispatchError(msg)


def register_fwd_op_impl(operator, inp, out):
    key = (operator, _canon_formats(inp), _canon_sp_formats(out))

    def decorator(func):
        FWD_OP_IMPLS[key] = func
        return func

    return decorator


def get_fwd_op_impl(operator, inp, out):
    key = (operator, _canon_formats(inp), _canon_sp_formats(out))
    impl = FWD_OP_IMPLS.get(key)
    if impl is None:
        raise DispatchError(
            f"Sparse operator implementation is not registered (fwd): operator={_op_name(operator)}, "
            f"inp={_name(key[1])}, out={_name(key[2])}")
    return impl


def register_bwd_op_impl(operator, grad_out, grad_inp, inp):
    key = (operator, _canon_formats(grad_out), _canon_sp_formats(grad_inp), _canon_formats(inp))

    def decorator(func):
        BWD_OP_IMPLS[key] = func
        return func

    return decorator


def get_bwd_op_impl(operator, grad_out, grad_inp, inp):
    key = (operator, _canon_formats(grad_out), _canon_sp_formats(grad_inp), _canon_formats(inp))
    impl = BWD_OP_IMPLS.get(key)
    if impl is None:
        raise DispatchError(
            f"Sparse operator implementation is not registered (bwd): operator={_op_name(operator)}, "
            f"grad_out={_name(key[1])}, grad_inp={_name(key[2])}, inp={_name(key[3])}")
    return impl


def _name(obj):
    if isinstance(obj, (list, tuple)):
        return "(" + ", ".join(_name(o) for o in obj) + ")"
    if inspect.isclass(obj):
        return obj.__qualname__ if obj.__module__ in ("builtins", "__main__") else f"{obj.__module__}.{obj.__qualname__}"
    return str(obj)


def _op_name(op):
    try:
        return torch.overrides.resolve_name(op) or getattr(op, "__name__", str(op))
    except Exception:
        return getattr(op, "__name__", str(op))


# ----------------------------------------------------------------------------- tree helpers

class _Leaf:
    __slots__ = ("i",)

    def __init__(self, i):
        self.i = i

    def __eq__(self, other):
        return isinstance(other, _Leaf) and other.i == self.i


def _flatten(tree, out):
    """Replace every tensor in a nest of list/tuple/dict by a _Leaf; collect tensors in ``out``."""
    if isinstance(tree, torch.Tensor):
        out.append(tree)
        return _Leaf(len(out) - 1)
    if type(tree) in (list, tuple):
        return type(tree)(_flatten(x, out) for x in tree)
    if type(tree) is dict:
        return {k: _flatten(v, out) for k, v in tree.items()}
    return tree


def _unflatten(tree, flat):
    if isinstance(tree, _Leaf):
        return flat[tree.i]
    if type(tree) in (list, tuple):
        return type(tree)(_unflatten(x, flat) for x in tree)
    if type(tree) is dict:
        return {k: _unflatten(v, flat) for k, v in tree.items()}
    return tree


def _is_sparse(t):
    return isinstance(t, SparseTensorWrapper)


def _dense_of(t):
    return t.wrapped_tensor.to_dense() if _is_sparse(t) else t


def get_format(tensor):
    if hasattr(tensor, "wrapped_tensor"):
        return tensor.wrapped_tensor.__class__
    if isinstance(tensor, torch.Tensor):
        return torch.Tensor
    return None


def _has_format(tensor, fmt):
    if not hasattr(tensor, "wrapped_tensor"):
        return (isinstance(tensor, torch.Tensor) and fmt == torch.Tensor) or fmt is None
    return tensor.wrapped_tensor.__class__ == fmt


# --------------------------------------------------------------------------- wrapper tensors

_PLAIN_FUNCS = set()  # torch functions that run on the wrapper's own (dummy) tensor data
for _f in (
    torch.Tensor.register_hook,
    torch.Tensor.requires_grad.__get__,
    torch.Tensor._backward_hooks.__set__,
    torch.Tensor.grad.__set__,
    torch.Tensor.grad.__get__,
    torch.Tensor.is_leaf.__get__,
    torch.Tensor.grad_fn.__get__,
    torch.Tensor.__hash__,
    torch.Tensor.is_sparse.__get__,
    torch.Tensor.retain_grad,
    torch.Tensor.retains_grad.__get__,
    torch.Tensor.output_nr.__get__,
    torch.Tensor._version.__get__,
    torch.Tensor.name.__get__,
    torch.Tensor.names.__get__,
):
    _PLAIN_FUNCS.add(_f)


class SparseTensorWrapper(torch.Tensor):
    """A ``torch.Tensor`` subclass whose real payload is ``wrapped_tensor`` (any object with
    ``to_dense()``); its own storage is a one-element placeholder so autograd can track it."""

    @staticmethod
    def wrapped_from_dense(wrapped, dense, grad_fmt=None):
        if grad_fmt is None:
            grad_fmt = (KeepAll(), torch.Tensor, KeepAll(), DenseTensor)
        return SparseTensorWrapper([wrapped], dense.requires_grad, grad_fmt)

    def __new__(cls, wrapped_tensor_container, requires_grad, grad_fmt, *, dummy_shape=None):
        wt = wrapped_tensor_container[0]
        assert not isinstance(wt, SparseTensorWrapper)
        dtype = wt.dtype if hasattr(wt, "dtype") else wt.to_dense().dtype
        device = wt.device if hasattr(wt, "device") else wt.to_dense().device
        if not (dtype.is_floating_point or dtype.is_complex):
            requires_grad = False
        placeholder = torch.zeros([1], dtype=dtype, device=device)
        tensor = torch.Tensor._make_subclass(cls, placeholder, requires_grad)
        tensor._wrapped_tensor_container = wrapped_tensor_container
        tensor.grad_fmt = grad_fmt
        tensor._sync_grad_hook()
        return tensor

    # autograd hands plain tensors to .grad; keep the wrapper instead (sten.py:92-102)
    def _grad_hook(self, grad):
        self.grad = grad

    def _sync_grad_hook(self):
        has = hasattr(self, "_grad_hook_handle")
        if self.requires_grad and not has:
            self._grad_hook_handle = self.register_hook(self._grad_hook)
        elif not self.requires_grad and has:
            self._grad_hook_handle.remove()
            del self._grad_hook_handle

    @property
    def wrapped_tensor(self):
        return self._wrapped_tensor_container[0]

    @wrapped_tensor.setter
    def wrapped_tensor(self, value):
        self._wrapped_tensor_container[0] = value

    def init_from_other(self, other, replace_attributes=True):
        assert isinstance(other, SparseTensorWrapper)
        self.wrapped_tensor = other.wrapped_tensor
        if replace_attributes:
            self.requires_grad = other.requires_grad
            self.grad_fmt = other.grad_fmt

    def __copy__(self):
        return sparse_tensor_builder(type(self), self._wrapped_tensor_container, self.requires_grad,
                                     self.grad_fmt)

    def __deepcopy__(self, memo):
        if id(self) in memo:
            return memo[id(self)]
        result = sparse_tensor_builder(type(self), copy.deepcopy(self._wrapped_tensor_container),
                                       bool(self.requires_grad), copy.deepcopy(self.grad_fmt))
        if self.grad is not None:
            g = copy.deepcopy(self.grad)
            result.grad = g if not isinstance(g, SparseTensorWrapper) else SparseTensorWrapper(
                g._wrapped_tensor_container, g.requires_grad, g.grad_fmt)
        memo[id(self)] = result
        return result

    def __reduce_ex__(self, proto):
        return (sparse_tensor_builder,
                (type(self), self._wrapped_tensor_container, self.requires_grad, self.grad_fmt))

    def __repr__(self):
        return f"SparseTensorWrapper:\n{self.wrapped_tensor}"

    def __mul__(self, rhs):
        return torch.mul(self, rhs)

    def __rmul__(self, lhs):
        return torch.mul(lhs, self)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        try:
            handler = _HANDLERS.get(func)
            if handler is not None:
                return handler(func, types, args, kwargs)
            if func in _PLAIN_FUNCS:
                return super().__torch_function__(func, types, args, kwargs)
            return _route(func, args, kwargs)
        except Exception as e:
            warnings.warn(f"Exception raised during handling __torch_function__ ({func}): {e}")
            raise


class SparseParameterWrapper(SparseTensorWrapper, torch.nn.parameter.Parameter):
    def __new__(cls, sparse_tensor_wrapper):
        assert isinstance(sparse_tensor_wrapper, SparseTensorWrapper)
        return super().__new__(cls, sparse_tensor_wrapper._wrapped_tensor_container,
                               sparse_tensor_wrapper.requires_grad, sparse_tensor_wrapper.grad_fmt)

    def __repr__(self):
        return "SparseParameterWrapper containing:\n" + super().__repr__()

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        types = tuple(SparseTensorWrapper if t is SparseParameterWrapper else t for t in types)
        return SparseTensorWrapper.__torch_function__(func, types, args, kwargs)


def sparse_tensor_builder(wrapper_type, container, requires_grad, grad_fmt):
    result = SparseTensorWrapper(container, requires_grad, grad_fmt)
    if wrapper_type is SparseParameterWrapper:
        result = SparseParameterWrapper(result)
    return result


_HANDLERS = {}


def _plain_call(func, args, kwargs):
    """Run ``func`` on the wrappers' own placeholder tensors, without re-entering dispatch."""
    with torch._C.DisableTorchFunctionSubclass():
        return func(*args, **kwargs)


def _handles(*funcs):
    def deco(fn):
        for f in funcs:
            _HANDLERS[f] = fn
        return fn

    return deco


@_handles(torch.Tensor.requires_grad_, torch.Tensor.requires_grad.__set__)
def _h_requires_grad(func, types, args, kwargs):
    res = _plain_call(func, args, kwargs)
    args[0]._sync_grad_hook()
    return res


@_handles(torch.Tensor.data.__get__, torch.Tensor.detach)
def _h_detach(func, types, args, kwargs):
    return copy.copy(args[0]).requires_grad_(False)


@_handles(torch.Tensor.clone, torch.clone)
def _h_clone(func, types, args, kwargs):
    return copy.deepcopy(args[0])


@_handles(torch.Tensor.data.__set__)
def _h_data_set(func, types, args, kwargs):
    lhs, rhs = args
    if _is_sparse(lhs) and _is_sparse(rhs):
        lhs.wrapped_tensor = rhs.wrapped_tensor
    else:
        _catch_inplace(func, args, kwargs, resparsify=True)


@_handles(torch.Tensor.backward)
def _h_backward(func, types, args, kwargs):
    self = args[0]
    grad = args[1] if len(args) > 1 else kwargs.get("gradient")
    if _is_sparse(grad):
        grad = SparseTensorWrapper(grad._wrapped_tensor_container, grad.requires_grad, grad.grad_fmt)
    rest = dict(kwargs)
    rest.pop("gradient", None)
    return _plain_call(func, (self, grad) + tuple(args[2:]), rest)


@_handles(torch.Tensor.to)
def _h_to(func, types, args, kwargs):
    self = args[0]
    device, dtype = kwargs.get("device"), kwargs.get("dtype")
    rest = list(args[1:])
    if rest and isinstance(rest[0], torch.dtype):
        dtype = rest.pop(0)
    elif rest and isinstance(rest[0], torch.Tensor):
        other = rest.pop(0)
        device, dtype = other.device, other.dtype
    else:
        if rest:
            device = rest.pop(0)
        if rest and isinstance(rest[0], torch.dtype):
            dtype = rest.pop(0)
    wt = self.wrapped_tensor
    device = torch.device(device) if device is not None else wt.device
    dtype = dtype if dtype is not None else wt.dtype
    if device == wt.device and dtype == wt.dtype and not kwargs.get("copy", False):
        return self
    if hasattr(wt, "to"):
        moved = wt.to(device=device, dtype=dtype)
    else:
        impl = get_sparsifier_implementation(SameFormatSparsifier, torch.Tensor, type(wt))
        return impl(SameFormatSparsifier(self), wt.to_dense().to(device=device, dtype=dtype))
    return sparse_tensor_builder(type(self), [moved], self.requires_grad, self.grad_fmt)


def _semantics(func):
    name = getattr(func, "__name__", "")
    if name in ("__get__", "__set__"):
        return "attribute"
    if isinstance(func, types.MethodDescriptorType):
        return "method"
    return "function"


def _is_inplace(func):
    name = getattr(func, "__name__", "")
    if name == "__get__":
        return False
    if name == "__set__":
        return True
    return name.startswith("_") or name.endswith("_")


def _route(func, args, kwargs):
    """Default handling of a torch call that involves a wrapper (sten.py:587-627)."""
    sem = _semantics(func)
    inplace = _is_inplace(func)
    if sem == "attribute":
        if inplace:
            raise NotImplementedError("Attribute assignment is not supported")
        attr = func.__self__.__name__
        self = args[0]
        if hasattr(self.wrapped_tensor, attr):
            return getattr(self.wrapped_tensor, attr)
        return _catch_inplace(func, args, kwargs, resparsify=False)
    if sem == "method":
        self = args[0]
        if hasattr(self, "wrapped_tensor"):
            impl = getattr(type(self.wrapped_tensor), func.__name__, None)
            if impl is not None:
                res = impl(self.wrapped_tensor, *args[1:], **kwargs)
                return self if res is self.wrapped_tensor else res
        if inplace:
            return _catch_inplace(func, args, kwargs, resparsify=_is_sparse(self))
        return _call_sparsified(func, args, kwargs)
    if inplace:
        return _catch_inplace(func, args, kwargs, resparsify=True)
    return _call_sparsified(func, args, kwargs)


def _call_sparsified(func, args, kwargs):
    flat = []
    _flatten((args, kwargs), flat)
    op = None
    for t in flat:
        if _is_sparse(t) and func in getattr(t, "sparsified_ops", {}):
            op = t.sparsified_ops[func]
            break
    if op is None:
        op = sparsified_op(func, None, None)
        for t in flat:
            if _is_sparse(t):
                if not hasattr(t, "sparsified_ops"):
                    t.sparsified_ops = {}
                t.sparsified_ops[func] = op
    return op(*args, **kwargs)


def _catch_inplace(func, args, kwargs, resparsify):
    """Densify every wrapper argument, run ``func``, and write modified dense values back into
    the wrappers with the ``SameFormatSparsifier`` of their format (sten.py:1931-2001)."""
    flat = []
    tree = _flatten((args, kwargs), flat)
    if any(_is_sparse(t) and not isinstance(t.wrapped_tensor, DenseTensor) for t in flat):
        warnings.warn(f"Catching {_op_name(func)} called with the sparse arguments!", DispatchWarning)
    dense = [_dense_of(t) for t in flat]
    before = [d.clone() if (resparsify and _is_sparse(t)) else None for t, d in zip(flat, dense)]
    d_args, d_kwargs = _unflatten(tree, dense)
    with torch.no_grad() if resparsify else _nullcontext():
        out = func(*d_args, **d_kwargs)
    if resparsify:
        for t, d, b in zip(flat, dense, before):
            if b is None:
                continue
            if b.dtype == d.dtype and b.device == d.device and b.shape == d.shape and torch.equal(b, d):
                continue
            impl = get_sparsifier_implementation(SameFormatSparsifier, torch.Tensor,
                                                 t.wrapped_tensor.__class__)
            t.init_from_other(impl(SameFormatSparsifier(t), d), replace_attributes=False)
    out_flat = []
    out_tree = _flatten(out, out_flat)
    if not out_flat:
        return out
    mapped = []
    for o in out_flat:
        hit = None
        for t, d in zip(flat, dense):
            if o is d:
                hit = t
        mapped.append(o if hit is None else hit)
    return _unflatten(out_tree, mapped)


class _nullcontext:
    def __enter__(self):
        return None

    def __exit__(self, *a):
        return False


# ------------------------------------------------------------------------ autograd dispatcher

def _grad_fmt_of(t):
    if _is_sparse(t):
        return t.grad_fmt
    if isinstance(t, torch.Tensor):
        return (KeepAll(), torch.Tensor, KeepAll(), torch.Tensor)
    return (None, None, None, None)


def _dense_formats(fmts):
    return fmts is None or all(f in (None, torch.Tensor, DenseTensor) for f in fmts)


def _dense_sp_formats(pairs):
    if pairs is None:
        return True
    return all(p is None or (p[0] == KeepAll and p[1] in (torch.Tensor, DenseTensor)) for p in pairs)


def _classes(sparsifiers, formats):
    if sparsifiers is None and formats is None:
        return None
    return tuple(((s.__class__, f) if s is not None else None) for s, f in zip(sparsifiers, formats))


def _check_formats(what, tensors, formats):
    formats = formats if formats is not None else tuple(torch.Tensor for _ in tensors)
    if not all(_has_format(t, f) for t, f in zip(tensors, formats)):
        raise KeyError(f"Operator implementation {what} returned outputs in incorrect formats. "
                       f"Expected: {formats}. Returned: {tuple(get_format(t) for t in tensors)}.")


class SparseOperatorDispatcher(torch.autograd.Function):
    """Looks up and runs the registered forward / backward implementation for the formats of
    the actual arguments; falls back to the dense operator when nothing is registered."""

    @staticmethod
    def forward(ctx, state, *tensors):
        ctx.disp_state = state
        if "fwd_impl" not in state:
            state["inp_fmt"] = tuple(get_format(t) for t in tensors)
            state["grad_inp_fmt"] = tuple(_grad_fmt_of(t) for t in tensors)
            out_fmt = state["out_fmt"]
            cols = tuple(zip(*out_fmt)) if out_fmt is not None else (None, None, None, None)
            state["out_cols"] = cols
            state["op_out_fmt"] = _classes(cols[0], cols[1])
            state["fwd_fallback"] = False
            try:
                state["fwd_impl"] = get_fwd_op_impl(state["orig_op"], state["inp_fmt"], state["op_out_fmt"])
            except DispatchError as e:
                if not (_dense_formats(state["inp_fmt"]) and _dense_sp_formats(state["op_out_fmt"])):
                    warnings.warn(f"{e}\nFallback to dense implementation.", DispatchWarning)
                    if _dispatch_failure[0] == DISPATCH_RAISE:
                        raise
                state["fwd_fallback"] = True
                state["fwd_impl"] = _make_dense_fwd(cols[1])
        out_sp1, out_fmt1, out_sp2, out_fmt2 = state["out_cols"]
        tmp = state["fwd_impl"](ctx, tensors, out_sp1)
        flat = []
        tree = _flatten(tmp, flat)
        if "fwd_sp_impls" not in state:
            _check_formats(f"{state['orig_op']} (fwd)", flat, out_fmt1)
            f1 = out_fmt1 if out_fmt1 is not None else tuple(torch.Tensor for _ in flat)
            s2 = out_sp2 if out_sp2 is not None else tuple(KeepAll() for _ in flat)
            f2 = out_fmt2 if out_fmt2 is not None else tuple(torch.Tensor for _ in flat)
            state["fwd_ext"] = (s2, tuple(get_sparsifier_implementation(s.__class__, a, b)
                                          for a, s, b in zip(f1, s2, f2)))
            state["fwd_sp_impls"] = True
        s2, impls = state["fwd_ext"]
        outs = [impl(s, t) for impl, s, t in zip(impls, s2, flat)]
        return _unflatten(tree, outs)

    @staticmethod
    def backward(ctx, *grads):
        state = ctx.disp_state
        ginp_sp1, ginp_fmt1, ginp_sp2, ginp_fmt2 = zip(*state["grad_inp_fmt"])
        if "bwd_impl" not in state:
            actual = tuple(get_format(g) for g in grads)
            gof = state["grad_out_fmt"]
            expected = tuple(zip(*gof))[3] if gof is not None else None
            if _canon_formats(expected) != _canon_formats(actual):
                raise ValueError("Backward implementation received output gradients of incorrect "
                                 f"format. Expected: {gof}. Actual: {actual}.")
            state["gout_fmt"] = expected
            op_ginp = _classes(ginp_sp1, ginp_fmt1)
            try:
                impl = get_bwd_op_impl(state["orig_op"], expected, op_ginp, state["inp_fmt"])
            except DispatchError as e:
                dense = (_dense_formats(expected) and _dense_sp_formats(op_ginp)
                         and _dense_formats(state["inp_fmt"]))
                if dense or (_dispatch_failure[0] == DISPATCH_WARN and state["fwd_fallback"]):
                    impl = _make_dense_bwd(ginp_fmt1)
                elif _dispatch_failure[0] == DISPATCH_RAISE:
                    raise
                else:
                    err = e

                    def impl(ctx, grad_outputs, input_sparsifiers, _err=err):
                        raise DispatchError(_err)
            state["bwd_impl"] = impl
        tmp = state["bwd_impl"](ctx, grads, ginp_sp1)
        tmp = tmp if isinstance(tmp, (tuple, list)) else (tmp,)
        if "bwd_ext" not in state:
            _check_formats(f"{state['orig_op']} (bwd)", tmp, ginp_fmt1)
            state["bwd_ext"] = tuple(get_sparsifier_implementation(s.__class__, a, b)
                                     for a, s, b in zip(ginp_fmt1, ginp_sp2, ginp_fmt2))
        outs = [impl(s, t) for impl, s, t in zip(state["bwd_ext"], ginp_sp2, tmp)]
        fixed = []
        for o in outs:  # fresh wrappers so the placeholder shape matches the input's
            if _is_sparse(o):
                o = SparseTensorWrapper(o._wrapped_tensor_container, o.requires_grad, o.grad_fmt)
            fixed.append(o)
        return (None, *fixed)


def _make_dense_fwd(out_fmt1):
    def dense_fwd(ctx, tensors, output_sparsifiers):
        state = ctx.disp_state
        dense = tuple(d.detach().requires_grad_(d.is_floating_point() or d.is_complex())
                      for d in (_dense_of(t) for t in tensors))
        args, kwargs = _unflatten(state["call_tree"], list(dense))
        with torch.enable_grad():
            outs = state["orig_op"](*args, **kwargs)
        flat = []
        tree = _flatten(outs, flat)
        state["n_fwd_inputs"] = len(dense)
        ctx.save_for_backward(*dense, *flat)
        if "dense_fwd_sp" not in state:
            fmts = out_fmt1 if out_fmt1 is not None else tuple(torch.Tensor for _ in flat)
            sps = output_sparsifiers if output_sparsifiers is not None else tuple(KeepAll() for _ in flat)
            state["dense_fwd_sp"] = (sps, tuple(get_sparsifier_implementation(s.__class__, torch.Tensor, f)
                                                for f, s in zip(fmts, sps)))
        sps, impls = state["dense_fwd_sp"]
        return _unflatten(tree, [impl(s, o.detach()) for impl, s, o in zip(impls, sps, flat)])

    return dense_fwd


def _make_dense_bwd(grad_inp_fmts):
    def dense_bwd(ctx, grad_outputs, input_sparsifiers):
        state = ctx.disp_state
        k = state["n_fwd_inputs"]
        inputs, outputs = ctx.saved_tensors[:k], ctx.saved_tensors[k:]
        pairs = [(o, _dense_of(g)) for o, g in zip(outputs, grad_outputs) if o.requires_grad]
        if pairs:
            torch.autograd.backward([o for o, _ in pairs], grad_tensors=[g for _, g in pairs])
        res = []
        for fmt, sp, inp in zip(grad_inp_fmts, input_sparsifiers, inputs):
            if inp.grad is None:
                res.append(None)
                continue
            impl = get_sparsifier_implementation(sp.__class__, torch.Tensor, fmt)
            res.append(impl(sp, inp.grad))
        return tuple(res)

    return dense_bwd


class SparseOp:
    def __init__(self, orig_op, out_fmt, grad_out_fmt):
        self.orig_op, self.out_fmt, self.grad_out_fmt = orig_op, out_fmt, grad_out_fmt
        self._reset()

    def _reset(self):
        self.disp_state = {"orig_op": self.orig_op, "out_fmt": self.out_fmt,
                           "grad_out_fmt": self.grad_out_fmt}

    def __call__(self, *args, **kwargs):
        flat = []
        tree = _flatten((args, kwargs), flat)
        if self.disp_state.get("call_tree") != tree:
            self._reset()
            self.disp_state["call_tree"] = tree
        outputs = SparseOperatorDispatcher.apply(self.disp_state, *flat)
        outs = outputs if isinstance(outputs, (tuple, list)) else (outputs,)
        gof = self.grad_out_fmt
        for i, o in enumerate(outs):
            if _is_sparse(o):
                o.grad_fmt = tuple(gof[i]) if gof is not None else (KeepAll(), torch.Tensor, KeepAll(), torch.Tensor)
        return outputs


def sparsified_op(orig_op, out_fmt, grad_out_fmt):
    """Operator fused with sparsification of its outputs (sten.py:1875-1928)."""
    if out_fmt is not None or grad_out_fmt is not None:
        dense4 = [KeepAll(), torch.Tensor, KeepAll(), torch.Tensor]
        out_fmt = [list(x) for x in out_fmt] if out_fmt is not None else [list(dense4) for _ in grad_out_fmt]
        grad_out_fmt = ([list(x) for x in grad_out_fmt] if grad_out_fmt is not None
                        else [list(dense4) for _ in out_fmt])
        for o, g in zip(out_fmt, grad_out_fmt):
            if (o[3] == torch.Tensor) != (g[3] == torch.Tensor):
                if o[3] == torch.Tensor:
                    o[3] = DenseTensor
                if g[3] == torch.Tensor:
                    g[3] = DenseTensor
    op = SparseOp(orig_op, out_fmt, grad_out_fmt)

    def wrapper(*args, **kwargs):
        return op(*args, **kwargs)

    return wrapper


# ------------------------------------------------------------------------------- model builder

class SparsityBuilder:
    """Marks module weights for sparsification and swaps them for wrapped parameters
    (weight branch of sten.py:720-1019; intermediate tensors are outside this path)."""

    def __init__(self):
        self.initial_weight_sparsifiers = {}
        self.weights = {}
        self.grad_weights = {}

    def set_weight(self, name, initial_sparsifier=KeepAll(), inline_sparsifier=KeepAll(),
                   tmp_format=torch.Tensor, external_sparsifier=KeepAll(), out_format=DenseTensor):
        self.weights[name] = (inline_sparsifier, tmp_format, external_sparsifier, out_format)
        self.initial_weight_sparsifiers[name] = initial_sparsifier

    def set_weight_grad(self, name, inline_sparsifier=KeepAll(), tmp_format=torch.Tensor,
                        external_sparsifier=KeepAll(), out_format=DenseTensor):
        self.grad_weights[name] = (inline_sparsifier, tmp_format, external_sparsifier, out_format)

    def set_interm(self, *a, **k):
        raise NotImplementedError("intermediate-tensor sparsification is outside the nmg weight path")

    set_interm_grad = set_interm

    def _fill_remaining(self):
        for name in set(self.weights) - set(self.grad_weights):
            self.set_weight_grad(name)
        for name in set(self.grad_weights) - set(self.weights):
            self.set_weight(name)

    def sparsify_model_inplace(self, module):
        self._fill_remaining()
        with torch.no_grad():
            for name, (_, _, _, fmt) in self.weights.items():
                owner = module
                *path, leaf = name.split(".")
                for tok in path:
                    owner = getattr(owner, tok)
                original = getattr(owner, leaf)
                sp = self.initial_weight_sparsifiers[name]
                impl = get_sparsifier_implementation(sp.__class__, torch.Tensor, fmt)
                wrapped = impl(sp, original, tuple(self.grad_weights[name]))
                setattr(owner, leaf, SparseParameterWrapper(wrapped))
        return module

    def sparsify_model_and_optimizer_inplace(self, module, optimizer):
        before = [id(p) for p in module.parameters()]
        where = {id(p): (gi, pi) for gi, grp in enumerate(optimizer.param_groups)
                 for pi, p in enumerate(grp["params"])}
        module = self.sparsify_model_inplace(module)
        for p, old in zip(module.parameters(), before):
            if id(p) != old and old in where:
                gi, pi = where[old]
                optimizer.param_groups[gi]["params"][pi] = p
        return module, optimizer

    def get_sparse_model(self, module):
        return self.sparsify_model_inplace(copy.deepcopy(module))
