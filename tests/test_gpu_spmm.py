"""GPU parity of the nmg x dense matmul, its transposed form and the registered operators.
Oracle: the equation the reference asserts, C == to_dense(A) @ B (dace_gnm_mult.py:1123,1189-1199),
evaluated in fp64 from the oracle's own val/idx, plus the CPU restatement of the reference kernel.
Tolerances: rel-L2 <= 1e-3 for 16-bit inputs with fp32 accumulation, <= 1e-5 for fp32."""
import copy
import ctypes
import warnings

import numpy as np
import pytest
import torch

import sten_amd as sten
from sten_amd import native
from oracle import nmg_oracle as O
from helpers import oracle_sparsify, rel_l2, seeded, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-3, torch.bfloat16: 8e-3}


def make(W, n, m, g, sd):
    return sten.GroupedNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=1 - sd)


def dense_ref(W, n, m, g, sd):
    val, idx, lay = oracle_sparsify(W, n, m, sd, g, 1 - sd)
    return O.to_dense(val, idx, lay).astype(np.float64), (val, idx, lay)


@pytest.mark.parametrize("kernel", ["mfma"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g", [
    (768, 768, 256, 2, 4, 16),
    (200, 330, 77, 2, 4, 4),
    (130, 96, 5, 3, 6, 2),
    (64, 520, 129, 2, 8, 4),
    (40, 72, 300, 1, 8, 2),
])
@pytest.mark.parametrize("sd", [1, 0])
def test_spmm_both_directions(kernel, dtype, M, K, T, n, m, g, sd):
    print(f"case {kernel} {dtype} M={M} K={K} T={T} {n}:{m}:{g} sd={sd}", flush=True)
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, sd)
    w = make(W, n, m, g, sd)
    x = seeded((T, K), dtype, seed=1)
    y = sten.spmm(w, x.to(DEV), reduce_dim=1, kernel=kernel)            # X @ W^T
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T) <= TOL[dtype]
    gy = seeded((T, M), dtype, seed=2)
    gx = sten.spmm(w, gy.to(DEV), reduce_dim=0, kernel=kernel)          # G @ W
    assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[dtype]


def test_config1_against_reference_cpu_kernel():
    # benchmark config 1 through the reference orientation and the CPU restatement of its kernel
    torch.manual_seed(0)
    W = torch.randn(768, 768)
    X = torch.randn(768, 256)          # B [K, N]
    val, idx, lay = oracle_sparsify(W, 2, 4, 0, 16, 1)
    C_cpu = O.simd_spmm(val, idx, lay, X.numpy())
    w = make(W, 2, 4, 16, 0)
    C = sten.spmm(w, X.t().contiguous().to(DEV), reduce_dim=1).t()
    assert rel_l2(to_np(C), C_cpu) <= 1e-5
    w2 = make(W, 2, 4, 16, 1)          # n:m along the reduction dim (the benchmark's wording)
    Wd, _ = dense_ref(W, 2, 4, 16, 1)
    C2 = sten.spmm(w2, X.t().contiguous().to(DEV), reduce_dim=1).t()
    assert rel_l2(to_np(C2), Wd @ X.numpy().astype(np.float64)) <= 1e-5


@pytest.mark.parametrize("T", [1, 3, 4, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_skinny_kernel(T, dtype):
    W = seeded((515, 1024), dtype, seed=5, std=0.05)
    Wd, _ = dense_ref(W, 2, 4, 16, 1)
    w = make(W, 2, 4, 16, 1)
    x = seeded((T, 1024), dtype, seed=6)
    b = seeded((515,), dtype, seed=7)
    ref = to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)
    for kernel in ("skinny", "mfma", "auto"):
        y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel=kernel)
        assert rel_l2(to_np(y), ref) <= TOL[dtype], kernel


def test_spmm_argument_errors():
    w = make(seeded((64, 64), torch.float16, 1), 2, 4, 4, 1)
    with pytest.raises(sten.NmgError):
        sten.spmm(w, torch.zeros(4, 64, device=DEV), reduce_dim=1)           # dtype mismatch
    with pytest.raises(sten.NmgError):
        sten.spmm(w, torch.zeros(4, 60, device=DEV).half(), reduce_dim=1)    # wrong K
    with pytest.raises(sten.NmgError):
        sten.spmm(w, torch.zeros(64, 64, device=DEV).half(), reduce_dim=1, kernel="skinny")


def build_sparse_linear(lin, n, m, g, sd, compressed_grad=False):
    sb = sten.SparsityBuilder()
    sb.set_weight("weight", initial_sparsifier=sten.GroupedNMSparsifier(n, m, g, sparse_dim=sd, group_dim=1 - sd),
                  out_format=sten.GroupedNMTensor)
    if compressed_grad:
        sb.set_weight_grad("weight", tmp_format=sten.GroupedNMTensor, out_format=sten.GroupedNMTensor)
    return sb.get_sparse_model(lin)


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("sd", [1, 0])
@pytest.mark.parametrize("compressed_grad", [False, True])
def test_linear_module_forward_backward(bias, sd, compressed_grad):
    # builder flow of tests/test_nmg.py:12-30 on a local nn.Linear; values checked against dense autograd
    sten.set_dispatch_failure("raise")
    torch.manual_seed(0)
    lin = torch.nn.Linear(96, 200, bias=bias).to(DEV)
    sp = build_sparse_linear(lin, 2, 4, 4, sd, compressed_grad)
    assert isinstance(sp.weight, sten.SparseParameterWrapper)
    Wd = sp.weight.wrapped_tensor.to_dense().detach().clone().requires_grad_(True)
    bd = lin.bias.detach().clone().requires_grad_(True) if bias else None
    x = torch.randn(3, 7, 96, device=DEV, requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    y = sp(x)
    yr = torch.nn.functional.linear(xr, Wd, bd)
    assert y.shape == yr.shape
    assert rel_l2(to_np(y), to_np(yr)) <= 1e-5
    gy = torch.randn_like(y)
    y.backward(gy)
    yr.backward(gy)
    assert rel_l2(to_np(x.grad), to_np(xr.grad)) <= 1e-5
    mask = (Wd != 0).to(Wd.dtype)
    gw = sp.weight.grad
    assert isinstance(gw, sten.SparseTensorWrapper)
    if compressed_grad:
        assert isinstance(gw.wrapped_tensor, sten.GroupedNMTensor)
        # padded / zero-valued kept slots aside, the compressed gradient is the dense one at kept positions
        got = to_np(gw.wrapped_tensor.to_dense())
        keep = to_np(sp.weight.wrapped_tensor.clone_layout(torch.ones_like(Wd)).to_dense())
        assert rel_l2(got, to_np(Wd.grad) * keep) <= 1e-5
    else:
        assert isinstance(gw.wrapped_tensor, sten.DenseTensor)
        assert rel_l2(to_np(gw.wrapped_tensor.to_dense()), to_np(Wd.grad)) <= 1e-5
    if bias:
        assert rel_l2(to_np(sp.bias.grad), to_np(bd.grad)) <= 1e-5


def test_torch_mm_forward_backward():
    # registration pattern of tests/test_api.py:272-298 for torch.mm(sparse, dense)
    sten.set_dispatch_failure("raise")
    W = seeded((80, 48), torch.float32, 3)
    B = seeded((48, 33), torch.float32, 4).to(DEV).requires_grad_(True)
    sp = sten.get_sparsifier_implementation(sten.GroupedNMSparsifier, torch.Tensor, sten.GroupedNMTensor)(
        sten.GroupedNMSparsifier(2, 4, 4, sparse_dim=1, group_dim=0), W.to(DEV).requires_grad_(True))
    Wd = sp.wrapped_tensor.to_dense().detach().clone().requires_grad_(True)
    Br = B.detach().clone().requires_grad_(True)
    C = torch.mm(sp, B)
    Cr = torch.mm(Wd, Br)
    assert rel_l2(to_np(C), to_np(Cr)) <= 1e-5
    g = torch.randn_like(C)
    C.backward(g)
    Cr.backward(g)
    assert rel_l2(to_np(B.grad), to_np(Br.grad)) <= 1e-5
    assert rel_l2(to_np(sp.grad.wrapped_tensor.to_dense()), to_np(Wd.grad)) <= 1e-5


def test_optimizer_steps_keep_pattern():
    # optimizer flow of tests/test_api.py:421-450, :512-551 with the nmg format
    torch.manual_seed(1)
    lin = torch.nn.Linear(64, 48).to(DEV)
    sb = sten.SparsityBuilder()
    sb.set_weight("weight", initial_sparsifier=sten.GroupedNMSparsifier(2, 4, 4, sparse_dim=1, group_dim=0),
                  out_format=sten.GroupedNMTensor)
    opt = torch.optim.SGD(lin.parameters(), lr=0.1, momentum=0.9)
    lin, opt = sb.sparsify_model_and_optimizer_inplace(lin, opt)
    idx0 = lin.weight.wrapped_tensor.idx.clone()
    w0 = lin.weight.wrapped_tensor.to_dense().clone()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for _ in range(3):
            loss = lin(torch.randn(5, 64, device=DEV)).abs().sum()
            loss.backward()
            opt.step()
            opt.zero_grad()
    w1 = lin.weight.wrapped_tensor.to_dense()
    assert isinstance(lin.weight.wrapped_tensor, sten.GroupedNMTensor)
    assert torch.equal(lin.weight.wrapped_tensor.idx, idx0)
    assert not torch.allclose(w0, w1)
    assert bool(((w1 != 0) <= (w0 != 0)).all())        # nothing outside the pattern became non-zero
    assert lin.weight.requires_grad


def test_in_place_updates_with_an_independently_sparsified_tensor():
    # Two tensors of the same layout, compressed independently, keep different columns in the same
    # slots: add_ / mul_ / copy_ must combine them position by position (through the dense form and
    # this tensor's pattern), not slot by slot; tensors that share the pattern take the direct path.
    a = make(seeded((96, 64), torch.float32, seed=1), 2, 4, 4, 1)
    b = make(seeded((96, 64), torch.float32, seed=2), 2, 4, 4, 1)
    assert a.layout == b.layout and not torch.equal(a.idx, b.idx)
    da, db = a.to_dense().clone(), b.to_dense().clone()
    mask = a.clone_layout(torch.ones(96, 64, device=DEV)).to_dense() != 0
    a.add_(b, alpha=0.5)
    assert torch.equal(a.to_dense(), torch.where(mask, da + 0.5 * db, torch.zeros_like(da)))
    a.mul_(b)
    want = torch.where(mask, (da + 0.5 * db) * db, torch.zeros_like(da))
    assert torch.equal(a.to_dense(), want)
    a.copy_(b)
    assert torch.equal(a.to_dense(), torch.where(mask, db, torch.zeros_like(db)))
    # same pattern (clone_layout shares idx; an equal copy of idx counts too): slot by slot
    c = a.clone_layout(torch.full((96, 64), 2.0, device=DEV))
    d = sten.GroupedNMTensor(c.val.clone(), a.idx.clone(), a.layout)
    before = a.val.clone()
    a.add_(c)
    a.add_(d)
    assert torch.equal(a.val, (before + 2.0) + 2.0)


def test_pattern_comparison_is_not_remembered_by_address():
    # The comparison of two idx tensors is remembered per tensor object.  A tensor with an equal
    # pattern is freed, and a tensor with another pattern, created right after it, gets its idx at
    # the freed address (same size, caching allocator) with version 0 like every kernel output: the
    # remembered "equal" must not be served for it.
    a = make(seeded((96, 64), torch.float32, seed=1), 2, 4, 4, 1)
    da = a.to_dense().clone()
    mask = a.clone_layout(torch.ones(96, 64, device=DEV)).to_dense() != 0
    twin = sten.GroupedNMTensor(a.val.clone(), a.idx.clone(), a.layout)
    old_ptr = twin.idx.data_ptr()
    a.add_(twin)                                   # equal pattern: slot by slot, and remembered
    assert torch.equal(a.to_dense(), da + da)
    del twin
    b = make(seeded((96, 64), torch.float32, seed=2), 2, 4, 4, 1)
    hit = b.idx.data_ptr() == old_ptr
    other = b if hit else sten.GroupedNMTensor(b.val, b.idx.clone(), b.layout)
    assert not torch.equal(other.idx, a.idx)
    db = other.to_dense().clone()
    a.add_(other)
    assert torch.equal(a.to_dense(), torch.where(mask, da + da + db, torch.zeros_like(da))), \
        f"idx of the second tensor at the freed address: {hit}"


def test_derived_operands_follow_in_place_changes_of_the_pattern():
    # the matmul operands are keyed on the versions of val and idx: a pattern written in place
    # (idx.copy_) must not leave the operands of the old pattern behind
    a = make(seeded((128, 64), torch.float16, seed=3), 2, 4, 16, 1)
    b = make(seeded((128, 64), torch.float16, seed=4), 2, 4, 16, 1)
    x = seeded((32, 64), torch.float16, seed=5).to(DEV)
    y0 = sten.spmm(a, x, reduce_dim=1)
    a.idx.copy_(b.idx)
    a.val.copy_(b.val)
    assert torch.equal(sten.spmm(a, x, reduce_dim=1), sten.spmm(b, x, reduce_dim=1))
    assert not torch.equal(y0, sten.spmm(a, x, reduce_dim=1))


def test_unregistered_op_raises_in_raise_mode():
    sten.set_dispatch_failure("raise")
    w = sten.SparseTensorWrapper.wrapped_from_dense(
        make(seeded((16, 16), torch.float32, 1), 2, 4, 1, 1), torch.zeros(1))
    with pytest.raises(sten.DispatchError):
        torch.relu(w)


@pytest.mark.parametrize("variant", [-1, 0, 6, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g", [
    (768, 768, 256, 2, 4, 16),
    (512, 64, 128, 2, 4, 16),    # a single K step
    (256, 320, 100, 2, 4, 16),   # K steps not a multiple of the pipeline depth
    (520, 1024, 300, 2, 4, 16),  # several workgroup tiles, ragged lines / tokens, K % 64 == 0
    (200, 328, 77, 2, 4, 4),     # ragged lines / tokens, K not a multiple of 64
    (96, 64, 33, 1, 4, 8),
    (130, 520, 300, 2, 8, 4),
    (64, 128, 40, 1, 8, 2),
    (40, 16, 17, 1, 2, 3),
])
def test_spmm_sparse_matrix_cores(variant, dtype, M, K, T, n, m, g):
    print(f"case smfmac v{variant} {dtype} M={M} K={K} T={T} {n}:{m}:{g}", flush=True)
    W = seeded((M, K), dtype, seed=M + K + n, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    w.spmm_opt["variant"] = variant
    x = seeded((T, K), dtype, seed=1)
    b = seeded((M,), dtype, seed=2)
    y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="smfmac")
    ref = to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)
    assert rel_l2(to_np(y), ref) <= TOL[dtype]
    y2 = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="mfma")
    assert rel_l2(to_np(y), to_np(y2)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g,slices", [
    (512, 1152, 40, 2, 4, 16, None),     # planned: 2 tiles, 18 K steps -> 2 slices
    (512, 1152, 129, 2, 4, 16, 3),       # two token tiles, uneven slices (6 + 6 + 6)
    (1000, 2048, 200, 2, 4, 8, 7),       # ragged lines and tokens, slices of 5, 5, ..., 2
    (300, 704, 17, 1, 4, 4, 11),         # one K step per slice
    (2048, 4096, 64, 2, 8, 32, None),    # 2:8 in 2-of-4 slots, planned
])
def test_split_reduction_matches_dense(dtype, M, K, T, n, m, g, slices):
    print(f"case split-K {dtype} M={M} K={K} T={T} {n}:{m}:{g} slices={slices}", flush=True)
    W = seeded((M, K), dtype, seed=M + K + T, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    if slices is not None:
        w.spmm_opt["slices"] = slices
    else:
        planned, ws = ctypes.c_int(0), ctypes.c_int64(0)
        assert native.load().nmg_splitk_plan(M, K, T, ctypes.byref(planned), ctypes.byref(ws)) == 0
        assert planned.value > 1 and ws.value == planned.value * T * ((M + 255) // 256) * 256 * 4
    x = seeded((T, K), dtype, seed=1)
    b = seeded((M,), dtype, seed=2)
    for bias in (None, b.to(DEV)):
        y = sten.spmm(w, x.to(DEV), bias, reduce_dim=1)
        ref = to_np(x).astype(np.float64) @ Wd.T + (0 if bias is None else to_np(b).astype(np.float64))
        assert rel_l2(to_np(y), ref) <= TOL[dtype]
    w.spmm_opt["slices"] = 1                      # the same product on whole reductions
    y1 = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(y1)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g,rd,slices", [
    (1024, 2048, 100, 4, 8, 4, 1, None),     # 4:8 forward on the dense matrix cores, planned slices
    (2048, 1024, 100, 2, 4, 16, 0, None),    # grad_input: reduction along the group dim, planned
    (2048, 1000, 300, 2, 4, 16, 0, 5),       # ragged outputs, three token tiles, slices of 7, 7, 7, 7, 4
    (640, 320, 33, 2, 8, 4, 0, 10),          # one K step per slice
])
def test_split_reduction_dense_route(dtype, M, K, T, n, m, g, rd, slices):
    print(f"case split-K dense {dtype} M={M} K={K} T={T} {n}:{m}:{g} reduce_dim={rd} slices={slices}", flush=True)
    W = seeded((M, K), dtype, seed=M + K + T, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    R, Oo = (K, M) if rd == 1 else (M, K)       # reduction extent, outputs
    if slices is not None:
        w.spmm_opt["slices"] = slices
    else:
        planned, ws = ctypes.c_int(0), ctypes.c_int64(0)
        assert native.load().nmg_splitk_plan(Oo, R, T, ctypes.byref(planned), ctypes.byref(ws)) == 0
        assert planned.value > 1
    x = seeded((T, R), dtype, seed=1)
    y = sten.spmm(w, x.to(DEV), reduce_dim=rd, kernel="densefrag")
    ref = to_np(x).astype(np.float64) @ (Wd.T if rd == 1 else Wd)
    assert rel_l2(to_np(y), ref) <= TOL[dtype]
    w.spmm_opt["slices"] = 1
    y1 = sten.spmm(w, x.to(DEV), reduce_dim=rd, kernel="densefrag")
    assert rel_l2(to_np(y), to_np(y1)) <= 2 * TOL[dtype]


def test_split_reduction_on_the_target_weight_at_intermediate_batches():
    torch.manual_seed(0)
    W = (torch.randn(4096, 11008) * 0.02).half()
    w = make(W, 2, 4, 16, 1)
    Wd = w.to_dense().double()
    for T in (17, 128, 500):
        x = torch.randn(T, 11008, dtype=torch.float16, device=DEV)
        y = sten.spmm(w, x, reduce_dim=1)
        assert rel_l2(to_np(y), to_np(x.double() @ Wd.t())) <= TOL[torch.float16]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,n,m,g", [
    (4096, 1024, 2, 4, 16),     # 128 blocks of 32 lines: two workgroups per block
    (300, 640, 1, 4, 4),        # ragged lines, few blocks
    (11008, 512, 2, 4, 16),     # 344 blocks: one workgroup per block
])
def test_streaming_kernel_with_17_to_32_tokens(dtype, M, K, n, m, g):
    # the decode kernel with the second half of its 32 token columns in use; every count from 17 to
    # 32 (4 token rows per DMA load: 5 .. 8 loads per chunk), with a bias, against the fp64 product
    print(f"case wide decode {dtype} M={M} K={K} {n}:{m}:{g}", flush=True)
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    b = seeded((M,), dtype, seed=5)
    for T in range(17, 33):
        x = seeded((T, K), dtype, seed=T)
        ref = to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)
        w.spmm_opt["variant"] = 5
        y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
        assert y.shape == (T, M)
        assert rel_l2(to_np(y), ref) <= TOL[dtype], T
        w.spmm_opt.pop("variant")
        y2 = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)      # automatic choice (<= 24: the same kernel)
        assert rel_l2(to_np(y2), ref) <= TOL[dtype], T
        if T <= 24:
            assert torch.equal(y, y2), T


def test_target_weight_against_the_oracle_at_decode_and_large_batches():
    # the north-star weight 4096 x 11008 2:4:16 compressed by the CPU oracle (val / idx compared
    # bit for bit), then the product at 1 and 16 tokens (decode kernel) and 2048 tokens (direct
    # kernel of the sparse matrix cores) against the fp64 product with the oracle's dense form
    print("case target weight 4096x11008 vs oracle, T = 1, 16, 2048", flush=True)
    W = seeded((4096, 11008), torch.float16, seed=11, std=0.02)
    Wd, (val, idx, lay) = dense_ref(W, 2, 4, 16, 1)
    w = make(W, 2, 4, 16, 1)
    assert np.array_equal(to_np(w.idx), idx)
    assert np.array_equal(to_np(w.val).view(np.uint16), val.view(np.uint16))
    for T in (1, 16, 2048):
        x = seeded((T, 11008), torch.float16, seed=12 + T)
        y = sten.spmm(w, x.to(DEV), reduce_dim=1)
        assert y.shape == (T, 4096)
        assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T) <= TOL[torch.float16], f"T={T}"


@pytest.mark.parametrize("T", [3, 16, 300])
def test_one_of_eight_with_group_32_against_the_oracle(T):
    # benchmark config 3's sparsest pattern (1:8, group 32: chunks of 256 lines) at a size the
    # oracle compresses in seconds: decode kernel, split reduction and direct kernel
    print(f"case 1:8:32 T={T}", flush=True)
    W = seeded((1024, 1536), torch.float16, seed=21, std=0.05)
    Wd, (val, idx, lay) = dense_ref(W, 1, 8, 32, 1)
    w = make(W, 1, 8, 32, 1)
    assert np.array_equal(to_np(w.idx), idx)
    assert np.array_equal(to_np(w.val).view(np.uint16), val.view(np.uint16))
    x = seeded((T, 1536), torch.float16, seed=22)
    y = sten.spmm(w, x.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T) <= TOL[torch.float16]
    gy = seeded((T, 1024), torch.float16, seed=23)
    gx = sten.spmm(w, gy.to(DEV), reduce_dim=0)
    assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[torch.float16]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("R,C,N,n,m,g", [
    (256, 256, 128, 2, 4, 16),      # one tile
    (300, 192, 100, 2, 4, 4),       # ragged rows and columns (N % 8 != 0 goes through a padded pitch)
    (520, 448, 264, 1, 8, 2),       # several tiles both ways
    (1024, 1024, 1000, 2, 8, 4),
    (768, 3072, 4096, 2, 4, 16),    # the shape of the reference's own matmul test (dace_gnm_mult.py:1183)
])
def test_product_with_both_dense_operands_transposed(dtype, R, C, N, n, m, g):
    # torch.mm(W, B): C[R, N] = W @ B with B [C, N] as it lies in memory (no transposing copies),
    # against the fp64 product with the oracle's dense form, and against the copying route
    print(f"case spmm_tt {dtype} R={R} C={C} N={N} {n}:{m}:{g}", flush=True)
    W = seeded((R, C), dtype, seed=R + C, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    b = seeded((C, N), dtype, seed=9)
    ref = Wd @ to_np(b).astype(np.float64)
    pitch = -(-N // 8) * 8
    bb = torch.zeros(C, pitch, dtype=dtype, device=DEV)[:, :N]
    bb.copy_(b)
    c = sten.spmm_tt(w, bb)
    assert c.shape == (R, N) and c.is_contiguous()
    assert rel_l2(to_np(c), ref) <= TOL[dtype]
    c2 = sten.spmm(w, b.to(DEV).t().contiguous(), reduce_dim=1).t()
    assert rel_l2(to_np(c), to_np(c2)) <= 2 * TOL[dtype]
    # the C ABI with a bias per row and a padded output pitch
    lib = native.load()
    fp_val, fp_idx = w.fragpack()
    bias = seeded((R,), dtype, seed=10).to(DEV)
    out = torch.full((R, pitch + 8), 7.0, dtype=dtype, device=DEV)
    native.check(lib.nmg_spmm_smfmac_tt(native.ptr(fp_val), native.ptr(fp_idx), R, C, native.ptr(bb), pitch,
                                        native.ptr(out), pitch + 8, native.ptr(bias), N, native.dtype_code(dtype),
                                        None))
    torch.cuda.synchronize()
    assert rel_l2(to_np(out[:, :N]), ref + to_np(bias).astype(np.float64)[:, None]) <= TOL[dtype]
    assert bool((out[:, N:] == 7.0).all()), "columns beyond N must stay untouched"


def test_reference_matmul_test_shape_takes_the_dense_matrix_cores():
    # M, K, N = 768, 3072, 4096 with 3:6:12 ("BERT sizes", dace_gnm_mult.py:1013-1015, :1183): the
    # automatic choice must be the dense-matrix-core route, not the untuned fallback
    print("case reference shape 768x3072x4096 3:6:12", flush=True)
    W = seeded((768, 3072), torch.float16, seed=3, std=0.05)
    Wd, _ = dense_ref(W, 3, 6, 12, 1)
    w = make(W, 3, 6, 12, 1)
    x = seeded((4096, 3072), torch.float16, seed=4)
    y = sten.spmm(w, x.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T) <= TOL[torch.float16]
    assert getattr(w, "_densefrag", None) and 1 in w._densefrag, "the dense-core operand was not built"
    gx = sten.spmm(w, seeded((4096, 768), torch.float16, seed=5).to(DEV), reduce_dim=0)
    assert rel_l2(to_np(gx), to_np(seeded((4096, 768), torch.float16, seed=5)).astype(np.float64) @ Wd) <= TOL[torch.float16]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g,sd", [
    (300, 1001, 130, 2, 4, 16, 1),     # reduction not a multiple of 8: no sparse-core operand
    (257, 520, 77, 4, 8, 4, 1),        # 4:8 with a reduction that is not a multiple of 64
    (192, 455, 40, 2, 5, 3, 1),        # m = 5: no dense-core operand either
    (130, 333, 64, 3, 7, 2, 0),        # the other orientation
])
def test_odd_16_bit_shapes_take_the_padded_dense_route(dtype, M, K, T, n, m, g, sd):
    print(f"case padded expand {dtype} M={M} K={K} T={T} {n}:{m}:{g} sd={sd}", flush=True)
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, sd)
    w = make(W, n, m, g, sd)
    x = seeded((T, K), dtype, seed=1)
    b = seeded((M,), dtype, seed=2)
    y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)) <= TOL[dtype]
    assert any(isinstance(k, tuple) for k in getattr(w, "_dense_operand", {})), "the padded operand was not built"
    gy = seeded((T, M), dtype, seed=3)
    gx = sten.spmm(w, gy.to(DEV), reduce_dim=0)
    assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[dtype]
    # a single token along the group dim takes the padded route too (the streaming kernel has no form for it)
    one = (gy if sd == 1 else x)[:1]
    g1 = sten.spmm(w, one.to(DEV), reduce_dim=1 - sd)
    ref1 = to_np(one).astype(np.float64) @ (Wd if sd == 1 else Wd.T)
    assert rel_l2(to_np(g1), ref1) <= TOL[dtype]
    # a view of the activations with an odd pitch goes through a padded copy as well
    xv = seeded((T, K + 3), dtype, seed=4).to(DEV)[:, 1:K + 1]
    yv = sten.spmm(w, xv, reduce_dim=1)
    assert rel_l2(to_np(yv), to_np(xv).astype(np.float64) @ Wd.T) <= TOL[dtype]
    # the kernel that expands inside its loop stays reachable and agrees
    w.spmm_opt["expand"] = False
    y2 = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y2), to_np(y).astype(np.float64)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("T", [1, 3, 16])
@pytest.mark.parametrize("dtype,M,K,n,m,g,sd", [
    (torch.float16, 512, 1088, 4, 8, 4, 1),       # no sparse-core operand for 4:8 (and no whole sets of 32 blocks for the streaming kernel)
    (torch.bfloat16, 760, 640, 3, 4, 16, 0),      # the reference's default orientation (reduction along the group dim) at 3:4, which the streaming kernel does not take
    (torch.float16, 320, 1152, 3, 6, 12, 1),
    (torch.float32, 512, 1024, 2, 4, 16, 1),      # fp32: dense copy + fp32 GEMM
])
def test_few_tokens_without_a_sparse_core_operand_take_the_dense_routes(dtype, M, K, n, m, g, sd, T):
    print(f"case few tokens {dtype} M={M} K={K} {n}:{m}:{g} sd={sd} T={T}", flush=True)
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, sd)
    w = make(W, n, m, g, sd)
    x = seeded((T, K), dtype, seed=T)
    b = seeded((M,), dtype, seed=2)
    y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)) <= TOL[dtype]
    if dtype == torch.float32:
        assert 1 in getattr(w, "_dense_operand", {}), "the dense copy was not built"
    else:
        assert getattr(w, "_densefrag", None) and 1 in w._densefrag, "the dense-core operand was not built"
    # the streaming kernel stays reachable and agrees
    alt = "skinny" if dtype != torch.float32 and sd == 1 else "mfma"
    y2 = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel=alt)
    assert rel_l2(to_np(y2), to_np(y).astype(np.float64)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("T", [1, 3, 16])
@pytest.mark.parametrize("dtype,M,K,n,m,g", [
    (torch.float16, 768, 640, 2, 4, 16),       # three spans of 256 outputs, 640 lines
    (torch.bfloat16, 768, 640, 2, 4, 16),
    (torch.float16, 272, 328, 1, 4, 8),        # 68 blocks: part of a span; 41 groups of 8 lines
    (torch.bfloat16, 760, 640, 2, 4, 16),      # 190 blocks: the last lane of a span holds two blocks of its four
    (torch.float16, 512, 1000, 2, 8, 4),
    (torch.bfloat16, 1040, 2056, 1, 8, 32),    # 130 blocks of 8, ragged chunks of the group dim
    (torch.float16, 4096, 2816, 2, 4, 16),     # sixteen spans, several slices of the reduction
    (torch.bfloat16, 8192, 9000, 2, 4, 16),    # 32 spans: slices of 1152 lines, up to five tiles of 32 lines per wavefront
])
def test_few_tokens_along_the_group_dim_stream_the_compressed_lines(dtype, M, K, n, m, g, T):
    # F.linear with a weight in the reference's default orientation (n:m blocks along the outputs):
    # the reduction runs along the group dim; <= 16 tokens stream the rowpack operand
    print(f"case gstream {dtype} M={M} K={K} {n}:{m}:{g} T={T}", flush=True)
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 0)
    w = make(W, n, m, g, 0)
    x = seeded((T, K), dtype, seed=T)
    b = seeded((M,), dtype, seed=2)
    ref = to_np(x).astype(np.float64) @ Wd.T
    y = sten.spmm(w, x.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), ref) <= TOL[dtype]
    assert not getattr(w, "_densefrag", None), "the dense-core operand was built"
    yb = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="gstream")
    assert rel_l2(to_np(yb), ref + to_np(b).astype(np.float64)) <= TOL[dtype]
    # a view with a row pitch (every second row of a larger buffer) and repeated calls agree bit for bit
    xs = torch.zeros((2 * T, K + 8), dtype=dtype, device=DEV)[::2, :K]
    xs.copy_(x.to(DEV))
    for _ in range(3):
        assert torch.equal(sten.spmm(w, xs, reduce_dim=1), y)


@pytest.mark.parametrize("T", [1, 5, 16])
@pytest.mark.parametrize("dtype,M,K,n,m,g", [
    (torch.float16, 512, 1024, 2, 8, 32),      # sixteen workgroups, four sets: some wavefronts have none
    (torch.bfloat16, 512, 1024, 2, 8, 32),
    (torch.float16, 200, 2560, 1, 8, 4),       # lines that are not a multiple of 32, ten sets over eight wavefronts
    (torch.float16, 264, 768, 4, 8, 2),        # 4:8: no operand of the sparse matrix cores exists
    (torch.bfloat16, 96, 6144, 4, 8, 1),       # 24 sets: three per wavefront, one round at 4:8
    (torch.float16, 1056, 8192, 2, 8, 8),      # 32 sets: four per wavefront, one round
    (torch.float16, 160, 16384, 2, 8, 4),      # 64 sets: two rounds of four per wavefront
    (torch.bfloat16, 64, 11008 + 256, 4, 8, 2),    # 44 sets: six per wavefront (two rounds), the last wavefront with two
    (torch.float16, 40, 9216 + 256, 1, 8, 16),     # 37 sets: five per wavefront (a second round of one set), the last wavefront with two
])
def test_few_tokens_on_blocks_of_eight_stream_the_compressed_lines(dtype, M, K, n, m, g, T):
    # 1:8, 2:8, 4:8 with the blocks along the reduction and <= 16 tokens: the rowpack operand, streamed
    print(f"case sstream {dtype} M={M} K={K} {n}:{m}:{g} T={T}", flush=True)
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    x = seeded((T, K), dtype, seed=T)
    b = seeded((M,), dtype, seed=2)
    ref = to_np(x).astype(np.float64) @ Wd.T
    y = sten.spmm(w, x.to(DEV), reduce_dim=1, kernel="sstream")
    assert rel_l2(to_np(y), ref) <= TOL[dtype]
    yb = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="sstream")
    assert rel_l2(to_np(yb), ref + to_np(b).astype(np.float64)) <= TOL[dtype]
    # the automatic choice: this route for 4:8, from 3072 lines on and up to 8 tokens, else the sparse matrix cores
    ya = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(ya), ref + to_np(b).astype(np.float64)) <= TOL[dtype]
    xs = torch.zeros((2 * T, K + 8), dtype=dtype, device=DEV)[::2, :K]
    xs.copy_(x.to(DEV))
    for _ in range(3):
        assert torch.equal(sten.spmm(w, xs, reduce_dim=1, kernel="sstream"), y)
    if n < 4:
        y2 = sten.spmm(w, x.to(DEV), reduce_dim=1, kernel="skinny")      # the operand of the sparse matrix cores
        assert rel_l2(to_np(y2), to_np(y).astype(np.float64)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("T", [1, 2, 3, 4])
@pytest.mark.parametrize("dtype,M,K", [
    (torch.float16, 768, 640),        # 48 spans of 16 outputs, three sets of 256 lines: most wavefronts have none
    (torch.bfloat16, 760, 4136),      # 190 blocks: the last span holds two blocks; 17 sets, the last with 40 lines
    (torch.float16, 40, 8),           # one group of 8 lines
    (torch.float16, 4096, 2816),      # 256 workgroups, 11 sets
])
def test_a_handful_of_tokens_along_the_group_dim_with_16_outputs_per_workgroup(dtype, M, K, T):
    # 2:4 in the reference's default orientation: every workgroup owns 16 outputs over the whole
    # reduction, one kernel without matrix instructions; the automatic choice up to 2 tokens
    print(f"case ostream {dtype} M={M} K={K} T={T}", flush=True)
    n, m, g = 2, 4, 16
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 0)
    w = make(W, n, m, g, 0)
    x = seeded((T, K), dtype, seed=T)
    b = seeded((M,), dtype, seed=2)
    ref = to_np(x).astype(np.float64) @ Wd.T
    y = sten.spmm(w, x.to(DEV), reduce_dim=1, kernel="ostream")
    assert rel_l2(to_np(y), ref) <= TOL[dtype]
    yb = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="ostream")
    assert rel_l2(to_np(yb), ref + to_np(b).astype(np.float64)) <= TOL[dtype]
    ya = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)      # the automatic choice: this kernel or the sliced one
    assert rel_l2(to_np(ya), ref + to_np(b).astype(np.float64)) <= TOL[dtype]
    if K % 8 == 0 and T > 1:
        xs = torch.zeros((2 * T, K + 8), dtype=dtype, device=DEV)[::2, :K]
        xs.copy_(x.to(DEV))
        for _ in range(3):
            assert torch.equal(sten.spmm(w, xs, reduce_dim=1, kernel="ostream"), y)
    y2 = sten.spmm(w, x.to(DEV), reduce_dim=1, kernel="gstream")      # the sliced kernel agrees
    assert rel_l2(to_np(y2), to_np(y).astype(np.float64)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("T", [1, 16])
def test_streamed_product_on_blocks_of_eight_at_full_size(T):
    # 8192 x 8192 at 2:8:32 against the dense form, in fp64 on the host
    print(f"case sstream full size T={T}", flush=True)
    W = seeded((8192, 8192), torch.float16, seed=6, std=0.02).to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 8, sparse_dim=1, group_size=32, group_dim=0)
    x = seeded((T, 8192), torch.float16, seed=T)
    y = sten.spmm(w, x.to(DEV), reduce_dim=1)
    ref = to_np(x).astype(np.float64) @ to_np(w.to_dense()).astype(np.float64).T
    assert rel_l2(to_np(y), ref) <= TOL[torch.float16]


@pytest.mark.parametrize("T", [1, 16])
def test_streamed_product_along_the_group_dim_at_full_size(T):
    # 4096 x 11008 at 2:4:16 in the reference's default orientation against the dense form (which the
    # sparsifier tests hold bit-exact against the oracle), in fp64 on the host
    print(f"case gstream full size T={T}", flush=True)
    W = seeded((4096, 11008), torch.float16, seed=5, std=0.02).to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=0, group_size=16, group_dim=1)
    x = seeded((T, 11008), torch.float16, seed=T)
    y = sten.spmm(w, x.to(DEV), reduce_dim=1)
    ref = to_np(x).astype(np.float64) @ to_np(w.to_dense()).astype(np.float64).T
    assert rel_l2(to_np(y), ref) <= TOL[torch.float16]


def test_reference_matmul_test_shape_in_single_precision():
    # the same sizes in the dtype of the reference's own test (fp32, dace_gnm_mult.py:1183): expand
    # once, then the fp32 matrix cores; B [K, N] and C [M, N] as torch.mm has them
    print("case reference shape 768x3072x4096 3:6:12 fp32", flush=True)
    W = seeded((768, 3072), torch.float32, seed=3, std=0.05)
    Wd, _ = dense_ref(W, 3, 6, 12, 1)
    w = make(W, 3, 6, 12, 1)
    x = seeded((4096, 3072), torch.float32, seed=4)
    y = sten.spmm(w, x.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T) <= TOL[torch.float32]
    assert 1 in getattr(w, "_dense_operand", {}), "the expanded operand was not kept"
    B = seeded((3072, 4096), torch.float32, seed=5)
    c = sten.spmm_tt(w, B.to(DEV))
    assert c.is_contiguous() and rel_l2(to_np(c), Wd @ to_np(B).astype(np.float64)) <= TOL[torch.float32]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("R,C,N,n,m,g,rd", [
    (256, 256, 128, 2, 4, 16, 0),      # one tile; W^T @ B: the gradient with respect to B of torch.mm(W, B)
    (320, 200, 100, 2, 4, 4, 0),       # ragged outputs and columns (N % 8 != 0 goes through a padded pitch)
    (576, 520, 264, 4, 8, 2, 0),       # several tiles both ways, a pattern the sparse cores do not take
    (1024, 1024, 1000, 1, 8, 4, 0),
    (4096, 1024, 2048, 2, 4, 16, 0),   # 64 K steps, full token tiles
    (264, 448, 136, 4, 8, 4, 1),       # W @ B on the dense matrix cores
])
def test_dense_core_product_with_both_dense_operands_transposed(dtype, R, C, N, n, m, g, rd):
    print(f"case spmm_tt_dense {dtype} R={R} C={C} N={N} {n}:{m}:{g} reduce_dim={rd}", flush=True)
    W = seeded((R, C), dtype, seed=R + C, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    K, O = (R, C) if rd == 0 else (C, R)
    b = seeded((K, N), dtype, seed=9)
    ref = (Wd.T if rd == 0 else Wd) @ to_np(b).astype(np.float64)
    pitch = -(-N // 8) * 8
    bb = torch.zeros(K, pitch, dtype=dtype, device=DEV)[:, :N]
    bb.copy_(b)
    c = sten.spmm_tt_dense(w, bb, reduce_dim=rd)
    assert c.shape == (O, N) and c.is_contiguous()
    assert rel_l2(to_np(c), ref) <= TOL[dtype]
    c2 = sten.spmm(w, b.to(DEV).t().contiguous(), reduce_dim=rd).t()
    assert rel_l2(to_np(c), to_np(c2)) <= 2 * TOL[dtype]
    # the C ABI with a bias per row and a padded output pitch
    lib = native.load()
    df = w.densefrag(rd)
    bias = seeded((O,), dtype, seed=10).to(DEV)
    out = torch.full((O, pitch + 8), 7.0, dtype=dtype, device=DEV)
    native.check(lib.nmg_spmm_densefrag_tt(native.ptr(df), O, K, native.ptr(bb), pitch, native.ptr(out), pitch + 8,
                                           native.ptr(bias), N, native.dtype_code(dtype), None))
    torch.cuda.synchronize()
    assert rel_l2(to_np(out[:, :N]), ref + to_np(bias).astype(np.float64)[:, None]) <= TOL[dtype]
    assert bool((out[:, N:] == 7.0).all()), "columns beyond N must stay untouched"
    assert lib.nmg_spmm_densefrag_tt(native.ptr(df), O, K, native.ptr(bb), pitch + 4, native.ptr(out), pitch + 8,
                                     None, N, native.dtype_code(dtype), None) == 2      # ldb % 8


def test_transposed_product_argument_errors():
    lib = native.load()
    w = make(seeded((64, 128), torch.float16, 1), 2, 4, 4, 1)
    fp_val, fp_idx = w.fragpack()
    b = torch.zeros(128, 40, dtype=torch.float16, device=DEV)
    c = torch.zeros(64, 40, dtype=torch.float16, device=DEV)
    args = lambda K, ldb, dt: (native.ptr(fp_val), native.ptr(fp_idx), 64, K, native.ptr(b), ldb, native.ptr(c), 40,
                               None, 40, dt, None)
    assert lib.nmg_spmm_smfmac_tt(*args(128, 40, native.NMG_F16)) == 0
    assert lib.nmg_spmm_smfmac_tt(*args(100, 40, native.NMG_F16)) == 2      # K % 64
    assert lib.nmg_spmm_smfmac_tt(*args(128, 36, native.NMG_F16)) == 1      # ldb < T
    assert lib.nmg_spmm_smfmac_tt(*args(128, 44, native.NMG_F16)) == 2      # ldb % 8
    assert lib.nmg_spmm_smfmac_tt(*args(128, 40, native.NMG_F32)) == 2
    torch.cuda.synchronize()
    # torch.mm through the dispatcher takes this route and matches the dense product
    sp = sten.SparseTensorWrapper.wrapped_from_dense(w, w.to_dense(), None)
    bm = torch.randn(128, 96, device=DEV).half()
    got = torch.mm(sp, bm)
    assert rel_l2(to_np(got), to_np(w.to_dense().double() @ bm.double())) <= TOL[torch.float16]


def test_sparse_matrix_cores_refuse_incompatible_patterns():
    w = make(seeded((64, 64), torch.float16, 1), 4, 8, 1, 1)     # 4:8 can keep 3 of an aligned 4
    with pytest.raises(sten.NmgError):
        sten.spmm(w, torch.zeros(32, 64, device=DEV).half(), reduce_dim=1, kernel="smfmac")
    w32 = make(seeded((64, 64), torch.float32, 1), 2, 4, 4, 1)
    with pytest.raises(sten.NmgError):
        sten.spmm(w32, torch.zeros(32, 64, device=DEV), reduce_dim=1, kernel="smfmac")


def test_full_size_config2_smfmac_vs_mfma_and_linearity():
    # benchmark config 2 at full size: the two independent kernels agree, and the op is linear in X
    torch.manual_seed(0)
    W = (torch.randn(4096, 4096) * 0.02).half()
    X = torch.randn(2048, 4096).half().to(DEV)
    w = make(W, 2, 4, 16, 1)
    y_s = sten.spmm(w, X, reduce_dim=1, kernel="smfmac").float()
    y_m = sten.spmm(w, X, reduce_dim=1, kernel="mfma").float()
    assert float((y_s - y_m).norm() / y_m.norm()) <= 1e-3
    ref = (X.float() @ w.to_dense().float().t())
    assert float((y_s - ref).norm() / ref.norm()) <= 1e-3
    y2 = sten.spmm(w, (2 * X), reduce_dim=1, kernel="smfmac").float()
    assert float((y2 - 2 * y_s).norm() / y2.norm()) <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g", [
    (512, 640, 300, 2, 4, 16),     # several workgroup tiles in both directions, ragged tokens
    (320, 256, 130, 4, 8, 2),      # pattern that does not fit 2-of-4 groups
    (264, 192, 77, 3, 4, 4),
    (520, 128, 40, 1, 8, 4),
    (256, 320, 129, 2, 8, 2),
    (192, 64, 33, 1, 2, 8),
])
def test_dense_pipeline_kernel_both_directions(dtype, M, K, T, n, m, g):
    # kernel="mfma" with 16-bit data and reduction extents that are multiples of 64 runs the
    # pipelined dense-MFMA kernel: forward (reduce along the sparse dim) and the transposed product
    # (reduce along the group dim), the latter being grad_input of F.linear
    print(f"case dense-pipe {dtype} M={M} K={K} T={T} {n}:{m}:{g}", flush=True)
    W = seeded((M, K), dtype, seed=M + K + n, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    x = seeded((T, K), dtype, seed=1)
    b = seeded((M,), dtype, seed=2)
    ref = to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)
    gy = seeded((T, M), dtype, seed=3)
    for expand in (False, True):     # weights expanded inside the kernel / into scratch first
        w.spmm_opt["expand"] = expand
        y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="mfma")
        assert rel_l2(to_np(y), ref) <= TOL[dtype], expand
        if M % 64 == 0:
            gx = sten.spmm(w, gy.to(DEV), reduce_dim=0, kernel="mfma")
            assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[dtype], expand
    # the reference orientation (n:m along dim 0): forward reduces along the group dim
    w0 = make(W, n, m, g, 0)
    Wd0, _ = dense_ref(W, n, m, g, 0)
    y0 = sten.spmm(w0, x.to(DEV), reduce_dim=1, kernel="expand")
    assert rel_l2(to_np(y0), to_np(x).astype(np.float64) @ Wd0.T) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("R,C,n,m,g", [
    (768, 768, 2, 4, 16),
    (200, 330, 2, 4, 4),     # ragged on both dims
    (130, 96, 3, 6, 2),      # m does not divide the tile width
    (64, 520, 2, 8, 4),
    (70, 130, 5, 12, 1),     # 792 patterns: two-byte pattern numbers
])
@pytest.mark.parametrize("sd", [1, 0])
def test_dense_operand_matches_oracle_bit_exactly(dtype, R, C, n, m, g, sd):
    print(f"case expand {dtype} {R}x{C} {n}:{m}:{g} sd={sd}", flush=True)
    W = seeded((R, C), dtype, seed=R + C + m, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, sd)
    w = make(W, n, m, g, sd)
    a1 = w.dense_operand(1)          # [dim0, dim1]
    a0 = w.dense_operand(0)          # transposed
    assert a1.shape == (R, C) and a0.shape == (C, R)
    assert np.array_equal(to_np(a1).astype(np.float64), Wd)
    assert np.array_equal(to_np(a0).astype(np.float64), Wd.T)
    assert torch.equal(a1, w.to_dense())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("O_,K,T", [(256, 64, 128), (300, 320, 77), (1024, 1024, 512)])
def test_dense_nt_gemm_entry_point(dtype, O_, K, T):
    from sten_amd import native
    print(f"case gemm_nt {dtype} O={O_} K={K} T={T}", flush=True)
    A = seeded((O_, K), dtype, seed=3, std=0.5).to(DEV)
    X = seeded((T, K), dtype, seed=4).to(DEV)
    b = seeded((O_,), dtype, seed=5).to(DEV)
    Y = torch.empty((T, O_), dtype=dtype, device=DEV)
    native.check(native.load().nmg_gemm_nt(A.data_ptr(), K, X.data_ptr(), K, Y.data_ptr(), O_, b.data_ptr(),
                                           O_, K, T, native.dtype_code(dtype), native.stream_ptr(X.device)))
    ref = to_np(X).astype(np.float64) @ to_np(A).astype(np.float64).T + to_np(b).astype(np.float64)
    assert rel_l2(to_np(Y), ref) <= TOL[dtype]


@pytest.mark.parametrize("O_,K,T,pad", [
    (256, 64, 128, 0),        # whole 128-wide tiles
    (300, 323, 77, 0),        # ragged everywhere, rows not 16-byte aligned (scalar loads)
    (130, 40, 50, 4),         # small tiles, padded pitches
    (1024, 1024, 512, 0),
    (64, 17, 200, 3),         # reduction shorter than two K steps, odd pitch
    (96, 3072, 4096, 0),      # one column of 128 x 96 tiles
    (768, 768, 64, 0),        # 32 x 32 tiles, reduction split inside the workgroup
    (768, 100, 64, 0),        # the same with a ragged last step
    (512, 48, 4096, 0),       # 128 x 64 tiles, three steps: prologue and tail only
])
def test_dense_nt_gemm_entry_point_single_precision(O_, K, T, pad):
    from sten_amd import native
    print(f"case gemm_nt f32 O={O_} K={K} T={T} pad={pad}", flush=True)
    dtype = torch.float32
    A = seeded((O_, K + pad), dtype, seed=3, std=0.5).to(DEV)
    X = seeded((T, K + pad), dtype, seed=4).to(DEV)
    b = seeded((O_,), dtype, seed=5).to(DEV)
    Y = torch.full((T, O_ + pad), 7.0, dtype=dtype, device=DEV)
    native.check(native.load().nmg_gemm_nt(A.data_ptr(), K + pad, X.data_ptr(), K + pad, Y.data_ptr(), O_ + pad,
                                           b.data_ptr(), O_, K, T, native.dtype_code(dtype),
                                           native.stream_ptr(X.device)))
    ref = (to_np(X)[:, :K].astype(np.float64) @ to_np(A)[:, :K].astype(np.float64).T
           + to_np(b).astype(np.float64))
    assert rel_l2(to_np(Y)[:, :O_], ref) <= TOL[dtype]
    if pad:
        assert torch.all(Y[:, O_:] == 7.0)      # nothing written past the row


@pytest.mark.parametrize("O_,K,T,pad", [
    (256, 64, 128, 0),        # whole 128-wide tiles
    (300, 323, 77, 0),        # ragged everywhere
    (130, 40, 50, 4),         # padded pitches
    (1024, 1024, 512, 0),
    (66, 17, 200, 3),         # outputs not a multiple of 4, odd pitch
    (96, 3072, 4096, 0),      # one column of 128 x 96 tiles
    (768, 768, 64, 0),        # 32 x 32 tiles, reduction split inside the workgroup
])
def test_dense_nn_gemm_entry_point_single_precision(O_, K, T, pad):
    from sten_amd import native
    print(f"case gemm_nn f32 O={O_} K={K} T={T} pad={pad}", flush=True)
    dtype = torch.float32
    A = seeded((K, O_ + pad), dtype, seed=3, std=0.5).to(DEV)        # reduction-major
    X = seeded((T, K + pad), dtype, seed=4).to(DEV)
    b = seeded((O_,), dtype, seed=5).to(DEV)
    Y = torch.full((T, O_ + pad), 7.0, dtype=dtype, device=DEV)
    native.check(native.load().nmg_gemm_nn(A.data_ptr(), O_ + pad, X.data_ptr(), K + pad, Y.data_ptr(), O_ + pad,
                                           b.data_ptr(), O_, K, T, native.dtype_code(dtype),
                                           native.stream_ptr(X.device)))
    ref = (to_np(X)[:, :K].astype(np.float64) @ to_np(A)[:, :O_].astype(np.float64)
           + to_np(b).astype(np.float64))
    assert rel_l2(to_np(Y)[:, :O_], ref) <= TOL[dtype]
    if pad:
        assert torch.all(Y[:, O_:] == 7.0)      # nothing written past the row


@pytest.mark.parametrize("O_,K,T,pad", [
    (256, 64, 128, 0),
    (300, 323, 77, 0),        # ragged everywhere
    (130, 40, 50, 4),
    (1024, 1024, 512, 0),
    (66, 17, 202, 3),         # neither extent a multiple of 4, odd pitches
    (96, 3072, 4096, 0),      # one column of 128 x 96 tiles
    (768, 768, 64, 0),        # 32 x 32 tiles, reduction split inside the workgroup
])
def test_dense_tn_gemm_entry_point_single_precision(O_, K, T, pad):
    from sten_amd import native
    print(f"case gemm_tn f32 O={O_} K={K} T={T} pad={pad}", flush=True)
    dtype = torch.float32
    A = seeded((K, O_ + pad), dtype, seed=3, std=0.5).to(DEV)        # both reduction-major
    X = seeded((K, T + pad), dtype, seed=4).to(DEV)
    Y = torch.full((T, O_ + pad), 7.0, dtype=dtype, device=DEV)
    native.check(native.load().nmg_gemm_tn(A.data_ptr(), O_ + pad, X.data_ptr(), T + pad, Y.data_ptr(), O_ + pad,
                                           None, O_, K, T, native.dtype_code(dtype), native.stream_ptr(X.device)))
    ref = to_np(X)[:, :T].astype(np.float64).T @ to_np(A)[:, :O_].astype(np.float64)
    assert rel_l2(to_np(Y)[:, :O_], ref) <= TOL[dtype]
    if pad:
        assert torch.all(Y[:, O_:] == 7.0)


@pytest.mark.parametrize("R,C,N,n,m,g,sd", [(96, 240, 100, 3, 6, 4, 1), (256, 512, 64, 2, 4, 16, 0),
                                            (100, 90, 33, 1, 5, 2, 1)])
def test_single_precision_mm_and_its_gradients_keep_the_operands_as_they_lie(R, C, N, n, m, g, sd):
    print(f"case f32 torch.mm R={R} C={C} N={N} {n}:{m}:{g} sd={sd}", flush=True)
    dtype = torch.float32
    W = seeded((R, C), dtype, seed=R + C, std=0.5)
    Wd, _ = dense_ref(W, n, m, g, sd)
    w = make(W, n, m, g, sd)
    b = seeded((C, N), dtype, seed=7).to(DEV)
    c = sten.spmm_tt(w, b)
    assert c.shape == (R, N) and c.is_contiguous()
    assert rel_l2(to_np(c), Wd @ to_np(b).astype(np.float64)) <= TOL[dtype]
    gc = seeded((R, N), dtype, seed=8).to(DEV)
    gb = sten.spmm_tt_dense(w, gc, reduce_dim=0)
    assert gb.shape == (C, N) and gb.is_contiguous()
    assert rel_l2(to_np(gb), Wd.T @ to_np(gc).astype(np.float64)) <= TOL[dtype]


@pytest.mark.parametrize("sd", [1, 0])
@pytest.mark.parametrize("M,K,T,n,m,g", [(96, 240, 100, 3, 6, 4), (256, 512, 64, 2, 4, 16), (100, 90, 33, 1, 5, 2)])
def test_single_precision_large_batch_expands_then_multiplies(M, K, T, n, m, g, sd):
    print(f"case f32 expand route M={M} K={K} T={T} {n}:{m}:{g} sd={sd}", flush=True)
    dtype = torch.float32
    W = seeded((M, K), dtype, seed=M + K, std=0.5)
    x = seeded((T, K), dtype, seed=1)
    b = seeded((M,), dtype, seed=2)
    gy = seeded((T, M), dtype, seed=3)
    Wd, _ = dense_ref(W, n, m, g, sd)
    w = make(W, n, m, g, sd)
    y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)) <= TOL[dtype]
    gx = sten.spmm(w, gy.to(DEV), reduce_dim=0)
    assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[dtype]
    # the expanded operand follows the weight: an in-place update of val must show
    w.val.mul_(2.0)
    y2 = sten.spmm(w, x.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y2), 2.0 * (to_np(x).astype(np.float64) @ Wd.T)) <= TOL[dtype]
    # and the kernel that expands inside its loop stays reachable and agrees
    w.spmm_opt["expand"] = False
    y3 = sten.spmm(w, x.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y3), to_np(y2).astype(np.float64)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("dense_variant", [-1, 0, 1])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,T,n,m,g", [
    (256, 64, 128, 2, 4, 16),     # one tile, one K step
    (512, 320, 300, 4, 8, 4),     # 4:8 does not fit the sparse matrix cores; ragged tokens
    (320, 448, 77, 2, 4, 16),     # ragged outputs in both directions
    (1024, 1024, 512, 1, 2, 8),
    (192, 128, 40, 3, 16, 1),
    (320, 192, 70, 3, 6, 12),     # m = 6: tiles of 96 positions (the pattern of the reference's own matmul test)
    (384, 384, 130, 2, 3, 4),     # m = 3
    (192, 576, 33, 5, 12, 1),     # m = 12
])
def test_densefrag_route_both_directions(dense_variant, dtype, M, K, T, n, m, g):
    print(f"case densefrag v{dense_variant} {dtype} M={M} K={K} T={T} {n}:{m}:{g}", flush=True)
    W = seeded((M, K), dtype, seed=M + K + n, std=0.5)
    x = seeded((T, K), dtype, seed=1)
    b = seeded((M,), dtype, seed=2)
    gy = seeded((T, M), dtype, seed=3)
    for sd in (1, 0):
        Wd, _ = dense_ref(W, n, m, g, sd)
        w = make(W, n, m, g, sd)
        w.spmm_opt["dense_variant"] = dense_variant
        y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1, kernel="densefrag")
        ref = to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)
        assert rel_l2(to_np(y), ref) <= TOL[dtype], sd
        gx = sten.spmm(w, gy.to(DEV), reduce_dim=0, kernel="densefrag")
        assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[dtype], sd


def test_serialization_round_trip(tmp_path):
    # reference: tests/test_serialization.py saves and loads a model with sparse weights
    import pickle
    W = seeded((128, 128), torch.float16, seed=11, std=0.5)
    w = make(W, 2, 4, 16, 1)
    x = seeded((32, 128), torch.float16, seed=12).to(DEV)
    y = sten.spmm(w, x, reduce_dim=1)                    # builds the cached operands
    w2 = pickle.loads(pickle.dumps(w))
    assert torch.equal(w2.val, w.val) and torch.equal(w2.idx, w.idx) and w2.layout == w.layout
    assert torch.equal(sten.spmm(w2, x, reduce_dim=1), y)
    lin = build_sparse_linear(torch.nn.Linear(128, 128).half().to(DEV), 2, 4, 16, 1)
    path = tmp_path / "model.pt"
    torch.save(lin, path)
    lin2 = torch.load(path, weights_only=False)          # a file this test wrote itself
    assert isinstance(lin2.weight, sten.SparseParameterWrapper)
    with torch.no_grad():
        assert torch.equal(lin2(x), lin(x))


def _check_structure(w, n, m):
    """Size-independent properties of a compressed weight: every block of m keeps at most n
    entries, and the dense form reproduces the kept entries."""
    d = w.to_dense()
    blocks = d.reshape(d.shape[0], -1, m)
    assert int((blocks != 0).sum(dim=2).max()) <= n
    return d


@pytest.mark.parametrize("n,m", [(1, 8), (2, 8), (4, 8)])
def test_full_size_config3_forward(n, m):
    # benchmark config 3 at full size (8192 x 8192, group 32, 4096 tokens): structure of the
    # compressed weight, the product against the dense product of its own dense form, linearity
    print(f"case full size config 3 {n}:{m}", flush=True)
    torch.manual_seed(0)
    W = (torch.randn(8192, 8192) * 0.02).half().to(DEV)
    X = torch.randn(4096, 8192).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, n, m, sparse_dim=1, group_size=32, group_dim=0)
    d = _check_structure(w, n, m)
    kept = d != 0
    assert torch.equal(d[kept], W[kept])
    y = sten.spmm(w, X, reduce_dim=1)
    ref = torch.nn.functional.linear(X, d).float()
    assert float((y.float() - ref).norm() / ref.norm()) <= 1e-3
    y2 = sten.spmm(w, -0.5 * X, reduce_dim=1).float()
    assert float((y2 + 0.5 * y.float()).norm() / y2.norm()) <= 1e-3


def test_full_size_config5_training_step_pieces():
    # benchmark config 5 at full size: forward, grad_input (transposed product) and the masked
    # weight gradient in val layout, each against the dense computation on the dense form
    print("case full size config 5", flush=True)
    torch.manual_seed(0)
    W = (torch.randn(16384, 4096) * 0.02).half().to(DEV)
    X = torch.randn(4096, 4096).half().to(DEV)
    dY = torch.randn(4096, 16384).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=16, group_dim=0)
    d = _check_structure(w, 2, 4)
    y = sten.spmm(w, X, reduce_dim=1).float()
    ref = torch.nn.functional.linear(X, d).float()
    assert float((y - ref).norm() / ref.norm()) <= 1e-3
    gx = sten.spmm(w, dY, reduce_dim=0).float()
    ref = torch.mm(dY, d).float()
    assert float((gx - ref).norm() / ref.norm()) <= 1e-3
    gw_dense = torch.mm(dY.t(), X)                       # dense product; masked by the gather
    gw = w.clone_layout(gw_dense)
    assert torch.equal(gw.idx, w.idx)
    mask = w.clone_layout(torch.ones_like(W)).to_dense() != 0     # kept positions (a kept weight may be 0)
    back = gw.to_dense()
    assert torch.equal(back[mask], gw_dense[mask]) and not bool(back[~mask].any())


def test_cached_dense_operand_follows_weight_updates():
    W = seeded((256, 256), torch.float16, seed=21, std=0.5)
    w = make(W, 4, 8, 8, 1)
    w.spmm_opt["cache_dense"] = True
    x = seeded((64, 256), torch.float16, seed=22).to(DEV)
    y1 = sten.spmm(w, x, reduce_dim=1)
    assert torch.equal(sten.spmm(w, x, reduce_dim=1), y1)          # served from the cache
    w.mul_(2.0)                                                     # in-place update invalidates it
    y2 = sten.spmm(w, x, reduce_dim=1)
    assert rel_l2(to_np(y2), 2.0 * to_np(y1).astype(np.float64)) <= 1e-3


@pytest.mark.parametrize("T", [1, 2, 5, 7, 8, 9, 12, 13, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,n,m,g", [
    (515, 1024, 2, 4, 16),     # ragged lines, 16 wavefronts per line block
    (96, 128, 2, 4, 16),       # one chunk of 128 positions: most wavefronts have nothing to do
    (200, 2432, 1, 4, 8),      # k pairs not a multiple of the wavefront count
    (64, 192, 2, 4, 16),       # K % 128 != 0: the staging kernel steps aside
    (8224, 256, 2, 8, 4),      # >= 256 line blocks: 4 wavefronts per workgroup
])
def test_decode_kernels_all_token_counts(T, dtype, M, K, n, m, g):
    print(f"case decode {dtype} M={M} K={K} T={T} {n}:{m}:{g}", flush=True)
    W = seeded((M, K), dtype, seed=M + K + T, std=0.05)
    Wd, _ = dense_ref(W, n, m, g, 1)
    w = make(W, n, m, g, 1)
    x = seeded((T, K), dtype, seed=6)
    b = seeded((M,), dtype, seed=7)
    ref = to_np(x).astype(np.float64) @ Wd.T + to_np(b).astype(np.float64)
    y = sten.spmm(w, x.to(DEV), b.to(DEV), reduce_dim=1)
    assert rel_l2(to_np(y), ref) <= TOL[dtype]


@pytest.mark.parametrize("M,K,T", [
    (1024, 1024, 4),       # decode kernel
    (1024, 1024, 512),     # sparse matrix cores, direct kernel
])
def test_hip_graph_replays_match_eager(M, K, T):
    # A serving loop records the product once and replays it.  Every replay is checked against
    # an eager call on the same input, with eager work and synchronisations between the replays.
    print(f"case graph replay M={M} K={K} T={T}", flush=True)
    w = make(seeded((M, K), torch.float16, seed=31, std=0.05), 2, 4, 16, 1)
    x = seeded((T, K), torch.float16, seed=32).to(DEV)
    b = seeded((M,), torch.float16, seed=33).to(DEV)
    sten.spmm(w, x, b, reduce_dim=1)           # first call: tables and operand caches are set up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = sten.spmm(w, x, b, reduce_dim=1)
    for seed in (40, 41, 42):
        x.copy_(seeded((T, K), torch.float16, seed=seed).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        want = sten.spmm(w, x, b, reduce_dim=1)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay with input seed {seed} differs from the eager call"


@pytest.mark.parametrize("dtype,n,m,g,sd,T", [
    (torch.float16, 2, 4, 16, 0, 4),      # reduction along the group dim, few tokens: dense-core operand in slices
    (torch.float16, 4, 8, 4, 1, 16),      # no sparse-core operand
    (torch.float32, 2, 4, 16, 1, 4),      # fp32: dense copy + fp32 GEMM
    (torch.float32, 2, 4, 16, 1, 300),
])
def test_hip_graph_replays_of_the_dense_routes_match_eager(dtype, n, m, g, sd, T):
    # the split reduction allocates its workspace inside the capture; every replay is checked
    # against an eager call, with eager work and synchronisations between the replays
    print(f"case graph replay dense routes {dtype} {n}:{m}:{g} sd={sd} T={T}", flush=True)
    M, K = 1024, 2048
    w = make(seeded((M, K), dtype, seed=31, std=0.05), n, m, g, sd)
    x = seeded((T, K), dtype, seed=32).to(DEV)
    b = seeded((M,), dtype, seed=33).to(DEV)
    sten.spmm(w, x, b, reduce_dim=1)           # first call: tables and operand caches are set up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = sten.spmm(w, x, b, reduce_dim=1)
    for seed in (40, 41, 42):
        x.copy_(seeded((T, K), dtype, seed=seed).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        want = sten.spmm(w, x, b, reduce_dim=1)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay with input seed {seed} differs from the eager call"


def test_tile_boundary_sweep_default_route():
    # The reference sweeps every size across each tile boundary +-1 (matmul_generator.py:1482-1521).
    # Here the boundaries are those of the default kernels: 32 / 64 / 256 lines, 16 / 128 / 256
    # tokens, 64 / 128 reduction positions; whatever kernel the sizes select must agree with the
    # dense product of the oracle's weight.
    n, m, g = 2, 4, 16
    for M in (255, 256, 257, 96 * 3 + 1):
        for K in (64, 120, 128, 136, 192, 200):
            W = seeded((M, K), torch.float16, seed=M * 7 + K, std=0.5)
            Wd, _ = dense_ref(W, n, m, g, 1)
            w = make(W, n, m, g, 1)
            for T in (1, 15, 16, 17, 127, 128, 129, 255, 256, 257):
                print(f"case sweep M={M} K={K} T={T}", flush=True)
                x = seeded((T, K), torch.float16, seed=T)
                y = sten.spmm(w, x.to(DEV), reduce_dim=1)
                assert rel_l2(to_np(y), to_np(x).astype(np.float64) @ Wd.T) <= TOL[torch.float16], (M, K, T)
                gy = seeded((T, M), torch.float16, seed=T + 1)
                gx = sten.spmm(w, gy.to(DEV), reduce_dim=0)
                assert rel_l2(to_np(gx), to_np(gy).astype(np.float64) @ Wd) <= TOL[torch.float16], (M, K, T)


def test_weight_of_more_than_2_31_elements():
    # 40000 x 54016 fp16: element, slot and byte offsets beyond 32 bits in every kernel of the
    # path.  Tiles are independent, so the oracle checks whole chunks cut out of the weight; the
    # products are checked against the dense product of the library's own to_dense.
    M, K = 40000, 54016
    torch.manual_seed(0)
    W = torch.empty(M, K, dtype=torch.float16, device=DEV).normal_(0, 0.02)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=16, group_dim=0)
    lay = w.layout
    cols, nb = lay.cols, lay.num_blocks
    assert M * K > 2 ** 31 and w.val.numel() * 2 > 2 ** 31       # elements, bytes of val
    for kc in (0, M // cols - 1, M // cols):          # first, last whole and the ragged last chunk
        print(f"case big chunk {kc}", flush=True)
        r0, r1 = kc * cols, min(M, (kc + 1) * cols)
        val, idx, _ = oracle_sparsify(W[r0:r1].cpu(), 2, 4, 1, 16, 0)
        assert np.array_equal(to_np(w.idx[kc * nb:(kc + 1) * nb]), idx)
        assert np.array_equal(to_np(w.val[kc * nb:(kc + 1) * nb]).view(np.uint16), val.view(np.uint16))
    D = w.to_dense()
    assert bool(((D == W) | (D == 0)).all())
    del W
    for T in (5, 200):
        print(f"case big T={T}", flush=True)
        x = torch.randn(T, K, dtype=torch.float16, device=DEV)
        ref = (x @ D.t()).float()
        assert float((sten.spmm(w, x, reduce_dim=1).float() - ref).norm() / ref.norm()) <= 2e-3
        gy = torch.randn(T, M, dtype=torch.float16, device=DEV)
        ref = (gy @ D).float()
        assert float((sten.spmm(w, gy, reduce_dim=0).float() - ref).norm() / ref.norm()) <= 2e-3


def test_direct_kernels_on_a_full_chip_with_a_long_reduction():
    # One tile per CU (or two) and 256 K steps: the shape on which a mistimed wait in the
    # hand-scheduled kernels shows.  The pipelined variants must reproduce the plain kernel
    # (variant 0) bit for bit on every run, and the dense route the dense product.
    M, K, T = 4096, 16384, 4096
    print(f"case full chip M={M} K={K} T={T}", flush=True)
    w = make(seeded((M, K), torch.float16, seed=77, std=0.02), 2, 4, 16, 1)
    x = seeded((T, K), torch.float16, seed=78).to(DEV)
    w.spmm_opt["variant"] = 0
    ref = sten.spmm(w, x, reduce_dim=1, kernel="smfmac").clone()
    for variant in (6, 8):
        w.spmm_opt["variant"] = variant
        for _ in range(4):
            assert torch.equal(sten.spmm(w, x, reduce_dim=1, kernel="smfmac"), ref), f"variant {variant}"
    g = seeded((T, M), torch.float16, seed=79).to(DEV)
    want = (g @ w.to_dense()).float()
    for dense_variant in (0, 1):
        w.spmm_opt["dense_variant"] = dense_variant
        for _ in range(4):
            got = sten.spmm(w, g, reduce_dim=0, kernel="densefrag").float()
            assert float((got - want).norm() / want.norm()) <= 1e-4, f"dense variant {dense_variant}"
