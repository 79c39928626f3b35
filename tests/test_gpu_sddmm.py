"""GPU parity of the masked weight gradient written straight into the val layout (nmg_sddmm).
Oracle: the dense product dY^T X in fp64, merged into tiles and gathered at the oracle's own
pattern (the same-pattern gather the reference describes in grouped_nm_tensor.py:908-951).
Tolerance: rel-L2 <= 1e-3 for fp16 with fp32 accumulation (8e-3 for bf16, whose rounding step is
8x coarser); slots of padded lines and positions must be exact zeros; idx is shared, not copied."""
import ctypes

import numpy as np
import pytest
import torch

import sten_amd as sten
from sten_amd import native
from oracle import nmg_oracle as O
from helpers import oracle_sparsify, rel_l2, seeded, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float16: 1e-3, torch.bfloat16: 8e-3}


def oracle_masked_grad(gy, x, idx, lay):
    """fp64 dY^T X -> tiles -> values at the kept positions, plus the mask of real (unpadded) slots."""
    gw = to_np(gy).astype(np.float64).T @ to_np(x).astype(np.float64)
    ref = O.gather_merged(O.merge(gw, lay), idx, lay.n)
    real = O.gather_merged(O.merge(np.ones_like(gw), lay), idx, lay.n) != 0
    return ref, real


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("R,C,T,n,m,g,sd", [
    (256, 256, 64, 2, 4, 16, 1),        # one tile, whole K steps
    (256, 256, 64, 2, 4, 16, 0),        # the reference's default orientation
    (200, 136, 37, 2, 4, 4, 1),         # ragged everywhere: lines, positions, tokens
    (200, 136, 37, 2, 4, 4, 0),
    (520, 264, 100, 1, 8, 2, 1),        # several tiles in both dims, padded chunks
    (264, 776, 33, 2, 8, 4, 1),         # 112-line chunks straddle the 256-line tiles
    (264, 776, 129, 4, 8, 2, 0),
    (96, 528, 200, 3, 6, 2, 1),         # m does not divide 256: blocks straddle position tiles
    (528, 96, 31, 3, 6, 2, 0),
    (64, 48, 7, 1, 1, 8, 1),            # n == m: nothing dropped
    (768, 1024, 160, 2, 4, 1, 1),       # group size 1
    (1800, 512, 96, 2, 8, 32, 1),       # config 3's patterns: chunks of 896 / 2240 lines span several tiles
    (2240, 264, 64, 4, 8, 32, 0),
    (520, 512, 40, 1, 8, 32, 1),
])
def test_masked_product_matches_oracle(dtype, R, C, T, n, m, g, sd):
    print(f"case sddmm {dtype} R={R} C={C} T={T} {n}:{m}:{g} sd={sd}", flush=True)
    W = seeded((R, C), dtype, seed=R + C, std=0.5)
    gy = seeded((T, R), dtype, seed=3)
    x = seeded((T, C), dtype, seed=4)
    _, idx, lay = oracle_sparsify(W, n, m, sd, g, 1 - sd)
    ref, real = oracle_masked_grad(gy, x, idx, lay)
    w = sten.GroupedNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=1 - sd)
    assert np.array_equal(to_np(w.idx), idx)
    gw = w.masked_product(gy.to(DEV), x.to(DEV))
    assert gw.idx is w.idx and gw.layout == w.layout
    got = to_np(gw.val).astype(np.float64)
    assert got.shape == ref.shape
    assert not got[~real].any(), "slots of padded lines / positions must be zero"
    assert rel_l2(got, ref) <= TOL[dtype]
    # the same numbers through the separate dense product and gather
    two_pass = w.clone_layout(torch.mm(gy.to(DEV).t(), x.to(DEV)))
    assert rel_l2(got, to_np(two_pass.val).astype(np.float64)) <= 2 * TOL[dtype]


def test_masked_product_strided_operands_and_linearity():
    print("case sddmm strided operands", flush=True)
    torch.manual_seed(1)
    R, C, T = 512, 384, 96
    W = (torch.randn(R, C) * 0.1).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=16, group_dim=0)
    big_gy = torch.randn(T, R + 64, device=DEV).half()
    big_x = torch.randn(T, C + 8, device=DEV).half()
    gy, x = big_gy[:, 32:32 + R], big_x[:, 8:]          # leading dims 576 / 392, offsets keep 16-byte alignment
    a = w.masked_product(gy, x)
    b = w.masked_product(gy.contiguous(), x.contiguous())
    assert torch.equal(a.val, b.val)
    c = w.masked_product(gy.contiguous(), (-2 * x).contiguous())
    # linearity; not bit-exact: the matrix cores' fp32 accumulation is not symmetric under a sign
    # flip (measured: 5 of 110592 values differ by one fp16 step)
    assert float((c.val.float() + 2 * a.val.float()).norm() / c.val.float().norm()) <= 1e-3
    # deterministic: the same call gives the same bits
    assert torch.equal(w.masked_product(gy, x).val, a.val)


def test_masked_product_argument_errors():
    W = torch.randn(64, 64).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=4, group_dim=0)
    with pytest.raises(native.NmgError):
        w.masked_product(torch.randn(8, 64, device=DEV).half(), torch.randn(9, 64, device=DEV).half())
    with pytest.raises(native.NmgError):
        w.masked_product(torch.randn(8, 64, device=DEV), torch.randn(8, 64, device=DEV))
    lib = native.load()
    slot = w.slotmap()
    x = torch.randn(8, 64, device=DEV).half()
    out = torch.empty_like(w.val)
    # extents that are not multiples of 8 are refused, not mis-read
    rc = lib.nmg_sddmm(native.ptr(x), 64, native.ptr(x), 64, 8, native.ptr(slot), 60, 64, native.ptr(out),
                       2, 4, 4, native.NMG_F16, None)
    assert rc == 2 and b"multiples of 8" in lib.nmg_last_error()
    rc = lib.nmg_sddmm(None, 64, native.ptr(x), 64, 8, native.ptr(slot), 64, 64, native.ptr(out),
                       2, 4, 4, native.NMG_F16, None)
    assert rc == 1
    rc = lib.nmg_sddmm(native.ptr(x), 64, native.ptr(x), 64, 8, native.ptr(slot), 64, 64, native.ptr(out),
                       2, 4, 4, native.NMG_F32, None)
    assert rc == 2


def test_slotmap_is_the_inverse_of_idx():
    print("case slotmap", flush=True)
    for (R, C, n, m, g, sd) in [(200, 136, 2, 4, 4, 1), (264, 776, 2, 8, 4, 0), (96, 528, 3, 6, 2, 1)]:
        W = seeded((R, C), torch.float16, seed=R)
        _, idx, lay = oracle_sparsify(W, n, m, sd, g, 1 - sd)
        w = sten.GroupedNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=1 - sd)
        slot = to_np(w.slotmap())
        cg = lay.c * lay.g
        tiles = idx.reshape(lay.num_chunks, lay.num_blocks, cg).astype(np.int64)
        expect = np.empty((lay.num_blocks, lay.num_chunks * cg), dtype=np.int16)
        for kc in range(lay.num_chunks):
            for b in range(lay.num_blocks):
                expect[b, kc * cg + tiles[kc, b]] = np.arange(cg, dtype=np.int16)
        assert np.array_equal(slot, expect)


def test_full_size_config5_weight_gradient():
    # benchmark config 5 at full size: 16384 x 4096 weight, 2:4:16 along the reduction, 4096 tokens.
    # Against the dense library product gathered at the same pattern (all of it) and against the
    # fp64 product of a band of 96 lines (one chunk) computed on the host.
    print("case full size config 5 weight gradient", flush=True)
    torch.manual_seed(0)
    W = (torch.randn(16384, 4096) * 0.02).half().to(DEV)
    X = torch.randn(4096, 4096).half().to(DEV)
    dY = torch.randn(4096, 16384).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=16, group_dim=0)
    gw = w.masked_product(dY, X)
    two_pass = w.clone_layout(torch.mm(dY.t(), X))
    diff = (gw.val.float() - two_pass.val.float()).norm() / two_pass.val.float().norm()
    assert float(diff) <= 1e-3
    lines = slice(96 * 7, 96 * 8)
    band = dY[:, lines].double().t().cpu().numpy() @ X.double().cpu().numpy()          # [96, 4096] fp64
    dense = gw.to_dense()[lines].double().cpu().numpy()
    kept = w.clone_layout(torch.ones_like(W)).to_dense()[lines].cpu().numpy() != 0
    assert kept.sum() == 96 * 4096 // 2
    assert rel_l2(dense[kept], band[kept]) <= 1e-3
    assert not dense[~kept].any()


def test_training_step_uses_the_fused_kernel():
    # F.linear backward with a compressed weight gradient: same numbers as dense autograd masked
    print("case sddmm through the registered backward", flush=True)
    torch.manual_seed(2)
    lin = torch.nn.Linear(256, 384, bias=True).half().to(DEV)
    W = lin.weight.detach().clone()
    sb = sten.SparsityBuilder()
    sb.set_weight("weight", initial_sparsifier=sten.GroupedNMSparsifier(2, 4, 16, sparse_dim=1, group_dim=0),
                  out_format=sten.GroupedNMTensor)
    sb.set_weight_grad("weight", tmp_format=sten.GroupedNMTensor, out_format=sten.GroupedNMTensor)
    sp = sb.get_sparse_model(lin)
    x = torch.randn(100, 256, device=DEV).half().requires_grad_(True)
    gy = torch.randn(100, 384, device=DEV).half()
    sp(x).backward(gy)
    g = sp.weight.grad.wrapped_tensor
    assert isinstance(g, sten.GroupedNMTensor)
    w = sp.weight.wrapped_tensor
    ref = w.clone_layout((gy.double().t() @ x.detach().double()).half())
    assert float((g.val.float() - ref.val.float()).norm() / ref.val.float().norm()) <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("R,C,T,n,m,g,sd", [
    (256, 256, 64, 2, 4, 16, 1),
    (200, 136, 40, 2, 4, 4, 1),          # ragged lines and positions, tokens end inside a K step
    (203, 131, 24, 2, 4, 4, 0),          # extents that are no multiples of 8: fine in this form
    (520, 264, 104, 1, 8, 2, 1),         # patterns outside 2:4 go through the staged epilogue
    (264, 776, 136, 4, 8, 2, 0),
    (96, 528, 200, 3, 6, 2, 1),
    (768, 1024, 160, 2, 4, 1, 1),
    (256, 512, 72, 1, 4, 8, 1),          # the other epilogues in registers: m = 4 with n = 1, 3, 4 ...
    (512, 264, 96, 3, 4, 2, 0),
    (264, 256, 40, 4, 4, 4, 1),
    (512, 512, 136, 1, 8, 32, 1),        # ... and m = 8 with n = 1, 2, 4
    (896, 264, 64, 2, 8, 32, 0),
    (280, 512, 48, 4, 8, 4, 1),
])
def test_masked_product_reduction_contiguous_operands(dtype, R, C, T, n, m, g, sd):
    # operands given as [R, T] and [C, T] (the weight gradient of torch.mm(W, B)): same values as
    # the token-major form on the transposed copies, and the oracle's gather of the fp64 product
    print(f"case sddmm nt {dtype} R={R} C={C} T={T} {n}:{m}:{g} sd={sd}", flush=True)
    W = seeded((R, C), dtype, seed=R + C, std=0.5)
    gy = seeded((R, T), dtype, seed=5)
    b = seeded((C, T), dtype, seed=6)
    _, idx, lay = oracle_sparsify(W, n, m, sd, g, 1 - sd)
    ref, real = oracle_masked_grad(gy.t(), b.t(), idx, lay)
    w = sten.GroupedNMTensor.from_dense(W.to(DEV), n, m, sparse_dim=sd, group_size=g, group_dim=1 - sd)
    gw = w.masked_product(gy.to(DEV), b.to(DEV), reduction_last=True)
    got = to_np(gw.val).astype(np.float64)
    assert not got[~real].any()
    assert rel_l2(got, ref) <= TOL[dtype]
    if R % 8 == 0 and C % 8 == 0:
        other = w.masked_product(gy.t().contiguous().to(DEV), b.t().contiguous().to(DEV))
        assert torch.equal(gw.val, other.val)      # same products in the same order
    # strided operands (row pitch larger than T)
    big = torch.zeros((R, T + 24), dtype=dtype)
    big[:, 8:8 + T] = gy
    gw2 = w.masked_product(big.to(DEV)[:, 8:8 + T], b.to(DEV), reduction_last=True)
    assert torch.equal(gw2.val, gw.val)


def test_masked_product_reduction_contiguous_argument_errors():
    W = torch.randn(64, 64).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=4, group_dim=0)
    with pytest.raises(native.NmgError):   # token counts differ
        w.masked_product(torch.randn(64, 16, device=DEV).half(), torch.randn(64, 24, device=DEV).half(), reduction_last=True)
    with pytest.raises(native.NmgError):   # 12 tokens: not a multiple of 8
        w.masked_product(torch.randn(64, 12, device=DEV).half(), torch.randn(64, 12, device=DEV).half(), reduction_last=True)


def test_weight_gradient_of_torch_mm_from_its_operands_as_they_lie():
    print("case sddmm nt on the operands of a torch.mm backward", flush=True)
    torch.manual_seed(3)
    R, C, N = 192, 256, 72
    W = (torch.randn(R, C) * 0.1).half().to(DEV)
    w = sten.GroupedNMTensor.from_dense(W, 2, 4, sparse_dim=1, group_size=8, group_dim=0)
    B = torch.randn(C, N, device=DEV).half()
    gc = torch.randn(R, N, device=DEV).half()
    got = w.masked_product(gc, B, reduction_last=True)
    ref = w.clone_layout((gc.double() @ B.double().t()).half())
    assert float((got.val.float() - ref.val.float()).norm() / ref.val.float().norm()) <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("R,C,T,bias", [
    (256, 256, 64, False),       # one tile, whole K steps
    (200, 136, 37, True),        # ragged lines, positions and tokens
    (520, 776, 100, False),      # several tiles both ways
    (8, 8, 1, True),             # smallest extents the kernel takes
    (1024, 512, 4096, False),    # 128 K steps
])
def test_dense_weight_gradient_in_16_bit(dtype, R, C, T, bias):
    # the dense weight gradient dY^T X of a linear layer (default gradient format) on the kernel of
    # the masked product without its mask: nmg_gemm_tn in f16 / bf16 against the fp64 product
    print(f"case gemm_tn16 {dtype} R={R} C={C} T={T} bias={bias}", flush=True)
    gy = seeded((T, R), dtype, seed=R + T).to(DEV)
    x = seeded((T, C), dtype, seed=C + T + 1).to(DEV)
    b = seeded((C,), dtype, seed=3).to(DEV) if bias else None
    # a result with a row pitch: every second row of a larger buffer stays untouched
    buf = torch.full((R, 2 * C), 7.0, dtype=dtype, device=DEV)
    out = buf[:, :C]
    native.check(native.load().nmg_gemm_tn(
        native.ptr(x), x.stride(0), native.ptr(gy), gy.stride(0), native.ptr(out), out.stride(0),
        native.ptr(b), C, T, R, native.dtype_code(dtype), None))
    torch.cuda.synchronize()
    ref = to_np(gy).astype(np.float64).T @ to_np(x).astype(np.float64)
    if bias:
        ref = ref + to_np(b).astype(np.float64)
    assert rel_l2(to_np(out), ref) <= TOL[dtype]
    assert bool((buf[:, C:] == 7.0).all()), "wrote beyond the rows of the result"


@pytest.mark.parametrize("fin,fout,tokens", [
    (256, 384, 72),
    (250, 380, 37),     # extents that the 16-bit kernels do not take: widened, through the fp32 kernel
])
def test_default_gradient_format_takes_no_library_gemm(monkeypatch, fin, fout, tokens):
    # F.linear backward with the default (dense) weight-gradient format in fp16: forward, grad_input and
    # the dense dY^T X all run on this library's kernels -- torch.mm must not be called
    print(f"case default grad format {fin}->{fout} x {tokens}", flush=True)
    torch.manual_seed(0)
    lin = torch.nn.Linear(fin, fout, bias=True).half().to(DEV)
    sb = sten.SparsityBuilder()
    sb.set_weight("weight", initial_sparsifier=sten.GroupedNMSparsifier(2, 4, 16, sparse_dim=1, group_dim=0),
                  out_format=sten.GroupedNMTensor)
    sp = sb.get_sparse_model(lin)
    Wd = sp.weight.wrapped_tensor.to_dense().detach().float()
    x = torch.randn(tokens, fin, device=DEV).half().requires_grad_(True)
    gy = torch.randn(tokens, fout, device=DEV).half()

    def no_mm(*a, **k):
        raise AssertionError("torch.mm was called in the backward of the sparse linear")
    monkeypatch.setattr(torch, "mm", no_mm)
    y = sp(x)
    y.backward(gy)
    monkeypatch.undo()
    gw = sp.weight.grad.wrapped_tensor.to_dense().float()
    assert rel_l2(to_np(gw), to_np(gy.float().t() @ x.detach().float())) <= 1e-3
    assert rel_l2(to_np(x.grad.float()), to_np(gy.float() @ Wd)) <= 1e-3
