"""``GroupedNMTensor`` -- the grouped n:m container, API-compatible with the reference class
(src/sten/grouped_nm/grouped_nm_tensor.py:877-958: ``val``, ``idx``, ``nm_strides``,
``from_dense``, ``to_dense``, ``set_spmm_opt``) and extended with what a wrapped format needs on
a GPU: ``dtype`` / ``device`` / ``shape`` / ``to``, same-pattern re-compression
(the disabled ``clone_layout``, :904-951) and in-place ``add_`` / ``mul_`` for optimizers.

All compute goes through libnmg_hip.so; tensors must live on the GPU.
"""
import ctypes
import weakref

import torch

from . import native
from .layout import NMGLayout, bgs_view


class GroupedNMTensor:
    def __init__(self, val, idx, layout):
        if isinstance(layout, dict):  # accept the reference's nm_strides dict
            layout = NMGLayout(tuple(layout["dense_shape"]), layout["n"], layout["m"],
                               layout["group_size"], layout["sparse_dim"], layout["group_dim"])
        self.val = val
        self.idx = idx
        self.layout = layout
        self.spmm_opt = {"kernel": "auto"}
        self._rowpack = None

    def _version_key(self):
        """Identity and version of ``val`` and ``idx``: what every derived operand depends on.  The
        tensors are named by weak reference, not by address -- the allocator hands a freed block
        back at the same address, and tensors written by the library's kernels all carry version 0."""
        return (weakref.ref(self.val), self.val._version, weakref.ref(self.idx), self.idx._version)

    def _key_current(self, key):
        return (key is not None and key[0]() is self.val and key[1] == self.val._version
                and key[2]() is self.idx and key[3] == self.idx._version)

    def _drop_operands(self):
        """Forget every operand derived from ``val`` (in-place updates call this)."""
        self._rowpack = None
        self._fragpack = None
        self._densefrag = None
        self._dense_operand = None
        self._lanepack8 = None
        self._gpack = None
        self._opack = None

    # ---- construction ----------------------------------------------------------------------
    @staticmethod
    def from_dense(tensor, n, m, sparse_dim, group_size, group_dim):
        """Per-tile magnitude selection, bit-exact with the reference CPU sparsifier
        (grouped_nm_tensor.py:883-890 -> :701-710 -> :255-297)."""
        native.require_gpu(tensor)
        sparse_dim %= tensor.dim()
        group_dim %= tensor.dim()
        lay = NMGLayout(tuple(tensor.shape), n, m, group_size, sparse_dim, group_dim)
        t = tensor.detach()
        q, view = bgs_view(t, lay)
        val = torch.empty(lay.val_shape, dtype=t.dtype, device=t.device)
        idx = torch.empty(lay.idx_shape, dtype=torch.int16, device=t.device)
        with torch.cuda.device(t.device):
            native.check(native.load().nmg_sparsify(
                native.ptr(q), ctypes.byref(view), native.ptr(val), native.ptr(idx),
                n, m, group_size, native.dtype_code(t.dtype), native.stream_ptr(t.device)))
        return GroupedNMTensor(val, idx, lay)

    def clone_layout(self, dense_tensor):
        """New tensor with this tensor's pattern and the values of ``dense_tensor`` at the kept
        positions (what grouped_nm_tensor.py:908-951 describes)."""
        if tuple(dense_tensor.shape) != tuple(self.layout.dense_shape):
            raise ValueError(
                f"Shape mismatch: expected {self.layout.dense_shape}, received {tuple(dense_tensor.shape)}")
        native.require_gpu(dense_tensor, self.val)
        lay = self.layout
        t = dense_tensor.detach().to(dtype=self.val.dtype)
        q, view = bgs_view(t, lay)
        val = torch.empty_like(self.val)
        with torch.cuda.device(t.device):
            native.check(native.load().nmg_gather(
                native.ptr(q), ctypes.byref(view), native.ptr(self.idx), native.ptr(val),
                lay.n, lay.m, lay.group_size, native.dtype_code(val.dtype),
                native.stream_ptr(t.device)))
        out = GroupedNMTensor(val, self.idx, lay)
        out.spmm_opt = dict(self.spmm_opt)
        return out

    # ---- reference-compatible surface ------------------------------------------------------------
    @property
    def nm_strides(self):
        d = self.layout.as_nm_strides()
        d.update(self.spmm_opt)
        return d

    def set_spmm_opt(self, tile_a=None, acc_width=None, tile_b=None, kernel=None):
        """Reference signature (grouped_nm_tensor.py:892-902).  The CPU tile parameters have no
        meaning here; ``kernel`` selects the GPU matmul kernel: auto | mfma | smfmac | skinny."""
        if kernel is not None:
            if kernel not in native.KERNELS:
                raise ValueError(f"kernel must be one of {sorted(native.KERNELS)}")
            self.spmm_opt["kernel"] = kernel
        for k, v in (("tile_a", tile_a), ("acc_width", acc_width), ("tile_b", tile_b)):
            if v is not None:
                self.spmm_opt[k] = v

    def to_dense(self):
        lay = self.layout
        native.require_gpu(self.val)
        out = torch.empty(lay.dense_shape, dtype=self.val.dtype, device=self.val.device)
        q, view = bgs_view(out, lay)
        aliased = q.untyped_storage().data_ptr() == out.untyped_storage().data_ptr()
        with torch.cuda.device(out.device):
            native.check(native.load().nmg_to_dense(
                native.ptr(self.val), native.ptr(self.idx), native.ptr(q), ctypes.byref(view),
                lay.n, lay.m, lay.group_size, native.dtype_code(out.dtype),
                native.stream_ptr(out.device)))
        if not aliased:
            sizes = [lay.dense_shape[d] for d in lay.other_dims] + [lay.G, lay.S]
            perm = lay.other_dims + [lay.group_dim, lay.sparse_dim]
            inv = sorted(range(len(perm)), key=lambda i: perm[i])
            out = q.view(sizes).permute(inv).contiguous()
        return out

    # ---- tensor-like attributes the wrapper machinery looks for -------------------------------
    @property
    def dtype(self):
        return self.val.dtype

    @property
    def device(self):
        return self.val.device

    @property
    def shape(self):
        return torch.Size(self.layout.dense_shape)

    def size(self, dim=None):
        return self.shape if dim is None else self.shape[dim]

    def dim(self):
        return len(self.layout.dense_shape)

    def numel(self):
        return self.shape.numel()

    def to(self, device=None, dtype=None, non_blocking=False, copy=False, **_):
        val = self.val.to(device=device, dtype=dtype, non_blocking=non_blocking, copy=copy)
        idx = self.idx.to(device=device, non_blocking=non_blocking, copy=copy)
        out = GroupedNMTensor(val, idx, self.layout)
        out.spmm_opt = dict(self.spmm_opt)
        return out

    def clone(self):
        return self.to(copy=True)

    # ---- serialization: the canonical val/idx and the layout; derived operands are rebuilt ----
    def __getstate__(self):
        return {"val": self.val, "idx": self.idx, "layout": self.layout, "spmm_opt": dict(self.spmm_opt)}

    def __setstate__(self, state):
        self.__init__(state["val"], state["idx"], state["layout"])
        self.spmm_opt = state.get("spmm_opt", {"kernel": "auto"})

    # ---- in-place updates that keep the pattern (used by optimizers) ------------------------
    def _same_pattern(self, other):
        """True when ``other`` keeps the same positions in the same slots: it shares this
        tensor's ``idx`` (every ``clone_layout`` result does) or holds an equal copy.  The
        comparison of two distinct ``idx`` tensors is made once per pair and remembered."""
        if other.idx is self.idx or (other.idx.data_ptr() == self.idx.data_ptr()
                                     and other.idx.shape == self.idx.shape):
            return True
        cached = getattr(self, "_pattern_eq", None)
        if (cached is not None and cached[0]() is other.idx and cached[1] == other.idx._version
                and cached[2] == self.idx._version):
            return cached[3]
        same = other.idx.device == self.idx.device and bool(torch.equal(other.idx, self.idx))
        # remembered per tensor object (weak reference), not per address: a freed idx block comes
        # back at the same address with another pattern in it
        self._pattern_eq = (weakref.ref(other.idx), other.idx._version, self.idx._version, same)
        return same

    def _other_val(self, other):
        if isinstance(other, GroupedNMTensor):
            if other.layout != self.layout:
                raise ValueError("layout mismatch")
            if self._same_pattern(other):
                return other.val
            # same layout, another choice of columns: slot s of the two tensors names different
            # positions, so the values go through the dense view and are gathered at this
            # tensor's kept positions
            return self.clone_layout(other.to_dense()).val
        if hasattr(other, "wrapped_tensor"):
            return self._other_val(other.wrapped_tensor)
        if hasattr(other, "to_dense") and not isinstance(other, torch.Tensor):
            other = other.to_dense()
        if isinstance(other, torch.Tensor) and other.dim() > 0:
            return self.clone_layout(other).val
        return other

    def add_(self, other, *, alpha=1):
        self.val.add_(self._other_val(other), alpha=alpha)
        self._drop_operands()
        return self

    def mul_(self, other):
        self.val.mul_(self._other_val(other))
        self._drop_operands()
        return self

    def zero_(self):
        self.val.zero_()
        self._drop_operands()
        return self

    def copy_(self, other):
        self.val.copy_(self._other_val(other))
        self._drop_operands()
        return self

    # ---- matmul operand ---------------------------------------------------------------------------
    def _pack(self):
        """Derive the matmul operands from val/idx in one pass: the rowpack operand always, the
        operand of the sparse matrix cores when the type and the pattern have one."""
        lay = self.layout
        if len(lay.dense_shape) != 2:
            raise native.NmgError("matmul needs a 2-D grouped n:m tensor")
        if self._rowpack is not None and self._key_current(self._rowpack[0]):
            return
        key = self._version_key()
        native.require_gpu(self.val)
        lib = native.load()
        dev, dt = self.val.device, self.val.dtype
        pat_bytes = lib.nmg_rowpack_pat_bytes(lay.n, lay.m)
        pk_val = torch.empty((lay.G, lay.num_blocks, lay.n), dtype=dt, device=dev)
        pk_pat = torch.empty((lay.G, lay.num_blocks), dtype=torch.uint8 if pat_bytes == 1 else torch.int16,
                             device=dev)
        fp_val = fp_idx = None
        if dt in (torch.float16, torch.bfloat16) and lib.nmg_fragpack_supported(lay.n, lay.m):
            ve, iw = ctypes.c_int64(), ctypes.c_int64()
            native.check(lib.nmg_fragpack_sizes(lay.G, lay.S, ctypes.byref(ve), ctypes.byref(iw)))
            fp_val = torch.empty(ve.value, dtype=dt, device=dev)
            fp_idx = torch.empty(iw.value, dtype=torch.int32, device=dev)
        with torch.cuda.device(dev):
            native.check(lib.nmg_pack_operands(
                native.ptr(self.val), native.ptr(self.idx), lay.G, lay.S, native.ptr(pk_val),
                native.ptr(pk_pat), native.ptr(fp_val) if fp_val is not None else None,
                native.ptr(fp_idx) if fp_idx is not None else None, lay.n, lay.m, lay.group_size,
                native.dtype_code(dt), native.stream_ptr(dev)))
        self._rowpack = (key, pk_val, pk_pat)
        self._fragpack = (key, fp_val, fp_idx) if fp_val is not None else None

    def rowpack(self):
        """(pk_val [G, nb, n], pk_pat [G, nb]) -- per line of the group dim and block of the
        sparse dim, the kept values and the pattern number; cached until ``val`` changes."""
        self._pack()
        return self._rowpack[1], self._rowpack[2]

    def densefrag(self, reduce_dim):
        """The weight as the A operand of the dense matrix cores, [outputs, reduction] in
        fragment order, expanded from the rowpack operand.  It is as large as the dense weight.
        It is kept until ``val`` changes (one copy per reduction direction), so a frozen weight,
        or the forward and backward of one training step, pay the expansion once;
        ``spmm_opt["cache_dense"] = False`` rebuilds it per call instead and keeps the memory of
        the compressed format."""
        lay = self.layout
        lib = native.load()
        keep = self.spmm_opt.get("cache_dense", True)
        cache = getattr(self, "_densefrag", None)
        if cache is None or not self._key_current(cache.get("key")) or not keep:
            cache = self._densefrag = {"key": self._version_key()}
        if reduce_dim in cache:
            return cache[reduce_dim]
        pk_val, pk_pat = self.rowpack()
        O, K = lay.dense_shape[1 - reduce_dim], lay.dense_shape[reduce_dim]
        elems = ctypes.c_int64(0)
        native.check(lib.nmg_densefrag_elems(O, K, ctypes.byref(elems)))
        df = torch.empty((elems.value,), dtype=self.val.dtype, device=self.val.device)
        transpose = 1 if lay.group_dim == reduce_dim else 0   # rowpack lines run along the group dim
        with torch.cuda.device(df.device):
            native.check(lib.nmg_densefrag(
                native.ptr(pk_val), native.ptr(pk_pat), lay.G, lay.S, transpose, native.ptr(df),
                lay.n, lay.m, native.dtype_code(df.dtype), native.stream_ptr(df.device)))
        if keep:
            cache[reduce_dim] = df
        return df

    def dense_operand(self, reduce_dim, cached=False, pad_k=1):
        """Dense copy [outputs, reduction] of the weight (transposed when the reduction runs along
        dim 0), expanded from the rowpack operand into fresh scratch.  ``cached``: kept until
        ``val`` changes, like the densefrag operand (``spmm_opt["cache_dense"] = False`` turns
        that off).  ``pad_k``: the rows are padded with zeros to a multiple of it."""
        lay = self.layout
        keep = cached and self.spmm_opt.get("cache_dense", True)
        cache = getattr(self, "_dense_operand", None)
        if cache is None or not self._key_current(cache.get("key")):
            cache = self._dense_operand = {"key": self._version_key()}
        O, K = lay.dense_shape[1 - reduce_dim], lay.dense_shape[reduce_dim]
        Kp = -(-K // pad_k) * pad_k
        slot = reduce_dim if Kp == K else (reduce_dim, Kp)
        if keep and slot in cache:
            return cache[slot]
        pk_val, pk_pat = self.rowpack()
        alloc = torch.empty if Kp == K else torch.zeros
        out = alloc((O, Kp), dtype=self.val.dtype, device=self.val.device)
        # rowpack lines run along the group dim; the scratch has the reduction dim contiguous
        transpose = 1 if lay.group_dim == reduce_dim else 0
        with torch.cuda.device(out.device):
            native.check(native.load().nmg_rowpack_expand(
                native.ptr(pk_val), native.ptr(pk_pat), lay.G, lay.S, native.ptr(out), Kp, transpose,
                lay.n, lay.m, native.dtype_code(out.dtype), native.stream_ptr(out.device)))
        if keep:
            cache[slot] = out       # only an operand that was written is kept
        return out

    def lanepack8(self):
        """Operand of the streaming product on blocks of 8 along the reduction (1:8, 2:8, 4:8 with at
        most 16 tokens): the rowpack values and pattern bytes in the order in which the lanes of
        ``nmg_spmm_sstream`` take them; as large as the rowpack operand (0.625 bytes per dense weight
        at 2:8), kept until ``val`` changes."""
        lay = self.layout
        cached = getattr(self, "_lanepack8", None)
        if cached is not None and self._key_current(cached[0]):
            return cached[1], cached[2]
        pk_val, pk_pat = self.rowpack()
        lib = native.load()
        G, S = lay.G, lay.S
        ve, pb = ctypes.c_int64(), ctypes.c_int64()
        native.check(lib.nmg_lanepack8_sizes(G, S, lay.n, ctypes.byref(ve), ctypes.byref(pb)))
        lp_val = torch.empty(ve.value, dtype=self.val.dtype, device=self.val.device)
        lp_pat = torch.empty(pb.value, dtype=torch.uint8, device=self.val.device)
        with torch.cuda.device(lp_val.device):
            native.check(lib.nmg_lanepack8(native.ptr(pk_val), native.ptr(pk_pat), G, S, lay.n, native.ptr(lp_val),
                                           native.ptr(lp_pat), native.dtype_code(lp_val.dtype),
                                           native.stream_ptr(lp_val.device)))
        self._lanepack8 = (self._version_key(), lp_val, lp_pat)
        return lp_val, lp_pat

    def gpack(self):
        """Operand of the streaming product along the group dim (at most 16 tokens, m = 4 or 8 with
        n = 1 or 2): the rowpack operand in tiles of 32 lines x 256 outputs, each one contiguous
        run in the order in which the lanes of ``nmg_spmm_gstream`` take it, pattern numbers in 4
        bits where there are at most 16; kept until ``val`` changes."""
        lay = self.layout
        cached = getattr(self, "_gpack", None)
        if cached is not None and self._key_current(cached[0]):
            return cached[1]
        pk_val, pk_pat = self.rowpack()
        lib = native.load()
        nbytes = ctypes.c_int64()
        native.check(lib.nmg_gpack_bytes(lay.G, lay.S, lay.n, lay.m, ctypes.byref(nbytes)))
        gp = torch.empty(max(nbytes.value, 16), dtype=torch.uint8, device=self.val.device)
        with torch.cuda.device(gp.device):
            native.check(lib.nmg_gpack(native.ptr(pk_val), native.ptr(pk_pat), lay.G, lay.S, lay.n, lay.m,
                                       native.ptr(gp), native.dtype_code(self.val.dtype), native.stream_ptr(gp.device)))
        self._gpack = (self._version_key(), gp)
        return gp

    def opack(self):
        """Operand of ``nmg_spmm_ostream`` (a handful of tokens, 2:4, reduction along the group dim):
        the rowpack operand per span of 16 outputs and set of 256 lines in the order in which the
        lanes fetch it, pattern numbers in 4 bits; kept until ``val`` changes."""
        lay = self.layout
        cached = getattr(self, "_opack", None)
        if cached is not None and self._key_current(cached[0]):
            return cached[1]
        pk_val, pk_pat = self.rowpack()
        lib = native.load()
        nbytes = ctypes.c_int64()
        native.check(lib.nmg_opack_bytes(lay.G, lay.S, lay.n, lay.m, ctypes.byref(nbytes)))
        op = torch.empty(max(nbytes.value, 16), dtype=torch.uint8, device=self.val.device)
        with torch.cuda.device(op.device):
            native.check(lib.nmg_opack(native.ptr(pk_val), native.ptr(pk_pat), lay.G, lay.S, lay.n, lay.m,
                                       native.ptr(op), native.dtype_code(self.val.dtype), native.stream_ptr(op.device)))
        self._opack = (self._version_key(), op)
        return op

    def slotmap(self):
        """int16 [num_blocks, Gpad]: for every line of the (padded) group dim and block of the
        sparse dim, the slot that holds it -- the inverse of ``idx``.  Operand of the masked
        weight-gradient kernel; depends on the pattern only, cached until ``idx`` changes."""
        lay = self.layout
        if len(lay.dense_shape) != 2:
            raise native.NmgError("the slot map needs a 2-D grouped n:m tensor")
        cached = getattr(self, "_slotmap", None)
        if cached is not None and cached[0][0]() is self.idx and cached[0][1] == self.idx._version:
            return cached[1]
        key = (weakref.ref(self.idx), self.idx._version)
        native.require_gpu(self.idx)
        slot = torch.empty((lay.num_blocks, lay.num_chunks * lay.cols), dtype=torch.int16, device=self.idx.device)
        with torch.cuda.device(slot.device):
            native.check(native.load().nmg_slotmap(
                native.ptr(self.idx), lay.G, lay.S, native.ptr(slot), lay.n, lay.m, lay.group_size,
                native.stream_ptr(slot.device)))
        self._slotmap = (key, slot)
        return slot

    def masked_product(self, rows_op, cols_op, reduction_last=False):
        """New tensor with this tensor's pattern whose kept entries are those of
        ``rows_op^T @ cols_op`` (``rows_op`` [T, R], ``cols_op`` [T, C] for a weight [R, C]): the
        weight gradient of a linear layer, accumulated in fp32 and written straight into the
        ``val`` layout.  16-bit types; extents that are multiples of 8.
        ``reduction_last=True`` takes the operands transposed, ``rows_op`` [R, T] and ``cols_op``
        [C, T] (the product ``rows_op @ cols_op^T``, as the weight gradient of ``torch.mm(W, B)``
        finds them: grad_out and B); T must then be a multiple of 8, R and C may be anything."""
        lay = self.layout
        R, C = lay.dense_shape
        native.require_gpu(rows_op, cols_op, self.val)
        td, fd = (1, 0) if reduction_last else (0, 1)     # token dim / feature dim of the operands
        if rows_op.dim() != 2 or cols_op.dim() != 2 or rows_op.shape[td] != cols_op.shape[td] \
                or rows_op.shape[fd] != R or cols_op.shape[fd] != C:
            want = f"[{R}, T] and [{C}, T]" if reduction_last else f"[T, {R}] and [T, {C}]"
            raise native.NmgError(f"operands must be {want}, got {tuple(rows_op.shape)} and {tuple(cols_op.shape)}")
        dt = self.val.dtype
        if rows_op.dtype != dt or cols_op.dtype != dt:
            raise native.NmgError(f"dtype mismatch: operands {rows_op.dtype} / {cols_op.dtype}, weight {dt}")
        if rows_op.stride(1) != 1:
            rows_op = rows_op.contiguous()
        if cols_op.stride(1) != 1:
            cols_op = cols_op.contiguous()
        lines, pos = (rows_op, cols_op) if lay.group_dim == 0 else (cols_op, rows_op)
        val = torch.empty_like(self.val)
        T = rows_op.shape[td]
        if T == 0:
            val.zero_()
        else:
            slot = self.slotmap()
            entry = native.load().nmg_sddmm_nt if reduction_last else native.load().nmg_sddmm
            with torch.cuda.device(val.device):
                native.check(entry(
                    native.ptr(lines), lines.stride(0), native.ptr(pos), pos.stride(0), T, native.ptr(slot),
                    lay.G, lay.S, native.ptr(val), lay.n, lay.m, lay.group_size, native.dtype_code(dt),
                    native.stream_ptr(val.device)))
        out = GroupedNMTensor(val, self.idx, lay)
        out.spmm_opt = dict(self.spmm_opt)
        return out

    def masked_product_supported(self, rows_op, cols_op, reduction_last=False):
        lay = self.layout
        ok = (len(lay.dense_shape) == 2 and self.val.dtype in (torch.float16, torch.bfloat16)
              and rows_op.dtype == self.val.dtype and cols_op.dtype == self.val.dtype
              and all(t.stride(1) != 1 or (t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0)
                      for t in (rows_op, cols_op)))
        if reduction_last:
            return ok and rows_op.shape[1] % 8 == 0 and max(rows_op.stride(0), cols_op.stride(0)) < 2 ** 22
        return (ok and lay.dense_shape[0] % 8 == 0 and lay.dense_shape[1] % 8 == 0
                and max(rows_op.stride(0), cols_op.stride(0)) < 2 ** 25)

    def fragpack(self):
        """Operand of the sparse-matrix-core kernel (values + 2-bit positions in instruction
        register order); ``None`` when the n:m pattern does not fit 2-of-4 groups or the dtype is
        not 16-bit.  Cached until ``val`` changes."""
        self._pack()
        cached = getattr(self, "_fragpack", None)
        return None if cached is None else (cached[1], cached[2])

    def __repr__(self):
        lay = self.layout
        return (f"GroupedNMTensor(shape={tuple(lay.dense_shape)}, n:m:g={lay.n}:{lay.m}:{lay.group_size}, "
                f"sparse_dim={lay.sparse_dim}, group_dim={lay.group_dim}, dtype={self.val.dtype}, "
                f"device={self.val.device})")


OSTREAM_MAX_TOKENS = 4                # nmg_spmm_ostream: the token rows its lanes hold
OSTREAM_AUTO_TOKENS = 2               # ... and up to where it is ahead of the sliced kernel (4096 x 11008: 12.4 / 13.3 / 16.2 against 15.9 / 16.0 / 16.3 us at 1 / 2 / 3 tokens)
GSTREAM_MAX_TOKENS = 16               # nmg_spmm_gstream: tokens up to which the stream of the weight bounds the product
F32_GEMM_MAX_TOKENS = 65535 * 32      # one launch of the fp32 GEMM: token tiles of 32 in grid.y


def _mm_f32_expanded(weight, b, reduce_dim):
    """op(W) @ B in single precision with B and the result as they lie in memory: the dense copy of
    the weight (kept per weight version; the same one for both directions) as the row operand of
    the fp32 matrix-core GEMM, B as its reduction-major operand.  None when the route does not apply."""
    if (b.dtype != torch.float32 or b.shape[1] <= 16 or weight.spmm_opt.get("kernel", "auto") != "auto"
            or not weight.spmm_opt.get("expand", True) or b.shape[1] > F32_GEMM_MAX_TOKENS):
        return None
    lay = weight.layout
    K, O = lay.dense_shape[reduce_dim], lay.dense_shape[1 - reduce_dim]
    if b.stride(1) != 1:
        b = b.contiguous()
    N = b.shape[1]
    # the one dense copy [R, C]: row-major row operand of W @ B, reduction-major row operand of W^T @ B
    wd = weight.dense_operand(1, cached=True)
    entry = native.load().nmg_gemm_nn if reduce_dim == 1 else native.load().nmg_gemm_tn
    c = torch.empty((O, N), dtype=b.dtype, device=b.device)
    with torch.cuda.device(b.device):
        native.check(entry(
            native.ptr(b), b.stride(0) if K > 1 else N, native.ptr(wd), wd.stride(0), native.ptr(c), N, None, N, K, O,
            native.dtype_code(b.dtype), native.stream_ptr(b.device)))
    return c


def spmm_tt(weight, b):
    """C = W @ B for a 2-D ``GroupedNMTensor`` W [R, C] and a dense B [C, N] (``torch.mm``), without
    transposing copies when the sparse matrix cores can take it (16-bit, 2-of-4 compatible pattern
    along dim 1, C % 64 == 0, more than 16 columns, B row-contiguous with a row pitch that is a
    multiple of 8); otherwise through ``spmm`` on the transposed operands."""
    lay = weight.layout
    native.require_gpu(b, weight.val)
    R, C = lay.dense_shape
    if b.dim() != 2 or b.shape[0] != C:
        raise native.NmgError(f"B must be [{C}, N], got {tuple(b.shape)}")
    if b.dtype != weight.val.dtype:
        raise native.NmgError(f"dtype mismatch: B {b.dtype}, weight {weight.val.dtype}")
    N = b.shape[1]
    direct = (lay.sparse_dim == 1 and b.dtype in (torch.float16, torch.bfloat16) and C % 64 == 0 and N > 16
              and weight.spmm_opt.get("kernel", "auto") in ("auto", "smfmac"))
    if direct and b.stride(1) != 1:
        b = b.contiguous()
    if direct and (b.stride(0) % 8 != 0 or b.data_ptr() % 16 != 0):
        direct = False
    packed = weight.fragpack() if direct else None
    if packed is None:
        c = _mm_f32_expanded(weight, b, 1)
        if c is not None:
            return c
        return spmm(weight, b.t().contiguous(), reduce_dim=1).t()
    c = torch.empty((R, N), dtype=b.dtype, device=b.device)
    with torch.cuda.device(b.device):
        native.check(native.load().nmg_spmm_smfmac_tt(
            native.ptr(packed[0]), native.ptr(packed[1]), R, C, native.ptr(b), b.stride(0), native.ptr(c), N,
            None, N, native.dtype_code(b.dtype), native.stream_ptr(b.device)))
    return c


def spmm_tt_dense(weight, b, *, reduce_dim):
    """C = op(W) @ B with both dense operands as they lie in memory, on the dense matrix cores:
    ``reduce_dim=0``: B is [R, N], C = W^T @ B is [C, N] (the gradient with respect to B of
    ``torch.mm(W, B)``); ``reduce_dim=1``: B is [C, N], C = W @ B is [R, N].  Needs 16-bit data, a
    m that is a power of two or three times one, a reduction extent that is a multiple of 64, more than 16 columns and a B that is
    row-contiguous with a row pitch that is a multiple of 8; otherwise through ``spmm`` on the
    transposed operands."""
    lay = weight.layout
    native.require_gpu(b, weight.val)
    K, O = lay.dense_shape[reduce_dim], lay.dense_shape[1 - reduce_dim]
    if b.dim() != 2 or b.shape[0] != K:
        raise native.NmgError(f"B must be [{K}, N], got {tuple(b.shape)}")
    if b.dtype != weight.val.dtype:
        raise native.NmgError(f"dtype mismatch: B {b.dtype}, weight {weight.val.dtype}")
    N = b.shape[1]
    direct = (b.dtype in (torch.float16, torch.bfloat16) and K % 64 == 0 and N > 16
              and bool(native.load().nmg_densefrag_supported(lay.n, lay.m))
              and weight.spmm_opt.get("kernel", "auto") in ("auto", "densefrag")
              and weight.spmm_opt.get("expand", True))
    if direct and b.stride(1) != 1:
        b = b.contiguous()
    if direct and (b.stride(0) % 8 != 0 or b.data_ptr() % 16 != 0 or b.stride(0) >= 2 ** 24):
        direct = False
    if not direct:
        c = _mm_f32_expanded(weight, b, reduce_dim)
        if c is not None:
            return c
        return spmm(weight, b.t().contiguous(), reduce_dim=reduce_dim).t()
    df = weight.densefrag(reduce_dim)
    c = torch.empty((O, N), dtype=b.dtype, device=b.device)
    with torch.cuda.device(b.device):
        native.check(native.load().nmg_spmm_densefrag_tt(
            native.ptr(df), O, K, native.ptr(b), b.stride(0), native.ptr(c), N, None, N,
            native.dtype_code(b.dtype), native.stream_ptr(b.device)))
    return c


def spmm(weight, x, bias=None, *, reduce_dim, kernel=None):
    """Y = X @ op(W) for a 2-D ``GroupedNMTensor`` W of shape [R, C].

    ``reduce_dim=1``: X is [T, C], Y = X @ W^T is [T, R]  (F.linear forward).
    ``reduce_dim=0``: X is [T, R], Y = X @ W   is [T, C]  (gradient w.r.t. the input).
    """
    lay = weight.layout
    native.require_gpu(x, weight.val, bias)
    if x.dtype != weight.val.dtype:
        raise native.NmgError(f"dtype mismatch: activations {x.dtype}, weight {weight.val.dtype}")
    reduce_sparse = 1 if reduce_dim == lay.sparse_dim else 0
    K = lay.dense_shape[reduce_dim]
    O = lay.dense_shape[1 - reduce_dim]
    if x.dim() != 2 or x.shape[1] != K:
        raise native.NmgError(f"activations must be [tokens, {K}], got {tuple(x.shape)}")
    if x.stride(1) != 1:
        x = x.contiguous()
    T = x.shape[0]
    if T == 1 and x.stride(0) != K:
        x = x.as_strided((1, K), (K, 1))    # the stride of a dim of extent 1 means nothing; give it the plain one
    y = torch.empty((T, O), dtype=x.dtype, device=x.device)
    if bias is not None:
        bias = bias.to(dtype=x.dtype).contiguous()
    kname = kernel or weight.spmm_opt.get("kernel", "auto")
    variant = int(weight.spmm_opt.get("variant", -1))
    smf_ok = (reduce_sparse == 1 and K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
              and x.dtype in (torch.float16, torch.bfloat16))
    if kname == "skinny" and T > 16:
        raise native.NmgError("the skinny kernel serves at most 16 tokens")
    # Few tokens on blocks of 8 along the reduction (1:8, 2:8, 4:8): the rowpack operand holds 0.375 /
    # 0.625 / 1.125 bytes per dense weight where the operand of the sparse matrix cores holds 1.125
    # (and 4:8 has none): streamed once, expanded in registers, one kernel.
    if (kname in ("auto", "sstream") and reduce_sparse == 1 and T <= 16 and len(lay.dense_shape) == 2
            and x.dtype in (torch.float16, torch.bfloat16)
            and native.load().nmg_spmm_sstream_supported(lay.n, lay.m)
            and K % 256 == 0
            # weights of fewer than 3072 lines with more than 8 tokens: the operand of the sparse matrix
            # cores streams as fast or faster although it is larger (4:8 has none)
            and (kname == "sstream" or lay.n == 4 or O >= 96 * 32 or T <= 8)
            and (T == 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0
            and T * max(x.stride(0), K) * 2 < 2 ** 31 and 32 * (K // 8) * lay.n * 2 < 2 ** 31):
        lp_val, lp_pat = weight.lanepack8()
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_spmm_sstream(
                native.ptr(lp_val), native.ptr(lp_pat), O, K, native.ptr(x), x.stride(0) if T > 1 else K,
                native.ptr(y), O, native.ptr(bias), T, lay.n, lay.m, native.dtype_code(x.dtype),
                native.stream_ptr(x.device)))
        return y
    if kname == "sstream":
        raise native.NmgError("the streaming product along the sparse dim needs 16-bit data, at most 16 tokens, "
                              "1:8, 2:8 or 4:8 and a reduction extent that is a multiple of 256")
    packed = None
    if smf_ok and kname in ("auto", "skinny", "smfmac"):
        packed = weight.fragpack()
    if kname == "smfmac" and packed is None:
        raise native.NmgError(
            "the sparse-matrix-core kernel needs 16-bit data, a 2-of-4 compatible n:m "
            "pattern along the reduction dim and 16-byte aligned activations")
    if packed is not None:
        if T <= 16 and kname in ("auto", "skinny"):
            variant = 5                 # decode shapes: streaming kernel on the same operand
        elif (T <= 24 and kname == "auto" and variant == -1 and K % 128 == 0
              and T * x.stride(0) * 2 < 2 ** 31 and "slices" not in weight.spmm_opt):
            # 17 .. 24 tokens: the streaming kernel with the second half of its 32 token columns in
            # use is still ahead of the sliced reduction (4096 x 11008: 15.8 / 17.9 against 18.2 /
            # 18.7 us at 17 / 24 tokens; at 32 tokens 20.1 against 19.3)
            variant = 5
        lib = native.load()
        if T > 16 and variant == -1 and K % 64 == 0 and T * x.stride(0) * 2 < 2 ** 31:
            # few tiles for the chip: the reduction is cut into slices, summed by a second kernel
            slices, ws_bytes = ctypes.c_int(1), ctypes.c_int64(0)
            native.check(lib.nmg_splitk_plan(O, K, T, ctypes.byref(slices), ctypes.byref(ws_bytes)))
            slices = int(weight.spmm_opt.get("slices", slices.value))
            if slices > 1:
                tiles_m = (O + 255) // 256
                ws = torch.empty((slices * T * tiles_m * 256,), dtype=torch.float32, device=x.device)
                with torch.cuda.device(x.device):
                    native.check(lib.nmg_spmm_smfmac_splitk(
                        native.ptr(packed[0]), native.ptr(packed[1]), O, K, native.ptr(x), x.stride(0),
                        native.ptr(y), O, native.ptr(bias), T, native.dtype_code(x.dtype), slices,
                        native.ptr(ws), ws.numel() * 4, native.stream_ptr(x.device)))
                return y
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_spmm_smfmac(
                native.ptr(packed[0]), native.ptr(packed[1]), O, K, native.ptr(x),
                x.stride(0) if T > 1 else K, native.ptr(y), O, native.ptr(bias), T,
                native.dtype_code(x.dtype), variant, native.stream_ptr(x.device)))
        return y
    # Few tokens as well when the choice is automatic: without a sparse-core operand (another
    # pattern, the reduction along the group dim, fp32) the alternative for <= 16 tokens is the untuned
    # streaming kernel.  4096 x 11008 at 1 / 4 / 16 tokens: 4:8 25 / 25 / 26 us on the dense-core
    # operand with the reduction cut into slices against 63 / 119 / 342; 2:4 reduced along the
    # group dim (the reference's default orientation) 24 / 25 / 26 against 1190 / 1203 / 1286; fp32
    # 65 / 65 / 65 against 70 / 134 / 361.
    min_t = 1 if kname == "auto" else 17
    ldx = x.stride(0) if T > 1 else K      # the stride of a dim of extent 1 means nothing
    # Few tokens with the reduction along the group dim (what F.linear does with a weight in the
    # reference's default orientation): the compressed lines are streamed once and expanded in
    # registers -- 51 MB instead of the 90 MB of the dense-core operand for 4096 x 11008 at 2:4.
    # ... and with a handful of tokens at 2:4 every workgroup owns 16 outputs over the whole
    # reduction: one kernel, no sums through memory (the token rows are then read by every
    # workgroup, which is why this is for few of them)
    if (kname in ("auto", "ostream") and reduce_sparse == 0 and T <= (OSTREAM_AUTO_TOKENS if kname == "auto" else OSTREAM_MAX_TOKENS)
            and x.dtype in (torch.float16, torch.bfloat16) and len(lay.dense_shape) == 2
            and native.load().nmg_spmm_ostream_supported(lay.n, lay.m)
            and K % 8 == 0 and ldx % 8 == 0 and x.data_ptr() % 16 == 0 and T * ldx * 2 < 2 ** 31):
        op = weight.opack()
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_spmm_ostream(
                native.ptr(op), K, O, native.ptr(x), ldx, native.ptr(y), O, native.ptr(bias), T, lay.n, lay.m,
                native.dtype_code(x.dtype), native.stream_ptr(x.device)))
        return y
    if kname == "ostream":
        raise native.NmgError("the product with 16 outputs per workgroup needs 16-bit data, 2:4, the reduction along "
                              f"the group dim, at most {OSTREAM_MAX_TOKENS} tokens and a reduction extent that is a multiple of 8")
    if (kname in ("auto", "gstream") and reduce_sparse == 0 and T <= GSTREAM_MAX_TOKENS
            and x.dtype in (torch.float16, torch.bfloat16) and len(lay.dense_shape) == 2
            and native.load().nmg_spmm_gstream_supported(lay.n, lay.m)
            and K % 8 == 0 and ldx % 8 == 0 and x.data_ptr() % 16 == 0 and T * ldx * 2 < 2 ** 31):
        lib = native.load()
        gp = weight.gpack()
        slices, ws_bytes = ctypes.c_int(1), ctypes.c_int64(0)
        native.check(lib.nmg_spmm_gstream_plan(K, O, T, lay.n, lay.m, ctypes.byref(slices), ctypes.byref(ws_bytes)))
        ws = torch.empty((max(ws_bytes.value, 4) // 4,), dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            native.check(lib.nmg_spmm_gstream(
                native.ptr(gp), K, O, native.ptr(x), ldx, native.ptr(y), O,
                native.ptr(bias), T, lay.n, lay.m, native.dtype_code(x.dtype), native.ptr(ws), ws.numel() * 4,
                native.stream_ptr(x.device)))
        return y
    if kname == "gstream":
        raise native.NmgError("the streaming product along the group dim needs 16-bit data, at most "
                              f"{GSTREAM_MAX_TOKENS} tokens, m = 4 or 8 with n = 1 or 2 and a reduction extent that is a multiple of 8")
    dense16 = (T >= min_t and x.dtype in (torch.float16, torch.bfloat16) and K % 64 == 0
               and ldx % 8 == 0 and x.data_ptr() % 16 == 0 and T * ldx * 2 < 2 ** 31)
    if (kname in ("auto", "mfma", "densefrag") and dense16
            and native.load().nmg_densefrag_supported(lay.n, lay.m)
            and (kname == "densefrag" or weight.spmm_opt.get("expand", True))):
        # "expand, then multiply": one HBM-bound pass writes the weight in the register order of
        # the dense matrix cores into scratch, the pipelined kernel multiplies from there
        df = weight.densefrag(reduce_dim)
        lib = native.load()
        slices, ws_bytes = ctypes.c_int(1), ctypes.c_int64(0)
        if int(weight.spmm_opt.get("dense_variant", -1)) == -1:
            # (the plan leaves 16 tokens and fewer to the streaming kernel of the sparse-core operand;
            # here they are cut like 17)
            native.check(lib.nmg_splitk_plan(O, K, max(T, 17), ctypes.byref(slices), ctypes.byref(ws_bytes)))
        slices = int(weight.spmm_opt.get("slices", slices.value))
        if slices > 1:
            # few tiles for the chip: the reduction is cut into slices, summed by a second kernel
            ws = torch.empty((slices * T * ((O + 255) // 256) * 256,), dtype=torch.float32, device=x.device)
            with torch.cuda.device(x.device):
                native.check(lib.nmg_spmm_densefrag_splitk(
                    native.ptr(df), O, K, native.ptr(x), ldx, native.ptr(y), O, native.ptr(bias), T,
                    native.dtype_code(x.dtype), slices, native.ptr(ws), ws.numel() * 4,
                    native.stream_ptr(x.device)))
            return y
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_spmm_densefrag(
                native.ptr(df), O, K, native.ptr(x), ldx, native.ptr(y), O, native.ptr(bias), T,
                native.dtype_code(x.dtype), int(weight.spmm_opt.get("dense_variant", -1)),
                native.stream_ptr(x.device)))
        return y
    if kname == "densefrag":
        raise native.NmgError("the densefrag route needs 16-bit data, more than 16 tokens, an m that is a power of two or three times one "
                              "and a reduction extent that is a multiple of 64")
    if kname == "expand":
        if not (dense16 and O * K * 2 < 2 ** 31):
            raise native.NmgError("the expand-then-multiply route needs 16-bit data, more than 16 tokens "
                                  "and a reduction extent that is a multiple of 64")
        # the same idea with a plain row-major dense copy of the weight
        a = weight.dense_operand(reduce_dim)
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_gemm_nt(
                native.ptr(a), K, native.ptr(x), ldx, native.ptr(y), O, native.ptr(bias),
                O, K, T, native.dtype_code(x.dtype), native.stream_ptr(x.device)))
        return y
    if (x.dtype == torch.float32 and T >= min_t and kname == "auto" and len(lay.dense_shape) == 2
            and weight.spmm_opt.get("expand", True) and T <= F32_GEMM_MAX_TOKENS):
        # single precision: "expand, then multiply" as well -- a dense copy of the weight (kept per
        # weight version) and the pipelined fp32 matrix-core kernel; the kernel below, which expands
        # inside its reduction loop, runs at a tenth of that rate
        # One dense copy [R, C] serves both directions: row-major operand of the product that
        # reduces along dim 1, reduction-major operand of the one that reduces along dim 0.
        a = weight.dense_operand(1, cached=True)
        entry = native.load().nmg_gemm_nt if reduce_dim == 1 else native.load().nmg_gemm_nn
        with torch.cuda.device(x.device):
            native.check(entry(
                native.ptr(a), a.stride(0), native.ptr(x), ldx, native.ptr(y), O, native.ptr(bias),
                O, K, T, native.dtype_code(x.dtype), native.stream_ptr(x.device)))
        return y
    Kp = -(-K // 64) * 64
    if (x.dtype in (torch.float16, torch.bfloat16) and T >= (4 if reduce_sparse == 1 else 1) and kname == "auto"
            and len(lay.dense_shape) == 2
            and weight.spmm_opt.get("expand", True) and O * Kp * 2 < 2 ** 31 and T * Kp * 2 < 2 ** 31):
        # 16-bit shapes that none of the matrix-core routes above takes as they are (a reduction
        # extent that is not a multiple of 64 or 8, an m such as 5 or 7, unaligned activations):
        # a dense copy of the weight with zero-padded rows (kept per weight version) and, where
        # needed, a zero-padded copy of the activations, through the dense 16-bit GEMM -- the
        # kernel below runs at a hundredth of its rate (from 4 tokens on where the reduction runs
        # along the sparse dim: this GEMM does not cut its reduction, and at 1 token the streaming kernel
        # below is ahead, 81 us against 132; along the group dim that kernel takes 470 us at 4096^2)
        a = weight.dense_operand(reduce_dim, cached=True, pad_k=64)
        if Kp != K or ldx % 8 != 0 or x.data_ptr() % 16 != 0 or T * ldx * 2 >= 2 ** 31:
            xp = x.new_zeros((T, Kp))
            xp[:, :K] = x
        else:
            xp = x
        with torch.cuda.device(x.device):
            native.check(native.load().nmg_gemm_nt(
                native.ptr(a), Kp, native.ptr(xp), xp.stride(0) if T > 1 else Kp, native.ptr(y), O, native.ptr(bias),
                O, Kp, T, native.dtype_code(x.dtype), native.stream_ptr(x.device)))
        return y
    pk_val, pk_pat = weight.rowpack()
    with torch.cuda.device(x.device):
        native.check(native.load().nmg_spmm(
            native.ptr(pk_val), native.ptr(pk_pat), lay.G, lay.S, native.ptr(x),
            x.stride(0) if T > 1 else K, native.ptr(y), O, native.ptr(bias), T, reduce_sparse,
            lay.n, lay.m, native.dtype_code(x.dtype), native.KERNELS[kname],
            native.stream_ptr(x.device)))
    return y
