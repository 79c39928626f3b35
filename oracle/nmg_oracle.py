"""CPU oracle for the grouped n:m (nmg) path -- numpy + the C restatement in nmg_oracle.c.

TEST INFRASTRUCTURE ONLY.  Nothing under ``sten_amd/`` may import this module; it is the
checker used by ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``.

Reference lines restated here (paths relative to the reference repository root):

* ``merge`` / ``unmerge``     src/sten/grouped_nm/grouped_nm_tensor.py:71-217 (compute_nm_strides),
                              :688-710 (pad_to, dense_to_grouped_n_m), :848-874 (grouped_n_m_to_dense)
* ``sparsify``                :636-685 driver + :255-297 kernel (through nmg_oracle.c)
* ``to_dense``                :742-757 (through nmg_oracle.c)
* ``spmm`` / ``simd_spmm``    src/sten/grouped_nm/dace_gnm_mult.py:141-256, :724-805
* ``linear``                  src/sten/grouped_nm/sten_impls.py:143-174 with the operand
                              transposition stated explicitly (the `trans_b` override at :53 is
                              a defect of the reference and is not restated)

fp16 inputs: the reference sparsifier accepts fp32/fp64 only (grouped_nm_tensor.py:242).  The
parity definition for fp16 is upcast to fp32 -> algorithm -> downcast, which is exact because
selection only copies values.
"""
import ctypes
import math
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")


def build(force=False):
    """Compile nmg_oracle.c / nmg_cpu_simd.cpp with the Makefile next to this file."""
    need = force or not all(
        os.path.exists(os.path.join(_BUILD, f))
        for f in ("libnmg_oracle.so", "libnmg_simd_avx512.so", "libnmg_simd_avx2.so")
    )
    if need:
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)


_lib = None
_simd = None

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_I = ctypes.c_int


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(os.path.join(_BUILD, "libnmg_oracle.so"))
        _lib.nmg_ref_chunk.restype = _I64
        _lib.nmg_ref_chunk.argtypes = [_I, _I]
        _lib.nmg_ref_order.restype = _I64
        _lib.nmg_ref_order.argtypes = [_I, _I, _P]
        for name in ("nmg_ref_sparsify_f32", "nmg_ref_sparsify_f64", "nmg_ref_to_dense_f32",
                     "nmg_ref_to_dense_f64", "nmg_ref_gather_f32"):
            f = getattr(_lib, name)
            f.restype = _I
            f.argtypes = [_P, _P, _P, _I64, _I, _I, _I]
        _lib.nmg_ref_spmm_f32.restype = _I
        _lib.nmg_ref_spmm_f32.argtypes = [_P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _I, _I, _I]
    return _lib


def cpu_flags():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def simd():
    """AVX-512 build if the host has avx512f else AVX2 (rule of grouped_nm_tensor.py:893-897)."""
    global _simd
    if _simd is None:
        build()
        kind = "avx512" if "avx512f" in cpu_flags() else "avx2"
        _simd = ctypes.CDLL(os.path.join(_BUILD, f"libnmg_simd_{kind}.so"))
        _simd.nmg_simd_kernel_name.restype = ctypes.c_char_p
        _simd.nmg_simd_slab.restype = _I
        _simd.nmg_simd_threads.restype = _I
        _simd.nmg_simd_spmm_f32.restype = _I
        _simd.nmg_simd_spmm_f32.argtypes = [_P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _I, _I, _I]
    return _simd


def _ptr(a):
    return a.ctypes.data_as(_P)


def chunk(n, m):
    return math.comb(m, n)


def order(n, m):
    """Pattern table of make_n_m(n, m) as an int8 array [C(m,n), n]."""
    c = chunk(n, m)
    out = np.zeros((c, max(n, 1)), dtype=np.int8)
    got = lib().nmg_ref_order(n, m, _ptr(out))
    assert got == c
    return out[:, :n]


@dataclass(frozen=True)
class Layout:
    """Geometry of one nmg tensor: what compute_nm_strides returns, reduced to what is used."""
    dense_shape: tuple
    n: int
    m: int
    g: int
    sparse_dim: int
    group_dim: int

    @property
    def c(self):
        return chunk(self.n, self.m)

    @property
    def num_blocks(self):
        return -(-self.dense_shape[self.sparse_dim] // self.m)

    @property
    def num_chunks(self):
        return -(-self.dense_shape[self.group_dim] // (self.c * self.g))

    @property
    def padded_shape(self):
        s = list(self.dense_shape)
        s[self.sparse_dim] = self.num_blocks * self.m
        s[self.group_dim] = self.num_chunks * self.c * self.g
        return tuple(s)

    @property
    def other_dims(self):
        return [d for d in range(len(self.dense_shape)) if d not in (self.sparse_dim, self.group_dim)]

    @property
    def outer(self):
        o = self.num_chunks * self.num_blocks
        for d in self.other_dims:
            o *= self.dense_shape[d]
        return o


def merge(x, lay):
    """dense N-D array -> contiguous [outer, c, g, m] (zero padded).

    Tile index = (other dims..., group-dim chunk, sparse-dim block), chunk slower than block;
    inside a tile element (col, r) with col = pattern-major position c*g and r in [0, m)."""
    assert tuple(x.shape) == tuple(lay.dense_shape)
    pad = [(0, p - s) for s, p in zip(x.shape, lay.padded_shape)]
    xp = np.pad(x, pad)
    others = lay.other_dims
    xp = np.transpose(xp, others + [lay.group_dim, lay.sparse_dim])
    lead = xp.shape[:-2]
    xp = xp.reshape(*lead, lay.num_chunks, lay.c * lay.g, lay.num_blocks, lay.m)
    nd = xp.ndim
    xp = np.transpose(xp, list(range(nd - 4)) + [nd - 4, nd - 2, nd - 3, nd - 1])
    return np.ascontiguousarray(xp.reshape(-1, lay.c, lay.g, lay.m))


def unmerge(merged, lay):
    """Inverse of merge (drops the padding)."""
    others = lay.other_dims
    lead = [lay.dense_shape[d] for d in others]
    x = merged.reshape(*lead, lay.num_chunks, lay.num_blocks, lay.c * lay.g, lay.m)
    nd = x.ndim
    x = np.transpose(x, list(range(nd - 4)) + [nd - 4, nd - 2, nd - 3, nd - 1])
    x = x.reshape(*lead, lay.num_chunks * lay.c * lay.g, lay.num_blocks * lay.m)
    perm = others + [lay.group_dim, lay.sparse_dim]
    inv = np.argsort(perm)
    x = np.transpose(x, inv)
    sl = tuple(slice(0, s) for s in lay.dense_shape)
    return np.ascontiguousarray(x[sl])


def sparsify_merged(merged, n):
    """[outer,c,g,m] -> (val [outer,c,g,n], idx [outer,c,g,1] int16)."""
    outer, c, g, m = merged.shape
    assert c == chunk(n, m)
    src_dtype = merged.dtype
    work = np.float64 if src_dtype == np.float64 else np.float32
    d = np.ascontiguousarray(merged.astype(work))
    val = np.zeros((outer, c, g, n), dtype=work)
    idx = np.full((outer, c, g, 1), -1, dtype=np.int16)
    fn = lib().nmg_ref_sparsify_f64 if work == np.float64 else lib().nmg_ref_sparsify_f32
    rc = fn(_ptr(d), _ptr(val), _ptr(idx), outer, n, m, g)
    if rc != 0:
        raise ValueError("chunk_size * group_size must be < 2**15")
    return val.astype(src_dtype), idx


def sparsify(x, n, m, sparse_dim, g, group_dim):
    lay = Layout(tuple(x.shape), n, m, g, sparse_dim, group_dim)
    val, idx = sparsify_merged(merge(x, lay), n)
    return val, idx, lay


def to_dense_merged(val, idx, m):
    outer, c, g, n = val.shape
    src_dtype = val.dtype
    work = np.float64 if src_dtype == np.float64 else np.float32
    v = np.ascontiguousarray(val.astype(work))
    i = np.ascontiguousarray(idx.reshape(outer, c, g).astype(np.int16))
    dense = np.zeros((outer, c, g, m), dtype=work)
    fn = lib().nmg_ref_to_dense_f64 if work == np.float64 else lib().nmg_ref_to_dense_f32
    fn(_ptr(v), _ptr(i), _ptr(dense), outer, n, m, g)
    return dense.astype(src_dtype)


def to_dense(val, idx, lay):
    return unmerge(to_dense_merged(val, idx, lay.m), lay)


def gather_merged(merged, idx, n):
    """Re-compress a dense tile tensor with an existing pattern (same idx)."""
    outer, c, g, m = merged.shape
    d = np.ascontiguousarray(merged.astype(np.float32))
    i = np.ascontiguousarray(idx.reshape(outer, c, g).astype(np.int16))
    val = np.zeros((outer, c, g, n), dtype=np.float32)
    lib().nmg_ref_gather_f32(_ptr(d), _ptr(i), _ptr(val), outer, n, m, g)
    return val.astype(merged.dtype)


def _spmm_common(fn, val, idx, lay, B):
    """C[M, N] = to_dense(A) @ B for a 2-D A in the reference orientation
    (n:m blocks along dim 0, groups along dim 1 -- dace_gnm_mult.py:615-616)."""
    assert len(lay.dense_shape) == 2 and lay.sparse_dim == 0 and lay.group_dim == 1
    M, K = lay.dense_shape
    Kb, N = B.shape
    assert Kb == K
    v = np.ascontiguousarray(val.astype(np.float32))
    i = np.ascontiguousarray(idx.reshape(-1).astype(np.int16))
    Bc = np.ascontiguousarray(B.astype(np.float32))
    Mpad = lay.num_blocks * lay.m
    C = np.empty((Mpad, N), dtype=np.float32)
    rc = fn(_ptr(v), _ptr(i), _ptr(Bc), N, _ptr(C), N, M, K, N, lay.n, lay.m, lay.g)
    if rc != 0:
        raise ValueError(f"nmg spmm rejected the shape (code {rc})")
    return C[:M]


def spmm(val, idx, lay, B):
    return _spmm_common(lib().nmg_ref_spmm_f32, val, idx, lay, B)


def simd_spmm(val, idx, lay, B):
    return _spmm_common(simd().nmg_simd_spmm_f32, val, idx, lay, B)


def simd_info():
    s = simd()
    return {"kernel": s.nmg_simd_kernel_name().decode(), "slab": s.nmg_simd_slab(),
            "threads": s.nmg_simd_threads()}


def linear(x, val, idx, lay, bias=None):
    """y[..., :M] = x @ to_dense(W)^T (+ bias) -- sten_impls.py:143-174 with B = x2d^T."""
    M, K = lay.dense_shape
    x2 = x.reshape(-1, K)
    y = spmm(val, idx, lay, np.ascontiguousarray(x2.T)).T
    y = y.reshape(*x.shape[:-1], M)
    if bias is not None:
        y = y + bias
    return y


def perfect_nm(x, n, m, sparse_dim):
    """Ungrouped n:m, restating PerfectNMTensor.from_dense (grouped_nm_tensor.py:1018-1046): pad the
    sparse dim to a multiple of m, split it into (blocks, m), sort the magnitudes of a block in
    descending order and keep the first n.  Returns (val, idx) with the sparse dim replaced by
    (blocks, n).  The reference's argsort is unstable, so it leaves the order of equal magnitudes
    open; here equal magnitudes keep the lower position first (a stable sort) and NaN sorts first."""
    sparse_dim %= x.ndim
    S = x.shape[sparse_dim]
    blocks = -(-S // m)
    pad = [(0, 0)] * x.ndim
    pad[sparse_dim] = (0, blocks * m - S)
    y = np.moveaxis(np.pad(x, pad), sparse_dim, -1)
    y = y.reshape(*y.shape[:-1], blocks, m)
    mag = np.abs(y.astype(np.float64))
    mag = np.where(np.isnan(mag), np.inf, mag)
    order = np.argsort(-mag, axis=-1, kind="stable")[..., :n]
    val = np.take_along_axis(y, order, axis=-1)
    nd = val.ndim
    perm = list(range(sparse_dim)) + [nd - 2, nd - 1] + list(range(sparse_dim, nd - 2))
    return np.ascontiguousarray(np.transpose(val, perm)), np.ascontiguousarray(np.transpose(order, perm)).astype(np.int64)


def perfect_nm_to_dense(val, idx, m, sparse_dim, size):
    """Inverse scatter (grouped_nm_tensor.py:1048-1065)."""
    full = list(val.shape)
    full[sparse_dim + 1] = m
    dense = np.zeros(full, dtype=val.dtype)
    np.put_along_axis(dense, idx, val, axis=sparse_dim + 1)
    merged = full[:sparse_dim] + [full[sparse_dim] * m] + full[sparse_dim + 2:]
    dense = dense.reshape(merged)
    sl = [slice(None)] * dense.ndim
    sl[sparse_dim] = slice(0, size)
    return np.ascontiguousarray(dense[tuple(sl)])
