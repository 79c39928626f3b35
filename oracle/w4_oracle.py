"""CPU restatement (numpy) of the 2:4 + int4 format of sten_amd/csrc/nmg_w4.hip.  Test
infrastructure only: tests/ and __graft_entry__.smoke() may import it, the product may not.

Parity unpinned against the reference: its test for this configuration calls an external
library (marlin.mul_2_4, tests/test_sparse_marlin.py:113) on random operands with zero scales
and asserts nothing, and the packing tables of that library are not in the reference tree.  What
is checked is this library against this restatement (bit-exact packing) and the product against
the dequantised dense matmul.
"""
import numpy as np


def prune_quantise(w):
    """w fp16 [M, K], K % 128 == 0 -> (pos [M, K/4, 2] uint8, q [M, K/4, 2] uint8, s [M, K/128] fp16)."""
    M, K = w.shape
    a = w.astype(np.float32).reshape(M, K // 4, 4)
    order = np.argsort(-np.abs(a), axis=2, kind="stable")[:, :, :2]     # largest first, lower position on ties
    pos = np.sort(order, axis=2).astype(np.uint8)
    kept = np.take_along_axis(a, pos.astype(np.int64), axis=2)           # [M, K/4, 2]
    amax = np.abs(kept).reshape(M, K // 128, 64).max(axis=2)
    s = (amax / np.float32(7.0)).astype(np.float16)
    s[s == 0] = np.float16(1.0)
    sf = np.repeat(s.astype(np.float32), 32, axis=1).reshape(M, K // 4, 1)
    q = np.clip(np.rint(kept / sf) + 8.0, 0, 15).astype(np.uint8)
    return pos, q, s


def dequantise(pos, q, s, K):
    M = q.shape[0]
    sf = np.repeat(s, 32, axis=1).reshape(M, K // 4, 1)
    vals = ((q.astype(np.float16) - np.float16(8)) * sf).astype(np.float16)   # one rounding, in fp16
    dense = np.zeros((M, K // 4, 4), dtype=np.float16)
    np.put_along_axis(dense, pos.astype(np.int64), vals, axis=2)
    return dense.reshape(M, K)


def pack(pos, q, s, M, K):
    """The three arrays in the library's layout: B uint8 [MB*KQ*64*16], meta uint32 [MB*KQ*64*2],
    scales fp16 [MB*KQ*32]."""
    MB, KQ = (M + 31) // 32, K // 128
    words = np.zeros((MB, KQ, 64, 4), dtype=np.uint32)
    meta = np.zeros((MB, KQ, 64, 2), dtype=np.uint32)
    sc = np.ones((MB, KQ, 32), dtype=np.float16)
    # padding rows: nibble 8 everywhere, positions (0, 1)
    qp = np.full((MB * 32, K // 4, 2), 8, dtype=np.uint32)
    pp = np.zeros((MB * 32, K // 4, 2), dtype=np.uint32)
    pp[:, :, 1] = 1
    qp[:M] = q
    pp[:M] = pos
    sp = np.zeros((MB * 32, KQ), dtype=np.float16)
    sp[:M] = s
    rows = np.arange(MB * 32)
    mb, r = rows // 32, rows % 32
    for g4 in range(K // 4):
        kq, gq = g4 // 32, g4 % 32
        ins, kg = gq // 8, gq % 8
        ga = (kg >> 1) & 1
        qq = ((kg >> 2) << 1) | (kg & 1)
        lane = r + 32 * ga
        for i in range(2):
            e = 2 * qq + i
            words[mb, kq, lane, ins] |= qp[:, g4, i] << np.uint32(4 * (e >> 1) + 16 * (e & 1))
        code = pp[:, g4, 0] | (pp[:, g4, 1] << np.uint32(2))
        meta[mb, kq, lane, ins >> 1] |= code << np.uint32(4 * qq + 16 * (ins & 1))
    for kq in range(KQ):
        sc[mb, kq, r] = sp[:, kq]
    # scales of padding rows: the kernel computes max 0 -> scale 1
    pad = rows >= M
    for kq in range(KQ):
        sc[mb[pad], kq, r[pad]] = np.float16(1.0)
    return words.reshape(-1).view(np.uint8), meta.reshape(-1), sc.reshape(-1)


def linear(w_deq, x, bias=None):
    y = x.astype(np.float64) @ w_deq.astype(np.float64).T
    if bias is not None:
        y = y + bias.astype(np.float64)
    return y
