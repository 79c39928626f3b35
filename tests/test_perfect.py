"""PerfectNMTensor (ungrouped n:m, plain torch): host logic, runs on the CPU."""
import itertools

import torch

from sten_amd.perfect import PerfectNMTensor, is_correct_nm


def test_round_trip_and_block_structure():
    torch.manual_seed(0)
    for shape in [(3, 17, 5), (8, 8), (1, 13)]:
        x = torch.randn(*shape)
        for sd in range(len(shape)):
            for n, m in [(2, 4), (1, 8), (5, 12)]:
                p = PerfectNMTensor.from_dense(x, n, m, sd)
                d = p.to_dense()
                assert d.shape == x.shape == p.shape
                assert is_correct_nm(x, d, sd, n, m)
                # each block keeps exactly its n largest magnitudes (padding counts as zeros)
                xs = x.movedim(sd, -1)
                pad = (-xs.shape[-1]) % m
                blocks = torch.nn.functional.pad(xs, (0, pad)).reshape(*xs.shape[:-1], -1, m).abs()
                best = blocks.topk(n, dim=-1).values.sum()
                assert torch.isclose(d.abs().sum(), best)


def test_is_correct_nm_rejects_violations():
    x = torch.arange(1.0, 9.0).reshape(2, 4)
    assert is_correct_nm(x, x * torch.tensor([1.0, 1.0, 0.0, 0.0]), 1, 2, 4)
    assert not is_correct_nm(x, x, 1, 2, 4)                                   # 4 kept in a block of 4
    assert not is_correct_nm(x, torch.full_like(x, 0.5), 1, 2, 4)             # values changed
