"""CPU plumbing case: fp32 C = A.B with M=N=K=512, K split into 8 shards of 64;
each shard's partial is computed separately and the 8 partials are summed with
the all-reduce semantics of the atomics and one-shot paths (oracle only)."""

import torch

from oracle import iris_oracle as O


def test_eight_k_shards_sum_to_the_full_product():
    g = torch.Generator().manual_seed(123)
    A = torch.randn(512, 512, generator=g)
    B = torch.randn(512, 512, generator=g)
    shards = O.k_shards(A, B, 8)
    assert len(shards) == 8 and all(a.shape == (512, 64) and b.shape == (64, 512) for a, b in shards)
    full = A @ B
    by_atomics = O.atomics_all_reduce(shards)
    by_one_shot = O.one_shot_all_reduce(shards, torch.float32, torch.float32)
    assert torch.allclose(by_atomics, full, rtol=1e-4, atol=1e-3)
    assert torch.equal(by_atomics, by_one_shot)  # same partials, same rank order
    assert torch.allclose(by_one_shot.double(), A.double() @ B.double(), rtol=1e-4, atol=1e-3)
    # flags of the exchange: 8 ranks x (512/256)^2 tiles
    fm = O.FlagModel(8, 4)
    for r in range(8):
        for t in range(4):
            fm.signal(r, t)
    assert all(fm.try_consume(r, t) for r in range(8) for t in range(4)) and (fm.flags == 0).all()
