"""Shared helpers of the GPU parity tests."""

import torch


def make_topk_ids(T, K, E, *, gen, allow_dupe=False, invalid_frac=0.0, dtype=torch.int64):
    """Random expert ids in the style of the reference's GPU tests
    (tests/test_moe_utils_gpu.py:14-33): optional duplicates inside a token and a
    fraction of unused (-1) slots."""
    ids = torch.randint(0, E, (T, K), generator=gen, dtype=torch.int64)
    if K > 1 and not allow_dupe:
        for i in range(1, K):
            clash = ids[:, i] == ids[:, 0]
            ids[clash, i] = (ids[clash, i] + i) % E
    if invalid_frac > 0:
        ids = ids.masked_fill(torch.rand(T, K, generator=gen) < invalid_frac, -1)
    return ids.to(dtype)


def rel_l2(got: torch.Tensor, ref: torch.Tensor) -> float:
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    denom = float(ref.norm())
    return float((got - ref).norm()) / (denom if denom > 0 else 1.0)
