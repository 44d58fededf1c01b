"""TE-style permutation helpers on the GPU against the oracle and the reference's own cases
(reference tests/test_permute_utils.py:31-161)."""

import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def P():
    from steptronoss_amd.model.utils import permute_utils

    return permute_utils


TOKENS = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]])
MASK = torch.tensor([[1, 0, 1, 0], [0, 1, 0, 0], [1, 0, 0, 1]], dtype=torch.bool)
MASK_PROBS = torch.tensor([[0.6, 0.0, 0.4, 0.0], [0.0, 1.0, 0.0, 0.0], [0.5, 0.0, 0.0, 0.5]])


def _expected_mask_order(mask):
    T, E = mask.shape
    tok, rid = [], []
    for e in range(E):
        for t in range(T):
            if mask[t, e]:
                tok.append(t)
                rid.append(e * T + t)
    return torch.tensor(tok), torch.tensor(rid)


def test_mask_roundtrip_reference_case(P):
    out, pp, rid = P.moe_permute_with_probs(TOKENS.to(DEV), MASK_PROBS.to(DEV), MASK.to(DEV))
    tok, exp_rid = _expected_mask_order(MASK)
    assert rid.dtype == torch.int64 and torch.equal(rid.cpu(), exp_rid)
    assert torch.equal(out.cpu(), TOKENS[tok])
    assert torch.equal(pp.cpu(), MASK_PROBS.T.reshape(-1)[exp_rid])
    back = P.moe_unpermute(out, rid, merging_probs=MASK_PROBS.to(DEV), restore_shape=TOKENS.shape, map_type="mask")
    assert torch.allclose(back.cpu(), TOKENS)


def test_mask_padding_reference_case(P):
    tok, _ = _expected_mask_order(MASK)
    n_out = tok.numel() + 2
    out, rid = P.moe_permute(TOKENS.to(DEV), MASK.to(DEV), num_out_tokens=n_out, map_type="mask")
    assert out.shape[0] == n_out
    assert torch.equal(rid[-2:].cpu(), torch.tensor([-1, -1]))
    assert float(out[-2:].abs().sum()) == 0.0
    back = P.moe_unpermute(out, rid, merging_probs=MASK_PROBS.to(DEV), restore_shape=TOKENS.shape, map_type="mask")
    assert torch.allclose(back.cpu(), TOKENS)
    # trimmed instead of padded
    out, rid = P.moe_permute(TOKENS.to(DEV), MASK.to(DEV), num_out_tokens=3, map_type="mask")
    assert out.shape[0] == 3 and torch.equal(out.cpu(), TOKENS[tok[:3]])


def test_index_roundtrip_reference_case(P):
    rm = torch.tensor([[1, 0], [0, 2], [2, -1]], dtype=torch.int64)
    probs = torch.tensor([[0.6, 0.4], [0.5, 0.5], [1.0, 0.0]])
    out, rid = P.moe_permute(TOKENS.to(DEV), rm.to(DEV), map_type="index")
    flat = rm.reshape(-1)
    flat_pos = torch.arange(flat.numel())
    valid = flat >= 0
    order = torch.argsort(flat[valid] * flat.numel() + flat_pos[valid])
    exp_rid = flat_pos[valid][order]
    assert torch.equal(rid.cpu(), exp_rid)
    assert torch.equal(out.cpu(), TOKENS[exp_rid // 2])
    back = P.moe_unpermute(out, rid, merging_probs=probs.to(DEV), restore_shape=TOKENS.shape, map_type="index")
    assert torch.allclose(back.cpu(), TOKENS)


def test_sort_chunks_reference_cases(P):
    inp = torch.arange(12, dtype=torch.float32).view(6, 2)
    probs = torch.arange(6, dtype=torch.float32)
    sizes = torch.tensor([2, 1, 3])
    order = torch.tensor([2, 0, 1])
    exp = torch.cat([inp[3:6], inp[0:2], inp[2:3]])
    exp_p = torch.cat([probs[3:6], probs[0:2], probs[2:3]])
    assert torch.equal(P.moe_sort_chunks_by_index(inp.to(DEV), sizes, order).cpu(), exp)
    o, p = P.moe_sort_chunks_by_index_with_probs(inp.to(DEV), probs.to(DEV), sizes, order)
    assert torch.equal(o.cpu(), exp) and torch.equal(p.cpu(), exp_p)


def test_argument_errors_match_reference(P):
    x = TOKENS.to(DEV)
    with pytest.raises(ValueError, match="map_type"):
        P.moe_permute(x, MASK.to(DEV), map_type="rows")
    with pytest.raises(ValueError, match="2D"):
        P.moe_permute(x, MASK.to(DEV)[0], map_type="mask")
    with pytest.raises(ValueError, match="same num_tokens"):
        P.moe_permute(x, MASK.to(DEV)[:2], map_type="mask")
    with pytest.raises(ValueError, match="restore_shape or merging_probs"):
        P.moe_unpermute(x, torch.tensor([0, 1, 2], device=DEV))
    with pytest.raises(ValueError, match="deprecated"):
        P.moe_unpermute(x, torch.tensor([0, 1, 2], device=DEV), merging_probs=MASK_PROBS.to(DEV), probs=MASK_PROBS.to(DEV))
    with pytest.raises(ValueError, match="1D"):
        P.moe_sort_chunks_by_index(x, torch.tensor([[3]]), torch.tensor([0]))
    empty = torch.zeros(0, 4, device=DEV)
    out, rid = P.moe_permute(empty, torch.zeros(0, 2, dtype=torch.int64, device=DEV), map_type="index")
    assert out.numel() == 0 and rid.numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,K,H", [(257, 8, 2, 64), (1000, 130, 6, 200), (64, 5000, 4, 24)])
def test_index_map_matches_oracle(P, dtype, T, E, K, H):
    gen = torch.Generator().manual_seed(5)
    ids = torch.randint(-E // 6, E, (T, K), generator=gen)
    x = torch.randn(T, H, generator=gen).to(dtype)
    probs = torch.rand(T, K, generator=gen)
    ref_out, ref_rid = O.moe_permute(x, ids, map_type="index")
    xg = x.to(DEV).requires_grad_(True)
    out, rid = P.moe_permute(xg, ids.to(DEV), map_type="index")
    assert torch.equal(rid.cpu(), ref_rid)
    assert torch.equal(out.detach().cpu(), ref_out)
    ref_back = O.moe_unpermute(ref_out.float(), ref_rid, merging_probs=probs, restore_shape=x.shape, map_type="index")
    back = P.moe_unpermute(out, rid, merging_probs=probs.to(DEV), restore_shape=x.shape, map_type="index")
    assert rel_l2(back.detach(), ref_back) <= (1e-6 if dtype == torch.float32 else 1e-2)
    # gradient of the round trip w.r.t. the tokens: d x[t] = go[t] * sum of the probs of its valid slots
    go = torch.randn(T, H, generator=gen).to(dtype)
    back.backward(go.to(DEV))
    scale = (probs * (ids >= 0)).sum(1, keepdim=True)
    assert rel_l2(xg.grad, go.float() * scale) <= (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("pad", [-1, 7, -5])
def test_mask_map_matches_oracle(P, pad):
    gen = torch.Generator().manual_seed(6)
    T, E, H = 300, 40, 48
    mask = torch.rand(T, E, generator=gen) < 0.1
    probs = torch.rand(T, E, generator=gen) * mask
    x = torch.randn(T, H, generator=gen)
    n_true = int(mask.sum())
    n_out = -1 if pad == -1 else n_true + pad
    ref_out, ref_rid, ref_pp = O.moe_permute(x, mask, num_out_tokens=n_out, probs=probs)
    out, pp, rid = P.moe_permute_with_probs(x.to(DEV), probs.to(DEV), mask.to(DEV), num_out_tokens=n_out)
    assert torch.equal(rid.cpu(), ref_rid)
    assert torch.equal(out.cpu(), ref_out)
    assert torch.equal(pp.cpu(), ref_pp)
    ref_back = O.moe_unpermute(ref_out, ref_rid, merging_probs=probs, restore_shape=x.shape)
    back = P.moe_unpermute(out, rid, merging_probs=probs.to(DEV), restore_shape=x.shape)
    assert rel_l2(back, ref_back) <= 1e-6
    # unweighted, token count from restore_shape
    ref_plain = O.moe_unpermute(ref_out, ref_rid, restore_shape=x.shape)
    plain = P.moe_unpermute(out, rid, restore_shape=x.shape)
    assert rel_l2(plain, ref_plain) <= 1e-6


def test_probabilities_receive_gradients_like_the_reference(P):
    """The reference's helpers are plain differentiable torch code (permute_utils.py:43-89,
    157-234): merging_probs gets d out . row, probs the scatter-add of d permuted_probs."""
    gen = torch.Generator().manual_seed(9)
    T, E, H = 120, 12, 40
    mask = torch.rand(T, E, generator=gen) < 0.2
    probs = torch.rand(T, E, generator=gen) * mask
    x = torch.randn(T, H, generator=gen)
    go = torch.randn(T, H, generator=gen)
    gp = torch.randn(int(mask.sum()), generator=gen)

    # mask map: permute_with_probs -> (rows * permuted_probs) -> unpermute with merging_probs
    xr, pr, mr = x.clone().requires_grad_(True), probs.clone().requires_grad_(True), probs.clone().requires_grad_(True)
    r_out, r_rid, r_pp = O.moe_permute(xr, mask, probs=pr)
    r_back = O.moe_unpermute(r_out * r_pp.unsqueeze(1), r_rid, merging_probs=mr, restore_shape=x.shape)
    (r_back * go).sum().add((r_pp * gp).sum()).backward()
    xg, pg, mg = (t.clone().to(DEV).requires_grad_(True) for t in (x, probs, probs))
    out, pp, rid = P.moe_permute_with_probs(xg, pg, mask.to(DEV))
    back = P.moe_unpermute(out * pp.unsqueeze(1), rid, merging_probs=mg, restore_shape=x.shape)
    (back * go.to(DEV)).sum().add((pp * gp.to(DEV)).sum()).backward()
    assert rel_l2(back, r_back) <= 1e-6
    assert mg.grad is not None and rel_l2(mg.grad, mr.grad) <= 1e-5
    assert pg.grad is not None and rel_l2(pg.grad, pr.grad) <= 1e-5
    assert rel_l2(xg.grad, xr.grad) <= 1e-5
    assert float(mg.grad.cpu()[~mask].abs().sum()) == 0.0  # unrouted entries take no part

    # index map
    K = 3
    ids = torch.randint(-2, E, (T, K), generator=gen)
    w = torch.rand(T, K, generator=gen)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    r_out, r_rid = O.moe_permute(xr, ids, map_type="index")
    (O.moe_unpermute(r_out, r_rid, merging_probs=wr, restore_shape=x.shape, map_type="index") * go).sum().backward()
    xg, wg = x.clone().to(DEV).requires_grad_(True), w.clone().to(DEV).requires_grad_(True)
    out, rid = P.moe_permute(xg, ids.to(DEV), map_type="index")
    (P.moe_unpermute(out, rid, merging_probs=wg, restore_shape=x.shape, map_type="index") * go.to(DEV)).sum().backward()
    assert wg.grad is not None and rel_l2(wg.grad, wr.grad) <= 1e-5
    assert rel_l2(xg.grad, xr.grad) <= 1e-5

    # chunk sort with probabilities
    sizes, order = torch.tensor([50, 30, 40]), torch.tensor([2, 0, 1])
    pv = torch.rand(T, generator=gen)
    gv = torch.randn(T, generator=gen)
    pvr = pv.clone().requires_grad_(True)
    _, r_p = O.moe_sort_chunks_by_index(x, sizes, order, probs=pvr)
    (r_p * gv).sum().backward()
    pvg = pv.clone().to(DEV).requires_grad_(True)
    _, p_dev = P.moe_sort_chunks_by_index_with_probs(x.to(DEV), pvg, sizes, order)
    (p_dev * gv.to(DEV)).sum().backward()
    assert rel_l2(pvg.grad, pvr.grad) <= 1e-6
