"""GPU parity of the four bandwidth-bound ops against the CPU oracle.

Integer outputs and permuted rows are compared bit-exactly; sums within the stated
tolerances.  The known-answer cases are the reference's (tests/test_moe_utils.py), run
through the HIP path."""

import pytest
import torch

from oracle import moe_oracle as O
from steptronoss_amd.model.utils import moe_utils as M
from steptronoss_amd.utils.optimizable import set_optimization
from tests.helpers import make_topk_ids, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(autouse=True)
def _select_backend():
    set_optimization(default=M.BACKEND_NAME)
    yield
    set_optimization()


# ------------------------------------------------------------------ histogram
def test_histogram_kats():
    out = M.histogram(torch.tensor([0, 1, 1, 3, 3, 3], device=DEV), 4)
    assert out.dtype == torch.int32 and out.tolist() == [1, 2, 0, 3]
    assert M.histogram(torch.tensor([], dtype=torch.int32, device=DEV), 3).tolist() == [0, 0, 0]
    assert M.histogram(torch.tensor([0, -1, 2, -3, 2], device=DEV), 4).tolist() == [1, 0, 2, 0]
    with pytest.raises(ValueError, match="out-of-range"):
        M.histogram(torch.tensor([0, 2], device=DEV), 2)
    with pytest.raises(TypeError):
        M.histogram(torch.tensor([0.5], device=DEV), 2)
    assert M.histogram(torch.tensor([1], device=DEV), 0).shape == (0,)


@pytest.mark.parametrize(
    "T,K,E,dtype,dupe,inv",
    [
        (4096, 2, 64, torch.int32, False, 0.0),
        (4096, 2, 64, torch.int64, False, 0.3),
        (4096, 2, 64, torch.int64, True, 0.1),
        (16384, 8, 128, torch.int64, False, 0.0),
        (8192, 8, 256, torch.int32, False, 0.05),
        (1000, 3, 7, torch.int64, True, 0.5),
        (513, 1, 1, torch.int32, False, 0.0),
        (777, 5, 1000, torch.int64, False, 0.0),
        (300, 2, 4096, torch.int32, False, 0.1),
    ],
)
def test_histogram_and_index_match_oracle(T, K, E, dtype, dupe, inv):
    gen = torch.Generator().manual_seed(0)
    ids = make_topk_ids(T, K, E, gen=gen, allow_dupe=dupe, invalid_frac=inv, dtype=dtype)
    ref_h = O.histogram(ids, E)
    ref_p = O.index_compute(ids, ref_h)
    h = M.histogram(ids.to(DEV), E)
    assert h.dtype == torch.int32 and torch.equal(h.cpu(), ref_h)
    for hist_dtype in (torch.int32, torch.int64):
        p = M.index_compute(ids.to(DEV), h.to(hist_dtype))
        assert p.dtype == torch.int32 and torch.equal(p.cpu(), ref_p)
    hist, offsets, pos, status = M.route_plan(ids.to(DEV), E)
    assert torch.equal(hist.cpu(), ref_h) and torch.equal(pos.cpu(), ref_p)
    assert offsets.cpu().tolist() == [0] + torch.cumsum(ref_h, 0).tolist()
    assert status.tolist()[:2] == [0, int((ids >= 0).sum())]


def test_index_compute_kats_and_errors():
    out = M.index_compute(torch.tensor([[0, 1], [1, 0], [0, 1]], device=DEV), torch.tensor([3, 3], dtype=torch.int32, device=DEV))
    assert out.dtype == torch.int32 and out.tolist() == [[0, 3], [4, 1], [2, 5]]
    out = M.index_compute(torch.tensor([[0, -1], [1, -2], [0, 1]], device=DEV), torch.tensor([2, 2], dtype=torch.int32, device=DEV))
    assert out.tolist() == [[0, -1], [2, -2], [1, 3]]
    with pytest.raises(AssertionError, match="expert_histogram does not match"):
        M.index_compute(torch.tensor([[0, 1], [1, -1]], device=DEV), torch.tensor([1, 1], dtype=torch.int32, device=DEV))
    with pytest.raises(ValueError):
        M.index_compute(torch.tensor([0, 1], device=DEV), torch.tensor([1, 1], dtype=torch.int32, device=DEV))
    assert M.index_compute(torch.zeros((0, 2), dtype=torch.int64, device=DEV), torch.zeros(4, dtype=torch.int32, device=DEV)).shape == (0, 2)


def test_given_histogram_sets_the_base_offsets():
    # positions use the GIVEN histogram for the expert bases (reference moe_utils.py:188-189)
    ids = torch.tensor([[0, 2], [2, 0]], device=DEV)
    M.settings.validate = False
    try:
        out = M.index_compute(ids, torch.tensor([3, 1, 2], dtype=torch.int32, device=DEV))
    finally:
        M.settings.validate = True
    assert out.tolist() == [[0, 4], [5, 1]]


# ------------------------------------------------------------------ permute
def test_permute_kats():
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0]], device=DEV)
    assert M.moe_scatter(x, torch.tensor([[0, 2], [1, 3]], device=DEV)).tolist() == [[1, 2], [3, 4], [1, 2], [3, 4]]
    assert M.moe_scatter(x, torch.tensor([[0, -1], [1, -2]], device=DEV)).tolist() == [[1, 2], [3, 4]]
    xg = x.clone().requires_grad_(True)
    M.moe_scatter(xg, torch.tensor([[0, 2], [1, 3]], device=DEV)).sum().backward()
    assert xg.grad.tolist() == [[2, 2], [2, 2]]
    xg = x.clone().requires_grad_(True)
    M.moe_scatter(xg, torch.tensor([[0, -1], [1, -2]], device=DEV)).sum().backward()
    assert xg.grad.tolist() == [[1, 1], [1, 1]]
    with pytest.raises(ValueError):
        M.moe_scatter(x, torch.tensor([0, 1], device=DEV))


@pytest.mark.parametrize(
    "T,H,K,E,dtype,inv",
    [
        (2048, 256, 2, 64, torch.bfloat16, 0.2),
        (1024, 2048, 8, 128, torch.bfloat16, 0.0),
        (512, 7168, 8, 256, torch.bfloat16, 0.0),
        (300, 8, 2, 8, torch.float32, 0.3),
        (300, 6, 3, 8, torch.bfloat16, 0.1),  # 12-byte rows: no 128-bit path
        (257, 33, 1, 4, torch.float16, 0.0),
        (64, 1000, 4, 16, torch.float32, 0.0),
    ],
)
def test_permute_matches_oracle(T, H, K, E, dtype, inv):
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=gen).to(dtype)
    ids = make_topk_ids(T, K, E, gen=gen, invalid_frac=inv)
    pos = O.index_compute(ids, O.histogram(ids, E))
    ref = O.moe_scatter(x, pos)
    xg = x.to(DEV).requires_grad_(True)
    out = M.moe_scatter(xg, pos.to(DEV))
    assert out.dtype == dtype and out.shape == ref.shape
    assert torch.equal(out.detach().cpu().view(torch.uint8), ref.view(torch.uint8))  # bit-exact rows
    go = torch.randn(ref.shape, generator=gen).to(dtype)
    out.backward(go.to(DEV))
    xr = x.clone().float().requires_grad_(True)
    O.moe_scatter(xr, pos).backward(go.float())
    assert rel_l2(xg.grad, xr.grad) <= (4e-3 if dtype != torch.float32 else 1e-6)
    assert xg.grad.dtype == dtype


def test_permute_non_bijective_index_leaves_zero_rows():
    # two slots name row 0, row 2 is named by none: it must read as zeros (new_zeros in the reference)
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], device=DEV)
    out = M.moe_scatter(x, torch.tensor([[0], [1], [1]], device=DEV))
    assert out.shape == (3, 2) and out[0].tolist() == [1.0, 2.0] and out[2].tolist() == [0.0, 0.0]
    assert out[1].tolist() in ([3.0, 4.0], [5.0, 6.0])


def test_permute_empty():
    x = torch.randn(4, 8, device=DEV)
    assert M.moe_scatter(x, torch.full((4, 2), -1, device=DEV)).shape == (0, 8)
    assert M.moe_scatter(torch.zeros(0, 8, device=DEV), torch.zeros((0, 2), dtype=torch.int64, device=DEV)).shape == (0, 8)


# ------------------------------------------------------------------ unpermute / combine
def test_combine_kats():
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], device=DEV)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]], device=DEV)
    out = M.moe_weighted_gather(x, torch.tensor([[2, 0], [1, 2]], device=DEV), w)
    assert torch.allclose(out.cpu(), torch.tensor([[1.8, 2.8], [5.5, 7.0]]))
    out = M.moe_weighted_gather(x, torch.tensor([[2, -1], [1, -2]], device=DEV), w)
    assert torch.allclose(out.cpu(), torch.tensor([[1.0, 1.2], [3.0, 4.0]]))


def test_combine_grad_kats():
    # idx [[2,0],[1,2]] names row 2 twice: not a position map index_compute can produce; the
    # reference KAT with distinct rows is the "negative indices" one
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], device=DEV, requires_grad=True)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]], device=DEV, requires_grad=True)
    M.moe_weighted_gather(x, torch.tensor([[2, -1], [1, -2]], device=DEV), w).sum().backward()
    assert torch.allclose(x.grad.cpu(), torch.tensor([[0.0, 0.0], [1.0, 1.0], [0.2, 0.2]]))
    assert torch.allclose(w.grad.cpu(), torch.tensor([[11.0, 0.0], [7.0, 0.0]]))


def test_round_trip_symmetry():
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0]], device=DEV)
    idx = torch.tensor([[0, 1, 2], [3, 4, 5]], device=DEV)
    back = M.moe_weighted_gather(M.moe_scatter(x, idx), idx, torch.ones(2, 3, device=DEV))
    assert torch.allclose(back, x * 3)
    idx = torch.tensor([[0, -1, 1], [2, -2, 3]], device=DEV)
    back = M.moe_weighted_gather(M.moe_scatter(x, idx), idx, torch.ones(2, 3, device=DEV))
    assert torch.allclose(back, x * (idx >= 0).sum(1, keepdim=True))


@pytest.mark.parametrize(
    "T,H,K,E,dtype,wdtype,inv",
    [
        (2048, 256, 2, 8, torch.bfloat16, torch.float32, 0.0),
        (1024, 2048, 8, 128, torch.bfloat16, torch.float32, 0.0),
        (512, 7168, 8, 256, torch.bfloat16, torch.float32, 0.1),
        (512, 512, 4, 16, torch.bfloat16, torch.bfloat16, 0.3),
        (300, 8, 2, 8, torch.float32, torch.float32, 0.3),
        (300, 6, 3, 8, torch.bfloat16, torch.float32, 0.1),
        (257, 33, 1, 4, torch.float16, torch.float16, 0.0),
        (100, 96, 12, 32, torch.float32, torch.bfloat16, 0.0),
    ],
)
def test_combine_matches_oracle(T, H, K, E, dtype, wdtype, inv):
    gen = torch.Generator().manual_seed(2)
    ids = make_topk_ids(T, K, E, gen=gen, invalid_frac=inv)
    pos = O.index_compute(ids, O.histogram(ids, E))
    n_rows = int((ids >= 0).sum())
    rows = torch.randn(n_rows, H, generator=gen).to(dtype)
    w = torch.rand(T, K, generator=gen).to(wdtype)
    tol = 1e-5 if dtype == torch.float32 and wdtype == torch.float32 else 1e-2
    # oracle in the op's own dtypes (reproduces its rounding points) ...
    ref_same = O.moe_weighted_gather(rows, pos, w)
    # ... and in fp32 from the same rounded inputs
    rr = rows.clone().float().requires_grad_(True)
    wr = w.clone().float().requires_grad_(True)
    ref32 = O.moe_weighted_gather(rr, pos, wr)
    rg = rows.to(DEV).requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    out = M.moe_weighted_gather(rg, pos.to(DEV), wg)
    assert out.dtype == dtype and out.shape == (T, H)
    assert rel_l2(out, ref_same.float()) <= (1e-6 if dtype == torch.float32 else 4e-3)
    assert rel_l2(out, ref32) <= tol
    go = torch.randn(T, H, generator=gen).to(dtype)
    out.backward(go.to(DEV))
    ref32.backward(go.float())
    assert rg.grad.dtype == dtype and wg.grad.dtype == wdtype
    assert rel_l2(rg.grad, rr.grad) <= tol
    assert rel_l2(wg.grad, wr.grad) <= tol


def test_combine_backward_zeroes_unnamed_rows():
    rows = torch.randn(6, 16, device=DEV, requires_grad=True)
    pos = torch.tensor([[0, 3], [-1, 5]], device=DEV)
    w = torch.rand(2, 2, device=DEV, requires_grad=True)
    M.moe_weighted_gather(rows, pos, w).sum().backward()
    assert float(rows.grad[[1, 2, 4]].abs().sum()) == 0.0
    assert torch.allclose(rows.grad[3], w[0, 1].detach().expand(16))


def test_combine_backward_reference_kat_shared_rows():
    # reference tests/test_moe_utils.py:81-92: row 2 is named by two slots
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], device=DEV, requires_grad=True)
    idx = torch.tensor([[2, 0], [1, 2]], dtype=torch.int64, device=DEV)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]], device=DEV, requires_grad=True)
    M.moe_weighted_gather(x, idx, w).sum().backward()
    assert torch.allclose(x.grad.cpu(), torch.tensor([[0.8, 0.8], [1.0, 1.0], [0.7, 0.7]]))
    assert torch.allclose(w.grad.cpu(), torch.tensor([[11.0, 3.0], [7.0, 11.0]]))


def test_combine_backward_reference_kat_negative_indices():
    # reference tests/test_moe_utils.py:95-104
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], device=DEV, requires_grad=True)
    idx = torch.tensor([[2, -1], [1, -2]], dtype=torch.int64, device=DEV)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]], device=DEV, requires_grad=True)
    M.moe_weighted_gather(x, idx, w).sum().backward()
    assert torch.allclose(x.grad.cpu(), torch.tensor([[0.0, 0.0], [1.0, 1.0], [0.2, 0.2]]))
    assert torch.allclose(w.grad.cpu(), torch.tensor([[11.0, 0.0], [7.0, 0.0]]))


@pytest.mark.parametrize(
    "T,K,H,n_rows,dtype,idt",
    [
        (300, 4, 64, 97, torch.float32, torch.int64),  # many slots per row, one sort pass
        (700, 3, 72, 5000, torch.bfloat16, torch.int32),  # > 4096 rows: two sort passes, some rows unnamed
        (64, 8, 40, 9000, torch.float16, torch.int64),  # mostly unnamed rows, odd width
    ],
)
def test_combine_backward_any_index_matches_oracle(T, K, H, n_rows, dtype, idt):
    gen = torch.Generator().manual_seed(11)
    pos = torch.randint(-n_rows // 8, n_rows, (T, K), generator=gen).to(idt)  # repeats and negatives
    rows = torch.randn(n_rows, H, generator=gen).to(dtype)
    w = torch.rand(T, K, generator=gen)
    go = torch.randn(T, H, generator=gen).to(dtype)
    rr = rows.clone().float().requires_grad_(True)
    wr = w.clone().requires_grad_(True)
    O.moe_weighted_gather(rr, pos, wr).backward(go.float())
    rg = rows.to(DEV).requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    out = M.moe_weighted_gather(rg, pos.to(DEV), wg)
    out.backward(go.to(DEV))
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert rel_l2(rg.grad, rr.grad) <= tol
    assert rel_l2(wg.grad, wr.grad) <= tol
    unnamed = torch.ones(n_rows, dtype=torch.bool)
    unnamed[pos[pos >= 0].long()] = False
    assert float(rg.grad.cpu()[unnamed].abs().sum()) == 0.0
    # deterministic: a second run gives the same bits
    rg2 = rows.to(DEV).requires_grad_(True)
    M.moe_weighted_gather(rg2, pos.to(DEV), wg.detach().requires_grad_(True)).backward(go.to(DEV))
    assert torch.equal(rg.grad, rg2.grad)


def test_cpu_tensors_are_refused():
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        M.histogram(torch.tensor([0, 1]), 2)
