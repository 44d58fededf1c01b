"""The shapes and input recipes of the reference's own benchmark scripts, with the oracle as the
baseline (the scripts compare an alternative backend with the baseline path the same way,
`assert_close(rtol=atol=1e-2)` for floats and exact equality for integers):

  benchmarks/benchmark_grouped_gemm.py:15-26       G=36 x 3256 rows, k=4096, n=2560, bf16, trans_b=False
  benchmarks/benchmark_routed_grouped_ffn.py:15-28 T=8192 H=4096 K=2 E=36 F=1280, 10 % unused slots
  benchmarks/benchmark_moe_routing.py:15-36        T=8192 K=2 E=128 (10 % unused); T=32768 K=2 E=288 with duplicates
  benchmarks/benchmark_moe_scatter.py:15-32, benchmark_moe_gather.py:14-32   T=8192 H=256 K=2 E=8 and their edge cases
"""

import pytest
import torch

from oracle import moe_oracle as O
from steptronoss_amd.model.common.feed_forward import swiglu
from steptronoss_amd.model.utils import moe_utils as M
from steptronoss_amd.utils.optimizable import set_optimization
from tests.helpers import make_topk_ids, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 1e-2


@pytest.fixture(autouse=True)
def _select_backend():
    set_optimization(default=M.BACKEND_NAME)
    yield
    set_optimization()


def test_grouped_gemm_benchmark_shape():
    # the oracle at this size would take minutes on the host, so the GPU result is compared with
    # fp32 arithmetic on the same bf16 inputs for sampled groups (rows, input gradient) and whole
    # groups (weight gradient); trans_b=False: b is [G, k, n]
    G, rows, k, n = 36, 3256, 4096, 2560
    gen = torch.Generator(device=DEV).manual_seed(0)
    a = torch.randn(G * rows, k, device=DEV, generator=gen).bfloat16().requires_grad_(True)
    b = (torch.randn(G, k, n, device=DEV, generator=gen) * 0.02).bfloat16().requires_grad_(True)
    sizes = torch.full((G,), rows, dtype=torch.int64)
    out = M.grouped_gemm(a, b, sizes)  # trans_b defaults to False, as in the script
    assert out.shape == (G * rows, n) and out.dtype == torch.bfloat16
    go = torch.randn(out.shape, device=DEV, generator=gen).bfloat16()
    out.backward(go)
    for g in (0, 17, 35):
        lo = g * rows
        pick = lo + torch.linspace(0, rows - 1, 96, device=DEV).long()
        ref = a.detach()[pick].float() @ b.detach()[g].float()
        assert rel_l2(out.detach()[pick], ref) <= TOL
        assert rel_l2(a.grad[pick], go[pick].float() @ b.detach()[g].float().t()) <= TOL
        ref_db = a.detach()[lo : lo + rows].float().t() @ go[lo : lo + rows].float()
        assert rel_l2(b.grad[g], ref_db) <= TOL


def _bench_swiglu(x, swiglu_limit=None):  # the script's own activation (benchmark_routed_grouped_ffn.py:46-52)
    left, right = torch.chunk(x, 2, dim=-1)
    left = torch.nn.functional.silu(left)
    return left * right


@pytest.mark.parametrize("act_kind", ["known", "opaque"])
def test_routed_grouped_ffn_benchmark_shape(act_kind):
    T, H, K, E, Fh = 8192, 4096, 2, 36, 1280
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(T, H, generator=gen).bfloat16()
    w1 = (torch.randn(E, 2 * Fh, H, generator=gen) * 0.02).bfloat16()
    w2 = (torch.randn(E, H, Fh, generator=gen) * 0.02).bfloat16()
    ids = make_topk_ids(T, K, E, gen=gen, allow_dupe=False, invalid_frac=0.1)
    tw = torch.rand(T, K, generator=gen)
    tw = tw / tw.sum(1, keepdim=True)
    ref_in = [t.clone().float().requires_grad_(True) for t in (w1, w2, x, tw)]
    ref = O.routed_grouped_ffn(ref_in[0], ref_in[1], O.swiglu, ref_in[2], ids, ref_in[3])
    ref.sum().backward()  # the script's backward seed (benchmark_routed_grouped_ffn.py:109)
    got_in = [t.to(DEV).requires_grad_(True) for t in (w1, w2, x, tw)]
    act = swiglu if act_kind == "known" else _bench_swiglu
    out = M.routed_grouped_ffn(got_in[0], got_in[1], act, got_in[2], ids.to(DEV), got_in[3])
    out.sum().backward()
    assert rel_l2(out, ref) <= TOL
    for name, g, r in zip(("dw1", "dw2", "dx", "dtw"), got_in, ref_in):
        assert rel_l2(g.grad, r.grad) <= TOL, name


@pytest.mark.parametrize("T,K,E,inv,dupe", [(8192, 2, 128, 0.1, False), (32768, 2, 288, 0.0, True)])
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_routing_benchmark_shapes(T, K, E, inv, dupe, dtype):
    gen = torch.Generator().manual_seed(0)
    ids = make_topk_ids(T, K, E, gen=gen, allow_dupe=dupe, invalid_frac=inv, dtype=dtype)
    ref_h = O.histogram(ids, E)
    ref_p = O.index_compute(ids, ref_h)
    h = M.histogram(ids.to(DEV), E)
    assert torch.equal(h.cpu(), ref_h)
    assert torch.equal(M.index_compute(ids.to(DEV), h).cpu(), ref_p)


SCATTER_CASES = [
    # name, T, H, K, E, all_invalid, allow_dupe   (benchmark_moe_scatter.py:15-32)
    ("main", 8192, 256, 2, 8, False, False),
    ("zero_tokens", 0, 8, 1, 4, False, False),
    ("all_invalid", 8, 8, 2, 4, True, False),
    ("topk1", 16, 8, 1, 4, False, False),
    ("dupe_indices", 16, 8, 2, 4, False, True),
]


@pytest.mark.parametrize("name,T,H,K,E,all_invalid,dupe", SCATTER_CASES)
def test_scatter_benchmark_cases(name, T, H, K, E, all_invalid, dupe):
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=gen).bfloat16()
    ids = make_topk_ids(T, K, E, gen=gen, allow_dupe=dupe)
    if all_invalid:
        ids = torch.full_like(ids, -1)
    index = O.index_compute(ids, O.histogram(ids, E))
    xr = x.clone().float().requires_grad_(True)
    ref = O.moe_scatter(xr, index)
    xg = x.to(DEV).requires_grad_(True)
    out = M.moe_scatter(xg, index.to(DEV))
    assert out.shape == ref.shape and torch.equal(out.detach().cpu().float(), ref.detach())
    if out.numel():
        go = torch.randn(out.shape, generator=gen).bfloat16()
        ref.backward(go.float())
        out.backward(go.to(DEV))
        assert rel_l2(xg.grad, xr.grad) <= TOL


def _gather_inputs(T, H, K, inv, dupe, gen):
    """benchmark_moe_gather.py:35-58: the index is drawn over all T*K rows, so several slots may
    name one row (only column 0 is kept apart)."""
    x = torch.randn(T * K, H, generator=gen).bfloat16()
    if T == 0 or K == 0:
        return x, torch.empty((T, K), dtype=torch.int64), torch.empty((T, K))
    idx = torch.randint(0, T * K, (T, K), generator=gen, dtype=torch.int64)
    if not dupe and K > 1:
        for i in range(1, K):
            clash = idx[:, i] == idx[:, 0]
            idx[clash, i] = (idx[clash, i] + i) % (T * K)
    if inv > 0:
        idx[torch.rand(T, K, generator=gen) < inv] = -1
    w = torch.rand(T, K, generator=gen)
    return x, idx, w / w.sum(1, keepdim=True)


GATHER_CASES = [
    ("main", 8192, 256, 2, 0.1, False),
    ("zero_tokens", 0, 8, 1, 0.0, False),
    ("all_invalid", 8, 8, 2, 1.0, False),
    ("topk1", 16, 8, 1, 0.0, False),
    ("dupe_indices", 16, 8, 2, 0.0, True),
    ("stress0", 512, 64, 4, 0.0, False),
    ("stress1", 333, 40, 3, 0.3, True),
]


@pytest.mark.parametrize("name,T,H,K,inv,dupe", GATHER_CASES)
def test_gather_benchmark_cases(name, T, H, K, inv, dupe):
    gen = torch.Generator().manual_seed(2)
    x, idx, w = _gather_inputs(T, H, K, inv, dupe, gen)
    xr, wr = x.clone().float().requires_grad_(True), w.clone().requires_grad_(True)
    ref = O.moe_weighted_gather(xr, idx, wr)
    xg, wg = x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    out = M.moe_weighted_gather(xg, idx.to(DEV), wg)
    assert out.shape == ref.shape
    if out.numel() == 0:
        return
    assert rel_l2(out, ref) <= TOL
    ref.sum().backward()  # the script's backward seed
    out.sum().backward()
    assert rel_l2(xg.grad, xr.grad) <= TOL
    assert rel_l2(wg.grad, wr.grad) <= TOL
