"""Grouped GEMM forward / dgrad / wgrad on the GPU against the fp32 oracle.

Tolerance: rel-L2 <= 1e-2 for bf16/fp16 (inputs identical, products accumulated in fp32,
one rounding of the output), <= 1e-5 for fp32."""

import pytest
import torch

from oracle import moe_oracle as O
from steptronoss_amd.model.utils import moe_utils as M
from steptronoss_amd.utils.optimizable import set_optimization
from tests.helpers import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(autouse=True)
def _select_backend():
    set_optimization(default=M.BACKEND_NAME)
    yield
    set_optimization()


def _run_case(sizes, k, n, trans_b, dtype, sizes_on_device, tol, seed=0):
    gen = torch.Generator().manual_seed(seed)
    sizes = torch.tensor(sizes, dtype=torch.int64)
    G, Mrows = sizes.numel(), int(sizes.sum())
    a = torch.randn(Mrows, k, generator=gen).to(dtype)
    b = (torch.randn(G, n, k, generator=gen) if trans_b else torch.randn(G, k, n, generator=gen)).to(dtype)
    go = torch.randn(Mrows, n, generator=gen).to(dtype)
    ar = a.clone().float().requires_grad_(True)
    br = b.clone().float().requires_grad_(True)
    ref = O.grouped_gemm(ar, br, sizes, trans_b)
    ref.backward(go.float())
    ag = a.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True)
    out = M.grouped_gemm(ag, bg, sizes.to(DEV) if sizes_on_device else sizes, trans_b=trans_b)
    assert out.shape == ref.shape and out.dtype == dtype
    out.backward(go.to(DEV))
    assert rel_l2(out, ref) <= tol, ("fwd", rel_l2(out, ref))
    assert rel_l2(ag.grad, ar.grad) <= tol, ("dgrad", rel_l2(ag.grad, ar.grad))
    assert rel_l2(bg.grad, br.grad) <= tol, ("wgrad", rel_l2(bg.grad, br.grad))
    for g, m in enumerate(sizes.tolist()):
        if m == 0:
            assert float(bg.grad[g].abs().max()) == 0.0  # empty group => zero weight gradient


@pytest.mark.parametrize("trans_b", [False, True])
def test_reference_case_tiny_unaligned(trans_b):
    # the reference's own test shape (tests/test_grouped_gemm.py:24-49): rows of 12 bytes
    _run_case([3, 1, 4], 8, 6, trans_b, torch.bfloat16, False, 1e-2)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize(
    "sizes,k,n,dtype,tol",
    [
        ([3, 1, 4], 8, 6, torch.float32, 1e-5),
        ([5, 0, 70, 1], 24, 40, torch.float32, 1e-5),
        ([64, 64], 64, 64, torch.bfloat16, 1e-2),
        ([100, 0, 37, 1, 300], 64, 96, torch.bfloat16, 1e-2),
        ([130, 250, 0, 0, 129, 3], 200, 264, torch.bfloat16, 1e-2),  # k not a multiple of 64
        ([77, 200], 72, 136, torch.float16, 1e-2),
        ([300, 20, 500], 520, 512, torch.bfloat16, 1e-2),
    ],
)
def test_matches_oracle(sizes, k, n, dtype, tol, trans_b):
    _run_case(sizes, k, n, trans_b, dtype, False, tol)


@pytest.mark.parametrize("trans_b", [False, True])
def test_big_tile_path_ragged(trans_b):
    # >= 8192 rows and n >= 512 selects the 256x256 tile; ragged sizes incl. empty and huge groups
    sizes = [1024, 0, 3000, 17, 255, 257, 2048, 1, 0, 1600]
    _run_case(sizes, 256, 768, trans_b, torch.bfloat16, True, 1e-2)


def test_batch_sizes_shorter_than_rows():
    gen = torch.Generator().manual_seed(3)
    a = torch.randn(10, 16, generator=gen)
    b = torch.randn(2, 8, 16, generator=gen)
    sizes = torch.tensor([3, 4])
    out = M.grouped_gemm(a.to(DEV), b.to(DEV), sizes, trans_b=True)
    assert out.shape == (7, 8)
    assert rel_l2(out, O.grouped_gemm(a, b, sizes, True)) < 1e-5


def test_empty():
    a = torch.zeros(0, 16, device=DEV)
    b = torch.randn(3, 8, 16, device=DEV)
    assert M.grouped_gemm(a, b, torch.zeros(3, dtype=torch.int64), trans_b=True).shape == (0, 8)


def test_argument_errors():
    a = torch.zeros(4, 16, device=DEV)
    with pytest.raises(ValueError):
        M.grouped_gemm(a, torch.zeros(2, 8, 12, device=DEV), torch.tensor([2, 2]), trans_b=True)
    with pytest.raises(TypeError):
        M.grouped_gemm(a, torch.zeros(2, 8, 16, device=DEV, dtype=torch.bfloat16), torch.tensor([2, 2]), trans_b=True)


# ----- SwiGLU fused into the GEMM epilogues: same bits as the GEMM followed by the SwiGLU kernel
@pytest.mark.parametrize("limit", [None, 0.75])
@pytest.mark.parametrize(
    "sizes,k,ffn,dtype",
    [
        ([1000, 0, 37, 2500, 300, 900], 256, 192, torch.bfloat16),  # ragged groups, an empty one, half-used column tile
        ([513, 2047, 1536], 96, 768, torch.bfloat16),  # contraction a multiple of 32 only
        ([4096, 256], 128, 72, torch.float16),  # narrow FFN: most of a tile's columns unused
    ],
)
def test_fused_swiglu_epilogues_match_the_unfused_pair(sizes, k, ffn, dtype, limit):
    from steptronoss_amd.model.common.feed_forward import swiglu_bwd_rows, swiglu_fwd_rows

    gen = torch.Generator().manual_seed(9)
    E, m = len(sizes), sum(sizes)
    a = torch.randn(m, k, generator=gen).to(dtype).to(DEV)
    w1 = (torch.randn(E, 2 * ffn, k, generator=gen) * 0.2).to(dtype).to(DEV)
    w2 = (torch.randn(E, k, ffn, generator=gen) * 0.2).to(dtype).to(DEV)
    gy = torch.randn(m, k, generator=gen).to(dtype).to(DEV)
    offsets = M._group_offsets(torch.tensor(sizes), torch.device(DEV))
    def same(got, ref):
        # bf16: the same bits.  fp16: the compiler may merge a result's last multiplication with
        # its conversion to fp16 (one rounding, v_fma_mixlo_f16) in one kernel and not in the
        # other (two roundings), so single results may sit one fp16 step apart.
        if dtype == torch.bfloat16:
            return torch.equal(got, ref)
        g, r = got.float(), ref.float()
        return bool(((g - r).abs() <= 2.0**-10 * torch.maximum(g.abs(), r.abs()) + 1e-7).all())

    gu, h = M._gemm_swiglu_rows(a, w1, offsets, limit)
    assert h is not None, "the fused kernel declined a shape it should take"
    gu_ref = M._gemm_rows(a, w1, offsets, 2 * ffn, True)
    h_ref = swiglu_fwd_rows(gu_ref, limit)
    assert torch.equal(gu, gu_ref)
    assert same(h, h_ref)
    dgu = M._gemm_dswiglu_rows(gy, w2, gu_ref, offsets, limit)
    assert dgu is not None
    dh_ref = M._gemm_rows(gy, w2, offsets, ffn, False)
    dgu_ref = swiglu_bwd_rows(gu_ref, dh_ref, limit)
    assert same(dgu, dgu_ref)
    # and against the oracle in fp32
    ref32 = O.swiglu(O.grouped_gemm(a.cpu().float(), w1.cpu().float(), torch.tensor(sizes), trans_b=True), limit)
    assert rel_l2(h, ref32) <= 1e-2


def test_fused_swiglu_declines_small_or_odd_shapes():
    dev = torch.device(DEV)
    a = torch.randn(64, 40, device=dev).bfloat16()
    w1 = torch.randn(2, 48, 40, device=dev).bfloat16()
    offsets = M._group_offsets(torch.tensor([30, 34]), dev)
    assert M._gemm_swiglu_rows(a, w1, offsets, None) == (None, None)  # fewer than 4096 rows, k % 32 != 0


# ----- wgrad added straight into an fp32 accumulator -------------------------------------------
def test_wgrad_accumulates_into_fp32_buffer():
    gen = torch.Generator().manual_seed(4)
    sizes = [700, 0, 1300, 33]
    m, E, P, Q = sum(sizes), len(sizes), 256, 384
    x = torch.randn(m, P, generator=gen).bfloat16().to(DEV)
    y = torch.randn(m, Q, generator=gen).bfloat16().to(DEV)
    offsets = M._group_offsets(torch.tensor(sizes), torch.device(DEV))
    accum = torch.randn(E, P, Q, generator=gen).to(DEV)
    before = accum.clone()
    from steptronoss_amd._lib import dtype_code, ptr, stream, try_call

    ok = try_call("stm_grouped_gemm_wgrad_accum", ptr(x), ptr(y), ptr(accum), ptr(offsets), E, m, P, Q,
                  dtype_code(x.dtype), stream())  # fmt: skip
    assert ok
    _, ref = O.grouped_gemm_grads(x.cpu().float(), torch.zeros(E, P, Q), torch.tensor(sizes), False, y.cpu().float())
    assert rel_l2(accum - before, ref) <= 1e-5  # fp32 all the way: no 16-bit rounding of the gradient
    assert torch.equal(accum[1], before[1])  # the empty group adds nothing
    # a second call keeps adding
    try_call("stm_grouped_gemm_wgrad_accum", ptr(x), ptr(y), ptr(accum), ptr(offsets), E, m, P, Q,
             dtype_code(x.dtype), stream())  # fmt: skip
    assert rel_l2(accum - before, 2 * ref) <= 1e-5


def test_routed_ffn_can_accumulate_weight_grads_into_main_grad():
    from steptronoss_amd.model.common.feed_forward import swiglu

    gen = torch.Generator().manual_seed(6)
    T, H, E, K, F = 1024, 256, 4, 4, 256
    x = torch.randn(T, H, generator=gen).bfloat16().to(DEV)
    w1 = (torch.randn(E, 2 * F, H, generator=gen) * 0.05).bfloat16().to(DEV).requires_grad_(True)
    w2 = (torch.randn(E, H, F, generator=gen) * 0.05).bfloat16().to(DEV).requires_grad_(True)
    ids = torch.stack([torch.randperm(E, generator=gen)[:K] for _ in range(T)]).to(DEV)
    tw = torch.rand(T, K, generator=gen).to(DEV)
    go = torch.randn(T, H, generator=gen).bfloat16().to(DEV)
    M.routed_grouped_ffn(w1, w2, swiglu, x, ids, tw).backward(go)
    g1, g2 = w1.grad.clone(), w2.grad.clone()
    w1.grad = w2.grad = None
    w1.main_grad = torch.ones(w1.shape, device=DEV)
    w2.main_grad = torch.ones(w2.shape, device=DEV)
    old = M.settings.fuse_main_grad
    try:
        M.settings.fuse_main_grad = True
        M.routed_grouped_ffn(w1, w2, swiglu, x, ids, tw).backward(go)
    finally:
        M.settings.fuse_main_grad = old
    assert w1.grad is None and w2.grad is None  # nothing left for autograd to add
    assert rel_l2(w1.main_grad - 1, g1.float()) <= 1e-2
    assert rel_l2(w2.main_grad - 1, g2.float()) <= 1e-2
