"""Pins the CPU oracle: the reference's own known-answer tests (restated as data) plus
checks chosen so that a dropped term, wrong sign/index or transposed operand fails."""

import math

import pytest
import torch

from oracle import moe_oracle as O


# ----- histogram: reference tests/test_moe_utils.py:14-36 -------------------------------
def test_histogram_kats():
    out = O.histogram(torch.tensor([0, 1, 1, 3, 3, 3], dtype=torch.int64), 4)
    assert out.dtype == torch.int32 and out.tolist() == [1, 2, 0, 3]
    assert O.histogram(torch.tensor([], dtype=torch.int32), 3).tolist() == [0, 0, 0]
    assert O.histogram(torch.tensor([0, -1, 2, -3, 2], dtype=torch.int64), 4).tolist() == [1, 0, 2, 0]
    with pytest.raises(ValueError, match="out-of-range"):
        O.histogram(torch.tensor([0, 2], dtype=torch.int64), 2)


# ----- index_compute: reference tests/test_moe_utils.py:39-58 ---------------------------
def test_index_compute_kats():
    out = O.index_compute(torch.tensor([[0, 1], [1, 0], [0, 1]]), torch.tensor([3, 3], dtype=torch.int32))
    assert out.dtype == torch.int32 and out.tolist() == [[0, 3], [4, 1], [2, 5]]
    out = O.index_compute(torch.tensor([[0, -1], [1, -2], [0, 1]]), torch.tensor([2, 2], dtype=torch.int32))
    assert out.tolist() == [[0, -1], [2, -2], [1, 3]]
    with pytest.raises(AssertionError, match="expert_histogram does not match"):
        O.index_compute(torch.tensor([[0, 1], [1, -1]]), torch.tensor([1, 1], dtype=torch.int32))


@pytest.mark.parametrize("seed", range(4))
def test_index_compute_bruteforce_and_invariants(seed):
    g = torch.Generator().manual_seed(seed)
    T, K, E = 37, 3, 5
    ids = torch.randint(0, E, (T, K), generator=g)
    ids[torch.rand(T, K, generator=g) < 0.2] = -1
    hist = O.histogram(ids, E)
    pos = O.index_compute(ids, hist)
    assert torch.equal(pos, O.index_compute_bruteforce(ids, hist))
    valid = ids >= 0
    assert sorted(pos[valid].tolist()) == list(range(int(valid.sum())))
    # experts are non-decreasing along the output order
    order = torch.argsort(pos[valid])
    e_sorted = ids[valid][order]
    assert bool((e_sorted[1:] >= e_sorted[:-1]).all())
    assert torch.equal(pos[~valid].long(), ids[~valid])


# ----- combine: reference tests/test_moe_utils.py:61-101 -------------------------------
X3 = [[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]]


def test_combine_kats():
    x = torch.tensor(X3)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]])
    out = O.moe_weighted_gather(x, torch.tensor([[2, 0], [1, 2]]), w)
    assert torch.allclose(out, torch.tensor([[1.8, 2.8], [5.5, 7.0]]))
    out = O.moe_weighted_gather(x, torch.tensor([[2, -1], [1, -2]]), w)
    assert torch.allclose(out, torch.tensor([[1.0, 1.2], [3.0, 4.0]]))


def test_combine_grad_kats():
    x = torch.tensor(X3, requires_grad=True)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]], requires_grad=True)
    O.moe_weighted_gather(x, torch.tensor([[2, 0], [1, 2]]), w).sum().backward()
    assert torch.allclose(x.grad, torch.tensor([[0.8, 0.8], [1.0, 1.0], [0.7, 0.7]]))
    assert torch.allclose(w.grad, torch.tensor([[11.0, 3.0], [7.0, 11.0]]))
    x = torch.tensor(X3, requires_grad=True)
    w = torch.tensor([[0.2, 0.8], [1.0, 0.5]], requires_grad=True)
    O.moe_weighted_gather(x, torch.tensor([[2, -1], [1, -2]]), w).sum().backward()
    assert torch.allclose(x.grad, torch.tensor([[0.0, 0.0], [1.0, 1.0], [0.2, 0.2]]))
    assert torch.allclose(w.grad, torch.tensor([[11.0, 0.0], [7.0, 0.0]]))


# ----- permute: reference tests/test_moe_utils.py:104-155 ------------------------------
def test_permute_kats():
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    out = O.moe_scatter(x, torch.tensor([[0, 2], [1, 3]]))
    assert out.tolist() == [[1.0, 2.0], [3.0, 4.0], [1.0, 2.0], [3.0, 4.0]]
    out = O.moe_scatter(x, torch.tensor([[0, -1], [1, -2]]))
    assert out.tolist() == [[1.0, 2.0], [3.0, 4.0]]
    xg = x.clone().requires_grad_(True)
    O.moe_scatter(xg, torch.tensor([[0, 2], [1, 3]])).sum().backward()
    assert xg.grad.tolist() == [[2.0, 2.0], [2.0, 2.0]]
    xg = x.clone().requires_grad_(True)
    O.moe_scatter(xg, torch.tensor([[0, -1], [1, -2]])).sum().backward()
    assert xg.grad.tolist() == [[1.0, 1.0], [1.0, 1.0]]


def test_permute_combine_round_trip():
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    idx = torch.tensor([[0, 1, 2], [3, 4, 5]])
    back = O.moe_weighted_gather(O.moe_scatter(x, idx), idx, torch.ones(2, 3))
    assert torch.allclose(back, x * 3)
    idx = torch.tensor([[0, -1, 1], [2, -2, 3]])
    back = O.moe_weighted_gather(O.moe_scatter(x, idx), idx, torch.ones(2, 3))
    assert torch.allclose(back, x * (idx >= 0).sum(1, keepdim=True))


def test_permute_backward_is_a_weighted_row_sum():
    # a non-constant upstream gradient: a constant one hides which row goes where
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 4, generator=g, requires_grad=True)
    ids = torch.tensor([[0, 1], [1, 2], [2, 0], [0, -1], [1, 1]])
    pos = O.index_compute(ids, O.histogram(ids, 3))
    out = O.moe_scatter(x, pos)
    go = torch.randn(out.shape, generator=g)
    out.backward(go)
    expect = torch.zeros(5, 4)
    for t in range(5):
        for k in range(2):
            if pos[t, k] >= 0:
                expect[t] += go[pos[t, k]]
    assert torch.allclose(x.grad, expect)


# ----- grouped GEMM: reference tests/test_grouped_gemm.py ------------------------------
@pytest.mark.parametrize("trans_b", [False, True])
def test_grouped_gemm_is_block_diagonal_matmul(trans_b):
    g = torch.Generator().manual_seed(1)
    sizes = torch.tensor([3, 1, 0, 4])
    k, n = 8, 6
    a = torch.randn(8, k, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(4, n, k, generator=g, dtype=torch.float64) if trans_b else torch.randn(4, k, n, generator=g, dtype=torch.float64)
    b.requires_grad_(True)
    out = O.grouped_gemm(a, b, sizes, trans_b)
    # independent statement: one dense matmul against a [G*k, n] stack, rows masked by group
    stack = (b.transpose(1, 2) if trans_b else b).reshape(4 * k, n)
    a_wide = torch.zeros(8, 4 * k, dtype=torch.float64)
    row = 0
    for gi, m in enumerate(sizes.tolist()):
        a_wide[row : row + m, gi * k : (gi + 1) * k] = a.detach()[row : row + m]
        row += m
    assert torch.allclose(out, a_wide @ stack.detach())
    go = torch.randn(out.shape, generator=g, dtype=torch.float64)
    out.backward(go)
    ga, gb = O.grouped_gemm_grads(a.detach(), b.detach(), sizes, trans_b, go)
    assert torch.allclose(a.grad, ga) and torch.allclose(b.grad, gb)
    assert float(gb[2].abs().max()) == 0.0  # empty group => zero weight gradient


def test_swiglu_closed_form():
    x = torch.tensor([[1.0, -2.0, 0.5, 3.0], [10.0, 0.0, -8.0, 2.0]])
    out = O.swiglu(x)
    for r in range(2):
        for c in range(2):
            gate, up = float(x[r, c]), float(x[r, c + 2])
            assert math.isclose(float(out[r, c]), gate / (1 + math.exp(-gate)) * up, rel_tol=1e-6, abs_tol=1e-7)
    lim = O.swiglu(x, swiglu_limit=1.5)
    assert math.isclose(float(lim[1, 0]), 1.5 * -1.5, rel_tol=1e-6)  # silu(10) -> 1.5, up -8 -> -1.5
    assert math.isclose(float(lim[0, 1]), (-2 / (1 + math.exp(2))) * 1.5, rel_tol=1e-6)  # gate not clamped from below


def test_routed_grouped_ffn_matches_dense_formulation():
    g = torch.Generator().manual_seed(2)
    T, H, E, K, F = 23, 8, 4, 2, 6
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    w1 = torch.randn(E, 2 * F, H, generator=g, dtype=torch.float64)
    w2 = torch.randn(E, H, F, generator=g, dtype=torch.float64)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    ids[3, 1] = -1
    tw = torch.rand(T, K, generator=g, dtype=torch.float64).float()
    out = O.routed_grouped_ffn(w1, w2, O.swiglu, x, ids, tw)
    dense = O.routed_grouped_ffn_dense(w1, w2, O.swiglu, x, ids, tw)
    assert torch.allclose(out, dense, rtol=1e-5, atol=1e-5)  # fp32 weights => fp32 accumulation
    # nothing routed: the reference's early-out
    none = O.routed_grouped_ffn(w1, w2, O.swiglu, x, torch.full((T, K), -1), tw)
    assert torch.allclose(none, x * tw.sum())


# ----- router ------------------------------------------------------------------------------
@pytest.mark.parametrize("use_sigmoid,norm,bias", [(False, True, False), (False, False, False), (True, True, False), (True, True, True)])
def test_router_matches_python_loops(use_sigmoid, norm, bias):
    g = torch.Generator().manual_seed(3)
    T, E, K = 19, 12, 4
    logits = torch.randn(T, E, generator=g)
    logits[0] = 0.25  # full tie
    logits[1, 3] = logits[1, 7]  # partial tie
    bb = torch.randn(E, generator=g) * 0.1 if bias else None
    ids, w, aux, hist = O.forward_router(logits, K, use_sigmoid=use_sigmoid, norm_expert_weight=norm, balance_bias=bb)
    ids2, w2, aux2, hist2 = O.forward_router_bruteforce(logits, K, use_sigmoid=use_sigmoid, norm_expert_weight=norm, balance_bias=bb)
    assert torch.equal(ids, ids2) and torch.equal(hist, hist2)
    assert torch.allclose(w.double(), w2, rtol=1e-5, atol=1e-7)
    assert math.isclose(float(aux), aux2, rel_tol=1e-5)
    if not bias:
        assert ids[0].tolist() == list(range(K))  # ties go to the lower expert id


def test_router_closed_forms():
    T, E, K = 16, 8, 2
    ids, w, aux, hist = O.forward_router(torch.zeros(T, E), K)
    assert ids.tolist() == [[0, 1]] * T and torch.allclose(w, torch.full((T, K), 0.5))
    assert math.isclose(float(aux), T * K, rel_tol=1e-6)  # me = 1/E, sum(hist) = T*K, times E
    # the stable rule differs from an unstable top-k: equal scores keep ascending ids
    ids, _, _, _ = O.forward_router(torch.tensor([[0.25, 0.5, 0.5, 0.25, 0.5]]).log(), 3, norm_expert_weight=False)
    assert ids.tolist() == [[1, 2, 4]]
    # softmax without renormalisation returns the raw probabilities
    logits = torch.tensor([[2.0, 1.0, 0.0, -1.0]])
    _, w, _, _ = O.forward_router(logits, 2, norm_expert_weight=False)
    assert torch.allclose(w, torch.softmax(logits, 1)[:, :2])


@pytest.mark.parametrize("use_sigmoid", [False, True])
def test_group_limited_router(use_sigmoid):
    g = torch.Generator().manual_seed(4)
    T, E, K = 17, 16, 4
    logits = torch.randn(T, E, generator=g)
    a = O.forward_router(logits, K, use_sigmoid=use_sigmoid, n_group=1, topk_group=1)
    b = O.forward_router(logits, K, use_sigmoid=use_sigmoid)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    ids, w, aux, hist = O.forward_router(logits, K, use_sigmoid=use_sigmoid, n_group=4, topk_group=2)
    ids2, w2, aux2, hist2 = O.forward_router_bruteforce(logits, K, use_sigmoid=use_sigmoid, n_group=4, topk_group=2)
    assert torch.equal(ids, ids2) and torch.equal(hist, hist2)
    assert torch.allclose(w.double(), w2, rtol=1e-5)
    assert bool(((ids // 4).unsqueeze(2) == (ids // 4).unsqueeze(1)).sum((1, 2)).min() >= K)  # at most 2 groups used
    assert all(len(set((row // 4).tolist())) <= 2 for row in ids)


# ----- fp8 ---------------------------------------------------------------------------------
def test_e4m3_table_and_rounding():
    table = O.e4m3_decode_table()
    assert float(table[0x7E]) == 448.0 and float(table[0x01]) == 2.0**-9 and float(table[0x38]) == 1.0
    assert math.isnan(float(table[0x7F])) and math.isnan(float(table[0xFF]))
    native = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    ok = ~torch.isnan(table)
    assert torch.equal(native[ok], table[ok])
    # every representable value round-trips, midpoints go to even, overflow saturates
    codes = torch.arange(256, dtype=torch.uint8)[ok]
    assert torch.equal(O.e4m3_round(table[ok]), codes)
    assert O.e4m3_round(torch.tensor([1e6, -1e6])).tolist() == [0x7E, 0xFE]
    assert O.e4m3_round(torch.tensor([1.0625])).tolist() == [0x38]  # tie between 1.0 and 1.125 -> even mantissa
    assert O.e4m3_round(torch.tensor([1.1875])).tolist() == [0x3A]  # tie between 1.125 and 1.25 -> even mantissa
    x = torch.randn(1000, generator=torch.Generator().manual_seed(5)) * 20
    assert torch.equal(O.e4m3_round(x), x.clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8))


def test_quantize_1x128_round_trip():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(7, 300, generator=g)
    x[2, 128:256] = 0
    q, s = O.quantize_e4m3_1x128(x)
    assert q.shape == (7, 300) and s.shape == (7, 3) and float(s[2, 1]) == 1.0
    back = O.dequantize_e4m3_1x128(q, s)
    # 3 mantissa bits: relative error <= 2^-4 of the block maximum
    blk_max = torch.nn.functional.pad(x, (0, 84)).reshape(7, 3, 128).abs().amax(2).repeat_interleave(128, 1)[:, :300]
    assert bool(((back - x).abs() <= blk_max * 2.0**-4 + 1e-12).all())
    assert float((back - x).norm() / x.norm()) < 0.04


def test_quantize_1x128_power_of_two_scales():
    # hand-worked blocks: the scale is the smallest power of two >= amax / 448, never below 2^-126
    x = torch.zeros(5, 128)
    x[0, 0], x[1, 7], x[2, 3], x[3, 100] = 448.0, -449.0, 3.0, 1e-40
    q, s = O.quantize_e4m3_1x128(x, pow2=True)
    assert s.flatten().tolist() == [1.0, 2.0, 2.0**-7, 2.0**-126, 1.0]
    assert int(q[0, 0]) == 0x7E and int(q[1, 7]) == 0xF6  # 448 -> largest code; -449/2 = -224.5 -> -224 (1.75 * 2^7)
    assert int(q[2, 3]) == 0x7C  # 3 * 128 = 384 = 1.5 * 2^8
    # against the plain form: never a smaller scale, less than twice as large, same decoded values to 2^-3 relative
    g = torch.Generator().manual_seed(8)
    y = torch.randn(9, 384, generator=g) * torch.logspace(-3, 2, 9).unsqueeze(1)
    _, s_plain = O.quantize_e4m3_1x128(y)
    q2, s2 = O.quantize_e4m3_1x128(y, pow2=True)
    assert bool((s2 >= s_plain).all()) and bool((s2 < 2 * s_plain).all())
    mant, _ = torch.frexp(s2)
    assert bool((mant == 0.5).all())
    back = O.dequantize_e4m3_1x128(q2, s2)
    assert float((back - y).norm() / y.norm()) < 0.045


# ----- TE-style helpers: reference tests/test_permute_utils.py -------------------------
def _mask_expected(routing_map):
    T, E = routing_map.shape
    tok, rid = [], []
    for e in range(E):
        for t in range(T):
            if routing_map[t, e]:
                tok.append(t)
                rid.append(e * T + t)
    return torch.tensor(tok), torch.tensor(rid)


def test_te_permute_mask_roundtrip_and_padding():
    tokens = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]])
    rm = torch.tensor([[1, 0, 1, 0], [0, 1, 0, 0], [1, 0, 0, 1]], dtype=torch.bool)
    probs = torch.tensor([[0.6, 0.0, 0.4, 0.0], [0.0, 1.0, 0.0, 0.0], [0.5, 0.0, 0.0, 0.5]])
    out, rid, pp = O.moe_permute(tokens, rm, probs=probs)
    tok, exp_rid = _mask_expected(rm)
    assert torch.equal(rid, exp_rid) and torch.equal(out, tokens[tok])
    assert torch.allclose(pp, probs.t().reshape(-1)[exp_rid])
    assert torch.allclose(O.moe_unpermute(out, rid, merging_probs=probs, restore_shape=tokens.shape), tokens)
    out, rid, _ = O.moe_permute(tokens, rm, num_out_tokens=tok.numel() + 2)
    assert out.shape[0] == tok.numel() + 2 and rid[-2:].tolist() == [-1, -1] and float(out[-2:].abs().sum()) == 0
    assert torch.allclose(O.moe_unpermute(out, rid, merging_probs=probs, restore_shape=tokens.shape), tokens)


def test_te_permute_index_roundtrip_and_chunks():
    tokens = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]])
    rm = torch.tensor([[1, 0], [0, 2], [2, -1]])
    probs = torch.tensor([[0.6, 0.4], [0.5, 0.5], [1.0, 0.0]])
    out, rid = O.moe_permute(tokens, rm, map_type="index")
    assert rid.tolist() == [1, 2, 0, 3, 4]  # slots sorted by (expert, flat position)
    assert torch.equal(out, tokens[rid // 2])
    back = O.moe_unpermute(out, rid, merging_probs=probs, restore_shape=tokens.shape, map_type="index")
    assert torch.allclose(back, tokens)
    inp = torch.arange(12, dtype=torch.float32).view(6, 2)
    got = O.moe_sort_chunks_by_index(inp, torch.tensor([2, 1, 3]), torch.tensor([2, 0, 1]))
    assert torch.equal(got, torch.cat([inp[3:6], inp[0:2], inp[2:3]]))
    got, gp = O.moe_sort_chunks_by_index(inp, torch.tensor([2, 1, 3]), torch.tensor([2, 0, 1]), probs=torch.arange(6.0))
    assert gp.tolist() == [3.0, 4.0, 5.0, 0.0, 1.0, 2.0]


# ----- aux-loss-free balance bias: reference moe_block.py:470-478 -----------------------------
def test_balance_bias_update_closed_form():
    tokens = torch.tensor([10, 0, 5, 5])  # mean 5: over, under, at the mean twice
    bias = torch.tensor([0.5, -0.25, 0.0, 1.0])
    out = O.update_router_balance_bias(tokens, bias, 0.125)
    assert torch.equal(out, torch.tensor([0.375, -0.125, 0.0, 1.0]))
    # the update never changes the sum when loads are symmetric about the mean
    assert float(O.update_router_balance_bias(torch.tensor([3, 1]), torch.zeros(2), 1.0).sum()) == 0.0


def test_router_force_balance_rule():
    # reference moe_block.py:249-256: round-robin ids over the flat slots, equal counts when E divides T*K
    logits = torch.randn(12, 6, generator=torch.Generator().manual_seed(0))
    ids, w, aux, hist = O.forward_router(logits, 3, force_balance=True)
    assert ids.flatten().tolist() == [i % 6 for i in range(36)] and hist.tolist() == [6] * 6
    prob = torch.softmax(logits, 1)
    assert torch.allclose(w, prob.gather(1, ids) / prob.gather(1, ids).sum(1, keepdim=True))
    assert abs(float(aux) - 36.0) < 1e-4  # sum_e mean_t(p) * 6 * E = 6 * 6 * sum_e mean_t p = 36
    with pytest.raises(ValueError):
        O.forward_router(logits, 7, force_balance=True)
