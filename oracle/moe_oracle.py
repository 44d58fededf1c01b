"""CPU oracle for the MoE-layer hot path (router -> permute -> grouped FFN -> unpermute).

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a from-scratch restatement,
in plain PyTorch CPU ops, of what the reference computes on this path.  Only the
test-suite, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import it; nothing under ``steptronoss_amd/`` does.

Every public function names the reference lines whose behaviour it restates
(paths relative to the reference checkout).  How each one is pinned:

=====================  ==========================================================
function               pinned by
=====================  ==========================================================
histogram              reference KATs (tests/test_moe_utils.py:14-36)
index_compute          reference KATs (tests/test_moe_utils.py:39-58) +
                       O(N^2) brute force ``index_compute_bruteforce``
moe_scatter            reference KATs incl. explicit grads (:104-134), round trip
                       (:137-155)
moe_weighted_gather    reference KATs incl. explicit grads (:61-101)
grouped_gemm           per-group dense matmul (tests/test_grouped_gemm.py:9-19),
                       block-diagonal dense-matmul identity, autograd
swiglu                 closed form x*sigmoid(x)*y, scalar python loop
routed_grouped_ffn     dense "every token through every expert, masked" identity
forward_router         pure-python per-token loop ``forward_router_bruteforce``,
                       closed forms (all-equal logits, one-hot logits)
group-limited top-k    PARITY UNPINNED AGAINST THE REFERENCE (it has no such
                       routing); reduction n_group=1 => forward_router, python loop
fp8 e4m3 quantiser     PARITY UNPINNED AGAINST THE REFERENCE (it has no fp8 MoE
                       path); exhaustive 256-code decode table, round trip,
                       saturation; the power-of-two scale form by hand-worked
                       blocks (amax 448 -> 1, 449 -> 2, 3 -> 2^-7, tiny -> 2^-126)
TE-style permute       brute-force expectations of tests/test_permute_utils.py
update_router_balance  closed form on a hand-worked vector (over / under / at the
_bias                  mean), sign symmetry
=====================  ==========================================================

The reference's literal test vectors are also kept as data in
``tests/golden/reference_kats.json`` and run against these functions.
"""

from __future__ import annotations

import math

import torch

# --------------------------------------------------------------------------- #
# a3  histogram                     steptronoss/model/utils/moe_utils.py:90-129
# --------------------------------------------------------------------------- #


def histogram(top_k_rank: torch.Tensor, expert_num: int) -> torch.Tensor:
    """Per-expert count of non-negative ids, int32 ``[expert_num]``.

    Restates moe_utils.py:90-129: negative ids are ignored, an id ``>= expert_num``
    is a ``ValueError`` ("out-of-range"), empty input gives zeros.
    """
    if not isinstance(top_k_rank, torch.Tensor):
        raise TypeError("top_k_rank must be a torch.Tensor")
    if top_k_rank.dtype not in (torch.int32, torch.int64):
        raise TypeError("top_k_rank must be int32 or int64 tensor")
    if expert_num < 0:
        raise ValueError("expert_num must be non-negative")
    counts = torch.zeros(expert_num, dtype=torch.int32, device=top_k_rank.device)
    if expert_num == 0 or top_k_rank.numel() == 0:
        return counts
    ids = top_k_rank.reshape(-1).to(torch.int64)
    ids = ids[ids >= 0]
    if ids.numel() and int(ids.max()) >= expert_num:
        raise ValueError("top_k_rank contains out-of-range expert index")
    return torch.bincount(ids, minlength=expert_num).to(torch.int32)


# --------------------------------------------------------------------------- #
# a4  index_compute                 steptronoss/model/utils/moe_utils.py:137-214
# --------------------------------------------------------------------------- #


def index_compute(indices: torch.Tensor, expert_histogram: torch.Tensor) -> torch.Tensor:
    """Stable counting-sort position of every (token, k) slot, int32 ``[T, K]``.

    ``pos(t,k) = base[e] + #{earlier flat slots routed to e}`` with
    ``base = exclusive_cumsum(expert_histogram)`` and flat order token-major,
    k-minor; negative entries are passed through unchanged
    (moe_utils.py:137-214).  Mismatching histogram -> ``AssertionError``.
    """
    if not isinstance(indices, torch.Tensor):
        raise TypeError("indices must be a torch.Tensor")
    if not isinstance(expert_histogram, torch.Tensor):
        raise TypeError("expert_histogram must be a torch.Tensor")
    if indices.dtype not in (torch.int32, torch.int64):
        raise TypeError("indices must be int32 or int64 tensor")
    if expert_histogram.dtype not in (torch.int32, torch.int64):
        raise TypeError("expert_histogram must be int32 or int64 tensor")
    if indices.dim() != 2:
        raise ValueError("indices must be 2D [token_num, top_k]")
    if expert_histogram.dim() != 1:
        raise ValueError("expert_histogram must be 1D [num_experts]")
    if indices.device != expert_histogram.device:
        raise ValueError("indices and expert_histogram must be on the same device")

    out = indices.to(torch.int32, copy=True)
    if indices.numel() == 0:
        return out
    num_experts = expert_histogram.numel()
    flat = indices.reshape(-1).to(torch.int64)
    valid = flat >= 0
    n_valid = int(valid.sum())
    if n_valid:
        assert int(flat[valid].max()) < num_experts, "indices contains out-of-range expert index"
    assert not bool((expert_histogram < 0).any()), "expert_histogram must be non-negative"
    assert int(expert_histogram.sum()) == n_valid, "expert_histogram does not match number of valid indices"
    if n_valid == 0:
        return out

    hist = expert_histogram.to(torch.int64)
    base = torch.cumsum(hist, 0) - hist
    # Stable sort by expert id keeps the flat order inside each expert.
    slot = torch.nonzero(valid).reshape(-1)
    expert_of_slot = flat[slot]
    order = torch.sort(expert_of_slot, stable=True).indices
    sorted_expert = expert_of_slot[order]
    actual = torch.bincount(expert_of_slot, minlength=num_experts)
    first_rank = torch.cumsum(actual, 0) - actual
    rank = torch.arange(n_valid, dtype=torch.int64)
    pos_sorted = base[sorted_expert] + (rank - first_rank[sorted_expert])
    flat_out = out.reshape(-1)
    flat_out[slot[order]] = pos_sorted.to(torch.int32)
    return out


def index_compute_bruteforce(indices, expert_histogram):
    """O(N^2) pure-python statement of the same definition (tiny inputs only)."""
    T, K = indices.shape
    flat = [int(v) for v in indices.reshape(-1).tolist()]
    hist = [int(v) for v in expert_histogram.tolist()]
    base = [sum(hist[:e]) for e in range(len(hist))]
    out = []
    for i, e in enumerate(flat):
        if e < 0:
            out.append(e)
        else:
            out.append(base[e] + sum(1 for j in range(i) if flat[j] == e))
    return torch.tensor(out, dtype=torch.int32).reshape(T, K)


# --------------------------------------------------------------------------- #
# a5  moe_scatter (= permute)       steptronoss/model/utils/moe_utils.py:337-420
# --------------------------------------------------------------------------- #


class _Permute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, index):
        T, K = index.shape
        flat = index.reshape(-1).to(torch.int64)
        valid = flat >= 0
        n_out = int(valid.sum())
        out = x.new_zeros((n_out, x.shape[1]))
        token_of_slot = torch.arange(T, device=x.device).repeat_interleave(K)
        if n_out:
            out[flat[valid]] = x[token_of_slot[valid]]
        ctx.save_for_backward(flat, valid, token_of_slot)
        ctx.T = T
        return out

    @staticmethod
    def backward(ctx, go):
        flat, valid, token_of_slot = ctx.saved_tensors
        # Sum over a token's valid slots in fp32, round once to the gradient dtype
        # (what a dtype-preserving torch ``sum(dim=1)`` does, moe_utils.py:386-397).
        acc = torch.zeros((ctx.T, go.shape[1]), dtype=torch.float32, device=go.device)
        if go.numel() and bool(valid.any()):
            acc.index_add_(0, token_of_slot[valid], go[flat[valid]].float())
        return acc.to(go.dtype), None


def moe_scatter(input: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """``out[index[t,k], :] = input[t, :]`` for non-negative entries; ``out`` has
    one row per non-negative entry and starts from zeros (moe_utils.py:337-420)."""
    if index.dtype not in (torch.int32, torch.int64):
        raise TypeError("index must be int32 or int64 tensor")
    if index.dim() != 2:
        raise ValueError("index must be 2D [token_num, top_k]")
    if input.dim() != 2:
        raise ValueError("input must be 2D [token_num, hidden_dim]")
    if input.shape[0] != index.shape[0]:
        raise ValueError("input and index must have the same token_num")
    return _Permute.apply(input, index)


# --------------------------------------------------------------------------- #
# a8  moe_weighted_gather (= unpermute / combine)     moe_utils.py:247-334
# --------------------------------------------------------------------------- #


class _Combine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp, index, weight):
        T, K = index.shape
        H = inp.shape[-1]
        flat = index.reshape(-1).to(torch.int64)
        valid = flat >= 0
        # accumulate in fp32 iff the weights are fp32, else in the row dtype (:274)
        acc_dtype = torch.float32 if weight.dtype == torch.float32 else inp.dtype
        rows = inp[flat.clamp_min(0)].to(acc_dtype)
        rows = rows * valid.to(acc_dtype).unsqueeze(1)
        prod = rows * weight.reshape(-1, 1).to(acc_dtype)
        out = prod.reshape(T, K, H).sum(1).to(inp.dtype)
        ctx.save_for_backward(inp, index, weight)
        return out

    @staticmethod
    def backward(ctx, go):
        inp, index, weight = ctx.saved_tensors
        T, K = index.shape
        H = inp.shape[-1]
        flat = index.reshape(-1).to(torch.int64)
        valid = flat >= 0
        rows = inp[flat.clamp_min(0)].reshape(T, K, H) * valid.reshape(T, K, 1).to(inp.dtype)
        gw = (go.unsqueeze(1) * rows).sum(2).to(weight.dtype)
        contrib = go.unsqueeze(1) * weight.to(go.dtype).unsqueeze(2)
        contrib = (contrib.reshape(T * K, H) * valid.to(go.dtype).unsqueeze(1)).to(inp.dtype)
        gin = torch.zeros_like(inp)
        gin.index_add_(0, flat.clamp_min(0), contrib)
        return gin, None, gw


def moe_weighted_gather(input: torch.Tensor, index: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``out[t,:] = sum_k weight[t,k] * input[index[t,k], :]`` over non-negative
    entries; backward gives ``d input`` (index_add of ``go*w``) and ``d weight``
    (row dot products) (moe_utils.py:247-334)."""
    if index.dtype not in (torch.int32, torch.int64):
        raise TypeError("index must be int32 or int64 tensor")
    if weight.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError("weight must be a floating tensor")
    if index.dim() != 2 or weight.dim() != 2:
        raise ValueError("index and weight must be 2D [token_num, top_k]")
    if weight.shape != index.shape:
        raise ValueError("index and weight must have the same shape")
    return _Combine.apply(input, index, weight)


# --------------------------------------------------------------------------- #
# a6  grouped_gemm      moe_utils.py:443-453; optimizations/grouped_gemm/function_imple.py:6-75
# --------------------------------------------------------------------------- #


def grouped_gemm(mat_a_flat, mat_b, batch_sizes, trans_b=False):
    """Rows ``[s_g, s_g+m_g)`` of ``mat_a_flat`` times ``mat_b[g]`` (transposed when
    ``trans_b``), concatenated.  Differentiable through plain autograd, which yields
    the dgrad / wgrad formulas of function_imple.py:54-69 (zero wgrad for an empty
    group)."""
    sizes = [int(v) for v in batch_sizes.tolist()]
    n_out = mat_b.shape[1] if trans_b else mat_b.shape[2]
    pieces = []
    row = 0
    for g, m in enumerate(sizes):
        rhs = mat_b[g].t() if trans_b else mat_b[g]
        pieces.append(mat_a_flat[row : row + m] @ rhs)
        row += m
    if not pieces:
        return mat_a_flat.new_zeros((0, n_out))
    return torch.cat(pieces, 0)


def grouped_gemm_grads(mat_a_flat, mat_b, batch_sizes, trans_b, grad_out):
    """Explicit dgrad / wgrad (function_imple.py:54-69), used to pin autograd."""
    sizes = [int(v) for v in batch_sizes.tolist()]
    ga = torch.zeros_like(mat_a_flat)
    gb = torch.zeros_like(mat_b)
    row = 0
    for g, m in enumerate(sizes):
        a = mat_a_flat[row : row + m]
        d = grad_out[row : row + m]
        if m:
            if trans_b:
                ga[row : row + m] = d @ mat_b[g]
                gb[g] = d.t() @ a
            else:
                ga[row : row + m] = d @ mat_b[g].t()
                gb[g] = a.t() @ d
        row += m
    return ga, gb


# --------------------------------------------------------------------------- #
# a7  SwiGLU                        steptronoss/model/common/feed_forward.py:20-26
# --------------------------------------------------------------------------- #


def swiglu(x: torch.Tensor, swiglu_limit=None) -> torch.Tensor:
    """``silu(x[..., :F]) * x[..., F:]`` with the optional clamp of
    feed_forward.py:23-25 (gate clamped from above after the SiLU, up clamped to
    ``[-limit, limit]``)."""
    F = x.shape[-1] // 2
    gate, up = x[..., :F], x[..., F:]
    gate = gate * torch.sigmoid(gate)
    if swiglu_limit is not None:
        gate = torch.clamp(gate, max=swiglu_limit)
        up = torch.clamp(up, min=-swiglu_limit, max=swiglu_limit)
    return gate * up


# --------------------------------------------------------------------------- #
# a9  routed_grouped_ffn            steptronoss/model/utils/moe_utils.py:222-244
# --------------------------------------------------------------------------- #


def routed_grouped_ffn(w1, w2, act, x, token_expert_ids, token_weights):
    """histogram -> index_compute -> permute -> GEMM(w1^T) -> act -> GEMM(w2^T) ->
    weighted combine (moe_utils.py:222-244), with its "nothing routed" early-out."""
    hist = histogram(token_expert_ids, w1.shape[0])
    if hist.numel() == 0 or int(hist.sum()) == 0:
        return x * token_weights.sum()
    sizes = hist.to(torch.int64)
    pos = index_compute(token_expert_ids, hist)
    h = moe_scatter(x, pos)
    h = grouped_gemm(h, w1, sizes, trans_b=True)
    h = act(h)
    h = grouped_gemm(h, w2, sizes, trans_b=True)
    return moe_weighted_gather(h, pos, token_weights)


def routed_grouped_ffn_dense(w1, w2, act, x, token_expert_ids, token_weights):
    """Independent statement used to pin ``routed_grouped_ffn``: run every token
    through every expert and combine with a dense ``[T, E]`` weight matrix."""
    T = x.shape[0]
    E = w1.shape[0]
    dense_w = torch.zeros(T, E, dtype=torch.float64)
    for t in range(T):
        for k in range(token_expert_ids.shape[1]):
            e = int(token_expert_ids[t, k])
            if e >= 0:
                dense_w[t, e] += float(token_weights[t, k])
    out = torch.zeros(T, w2.shape[1], dtype=torch.float64)
    for e in range(E):
        y = act(x.double() @ w1[e].double().t()) @ w2[e].double().t()
        out += dense_w[:, e : e + 1] * y
    return out


# --------------------------------------------------------------------------- #
# a2  router                        steptronoss/model/common/moe_block.py:224-292
# --------------------------------------------------------------------------- #


def _stable_topk(scores: torch.Tensor, k: int):
    """First ``k`` columns of a stable descending sort: equal scores keep ascending
    column order, i.e. ties go to the lower id (moe_block.py:245-247)."""
    srt, idx = torch.sort(scores, dim=1, descending=True, stable=True)
    return srt[:, :k], idx[:, :k].contiguous()


def group_limited_scores(scores: torch.Tensor, n_group: int, topk_group: int) -> torch.Tensor:
    """Group-limited selection mask (DeepSeek-V3 form; NOT in the reference):
    experts are split into ``n_group`` contiguous groups, a group's score is the sum
    of its two largest member scores, the ``topk_group`` best groups (stable, ties to
    the lower group id) stay eligible, every other expert's score becomes ``-inf``."""
    if n_group <= 1:
        return scores
    T, E = scores.shape
    per = E // n_group
    g = scores.reshape(T, n_group, per)
    top2 = torch.sort(g, dim=2, descending=True, stable=True).values[:, :, : min(2, per)]
    gscore = top2.sum(2)
    _, keep = _stable_topk(gscore, topk_group)
    gmask = torch.zeros(T, n_group, dtype=torch.bool)
    gmask.scatter_(1, keep, True)
    emask = gmask.unsqueeze(2).expand(T, n_group, per).reshape(T, E)
    return scores.masked_fill(~emask, float("-inf"))


def forward_router(
    logits: torch.Tensor,
    top_k: int,
    *,
    use_sigmoid: bool = False,
    norm_expert_weight: bool = True,
    balance_bias: torch.Tensor | None = None,
    n_group: int = 1,
    topk_group: int = 1,
    force_balance: bool = False,
):
    """Router of moe_block.py:224-292 (single process: the TP/EP all-reduces of the
    count vector at :278-279 are identities).

    Returns ``(ids int64 [T,K], weights fp32 [T,K], aux_loss fp32 scalar,
    hist int32 [E])``.

    * scores = softmax(logits.float(), 1) or sigmoid                     (:229-232)
    * selection = stable descending sort of ``scores (+ balance_bias)``, first K
      (:235-247); weights are gathered from the un-biased scores
    * sigmoid: weights and scores are each divided by their row sum (+1e-20 iff a
      bias buffer exists) (:261-268); softmax: weights divided by their row sum iff
      ``norm_expert_weight`` (:269-272)
    * ``force_balance`` (debug switch, :249-256): the ids become ``arange(T*K) % E`` reshaped to
      ``[T, K]`` and the weights are gathered for those
    * ``aux = sum(mean(scores, 0) * hist) * E`` with ``hist`` the raw per-expert
      counts, which carries no gradient                                  (:274-292)
    """
    logits = logits.float()
    T, E = logits.shape
    prob = torch.sigmoid(logits) if use_sigmoid else torch.softmax(logits, dim=1)
    choice = prob if balance_bias is None else prob + balance_bias.float().unsqueeze(0)
    choice = group_limited_scores(choice, n_group, topk_group)
    _, ids = _stable_topk(choice, top_k)
    if force_balance:
        if top_k > E:
            raise ValueError("force_balance requires top_k <= num_experts")
        ids = (torch.arange(T * top_k, dtype=torch.int64) % E).view(T, top_k)
    topk_prob = prob.gather(1, ids)
    eps = 1e-20 if balance_bias is not None else 0.0
    weights = topk_prob
    if use_sigmoid:
        weights = weights / (weights.sum(-1, keepdim=True) + eps)
        prob = prob / (prob.sum(-1, keepdim=True) + eps)
    elif norm_expert_weight:
        weights = weights / (topk_prob.sum(-1, keepdim=True) + eps)
    hist = histogram(ids, E)
    me = prob.mean(0)
    aux = (me * hist).sum() * E
    return ids, weights, aux, hist


def forward_router_bruteforce(
    logits, top_k, *, use_sigmoid=False, norm_expert_weight=True, balance_bias=None, n_group=1, topk_group=1
):
    """Per-token python loops in float64; pins ``forward_router`` on tiny inputs."""
    T, E = logits.shape
    ids, weights = [], []
    colsum = [0.0] * E
    hist = [0] * E
    for t in range(T):
        row = [float(v) for v in logits[t].float().tolist()]
        if use_sigmoid:
            p = [1.0 / (1.0 + math.exp(-v)) for v in row]
        else:
            m = max(row)
            ex = [math.exp(v - m) for v in row]
            s = sum(ex)
            p = [v / s for v in ex]
        c = list(p) if balance_bias is None else [p[e] + float(balance_bias[e]) for e in range(E)]
        if n_group > 1:
            per = E // n_group
            gs = []
            for g in range(n_group):
                mem = sorted(c[g * per : (g + 1) * per], reverse=True)
                gs.append(sum(mem[:2]))
            keep = sorted(range(n_group), key=lambda g: (-gs[g], g))[:topk_group]
            c = [c[e] if (e // per) in keep else float("-inf") for e in range(E)]
        chosen = sorted(range(E), key=lambda e: (-c[e], e))[:top_k]
        w = [p[e] for e in chosen]
        eps = 1e-20 if balance_bias is not None else 0.0
        if use_sigmoid:
            sw = sum(w) + eps
            w = [v / sw for v in w]
            sp = sum(p) + eps
            p = [v / sp for v in p]
        elif norm_expert_weight:
            sw = sum(w) + eps
            w = [v / sw for v in w]
        for e in chosen:
            hist[e] += 1
        for e in range(E):
            colsum[e] += p[e]
        ids.append(chosen)
        weights.append(w)
    aux = sum(colsum[e] / T * hist[e] for e in range(E)) * E
    return (
        torch.tensor(ids, dtype=torch.int64),
        torch.tensor(weights, dtype=torch.float64),
        aux,
        torch.tensor(hist, dtype=torch.int32),
    )


# --------------------------------------------------------------------------- #
# a11 MoE layer body (single GPU)   steptronoss/model/common/moe_block.py:376-420
# --------------------------------------------------------------------------- #


class _BindAux(torch.autograd.Function):
    """Identity on ``out``; backward hands the aux loss a gradient of one
    (steptronoss/model/utils/utils.py:68-90)."""

    @staticmethod
    def forward(ctx, out, aux):
        ctx.save_for_backward(aux)
        return out.view_as(out)

    @staticmethod
    def backward(ctx, go):
        (aux,) = ctx.saved_tensors
        return go, torch.ones_like(aux)


def bind_aux_loss(out, aux):
    return _BindAux.apply(out, aux)


def moe_layer(
    x,
    logits,
    w1,
    w2,
    *,
    top_k,
    use_sigmoid=False,
    norm_expert_weight=True,
    aux_loss_coef=0.0,
    routed_scaling_factor=1.0,
    swiglu_limit=None,
    n_group=1,
    topk_group=1,
    balance_bias=None,
):
    """router -> routed grouped FFN -> bind aux -> scale (moe_block.py:376-420 with the
    gate matmul replaced by ready-made logits)."""
    ids, weights, aux, _ = forward_router(
        logits,
        top_k,
        use_sigmoid=use_sigmoid,
        norm_expert_weight=norm_expert_weight,
        balance_bias=balance_bias,
        n_group=n_group,
        topk_group=topk_group,
    )
    out = routed_grouped_ffn(w1, w2, lambda h: swiglu(h, swiglu_limit), x, ids, weights.to(torch.float32))
    out = bind_aux_loss(out, aux * aux_loss_coef)
    return out * routed_scaling_factor, ids, weights, aux


def update_router_balance_bias(tokens_per_expert: torch.Tensor, bias: torch.Tensor, update_rate: float) -> torch.Tensor:
    """moe_block.py:470-478 for one layer (after the reference's all-reduces, which are identities
    on one GPU): ``bias + sign(mean(tokens) - tokens) * rate`` in fp32."""
    t = tokens_per_expert.float()
    offset = t.mean(dim=-1, keepdim=True) - t
    return bias + torch.sign(offset) * update_rate


# --------------------------------------------------------------------------- #
# fp8 e4m3 (OCP "fn": no inf, max 448) with 1x128 block scales.  NOT in the reference.
# --------------------------------------------------------------------------- #

E4M3_MAX = 448.0


def e4m3_decode_table() -> torch.Tensor:
    """All 256 e4m3fn codes decoded by the format's definition (1-4-3, bias 7,
    subnormals at exponent 0, 0x7f/0xff = NaN)."""
    vals = []
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            vals.append(float("nan"))
        elif e == 0:
            vals.append(s * (m / 8.0) * 2.0**-6)
        else:
            vals.append(s * (1.0 + m / 8.0) * 2.0 ** (e - 7))
    return torch.tensor(vals, dtype=torch.float32)


def e4m3_round(x: torch.Tensor) -> torch.Tensor:
    """Round fp32 to the nearest e4m3fn value (ties to even), saturating at +-448;
    returns uint8 codes."""
    table = e4m3_decode_table()
    pos = table[:127].double()  # codes 0..126 are the non-negative finite values, ascending
    a = x.double().abs().clamp(max=E4M3_MAX)
    hi = torch.searchsorted(pos, a).clamp(max=126)
    lo = (hi - 1).clamp(min=0)
    d_hi = (pos[hi] - a).abs()
    d_lo = (a - pos[lo]).abs()
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = torch.where(pick_lo, lo, hi)
    code = torch.where(x < 0, code + 128, code)
    code = torch.where(torch.signbit(x) & (code == 0), torch.full_like(code, 128), code)
    return code.to(torch.uint8)


def quantize_e4m3_1x128(x: torch.Tensor, block: int = 128, pow2: bool = False):
    """Per-row, per-``block``-column scaling: ``scale = amax/448`` (1.0 for an all-zero
    block), codes = round_e4m3(x/scale).  Returns ``(codes uint8 [R,C], scales fp32
    [R, ceil(C/block)])``.  ``pow2``: the scale is raised to the next power of two (at least
    the smallest normal fp32), the form a block-scaled matrix instruction applies in hardware."""
    R, C = x.shape
    nb = (C + block - 1) // block
    xf = x.float()
    pad = nb * block - C
    if pad:
        xf = torch.nn.functional.pad(xf, (0, pad))
    xb = xf.reshape(R, nb, block)
    amax = xb.abs().amax(2)
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    if pow2:
        mant, expo = torch.frexp(scale)  # scale = mant * 2^expo, mant in [0.5, 1)
        expo = torch.where(mant == 0.5, expo - 1, expo).clamp(min=-126)
        scale = torch.ldexp(torch.ones_like(scale), expo)
    q = e4m3_round((xb / scale.unsqueeze(2)).reshape(R, nb * block))[:, :C]
    return q.contiguous(), scale


def dequantize_e4m3_1x128(codes: torch.Tensor, scale: torch.Tensor, block: int = 128) -> torch.Tensor:
    table = e4m3_decode_table()
    R, C = codes.shape
    vals = table[codes.long()]
    s = scale.repeat_interleave(block, dim=1)[:, :C]
    return vals * s


# --------------------------------------------------------------------------- #
# a12 TE-style permute helpers      steptronoss/model/utils/permute_utils.py
# --------------------------------------------------------------------------- #


def _fit_length(row_ids: torch.Tensor, num_out_tokens: int) -> torch.Tensor:
    """Trim, or pad with -1, to ``num_out_tokens`` when it is non-negative
    (permute_utils.py:16-29)."""
    if num_out_tokens < 0 or num_out_tokens == row_ids.numel():
        return row_ids
    if num_out_tokens < row_ids.numel():
        return row_ids[:num_out_tokens]
    pad = row_ids.new_full((num_out_tokens - row_ids.numel(),), -1)
    return torch.cat([row_ids, pad])


def _rows_by_token(inp, token_ids):
    out = inp.new_zeros((token_ids.numel(), inp.shape[1]))
    ok = token_ids >= 0
    if bool(ok.any()):
        out[ok] = inp[token_ids[ok]]
    return out


def moe_permute(inp, routing_map, num_out_tokens=-1, max_token_num=-1, map_type="mask", probs=None):
    """permute_utils.py:43-143.  ``mask``: ``routing_map`` bool ``[T,E]``, rows emitted
    expert-major with ``row_id = e*T + t``; ``index``: ``routing_map`` int ``[T,K]``, slots
    sorted by (expert, flat position), ``row_id`` = flat position."""
    if map_type not in ("mask", "index"):
        raise ValueError("map_type should be one of 'mask' or 'index'")
    if inp.numel() == 0:
        empty = torch.zeros(0, dtype=torch.long)
        if map_type == "mask":
            return inp, empty, (None if probs is None else probs.new_empty((0,)))
        return inp, empty
    T = routing_map.shape[0]
    if map_type == "mask":
        e_ids, t_ids = torch.nonzero(routing_map.to(torch.bool).t(), as_tuple=True)
        row_ids = _fit_length(e_ids * T + t_ids, num_out_tokens)
        tok = torch.where(row_ids >= 0, row_ids % T, row_ids)
        out = _rows_by_token(inp, tok)
        pp = None
        if probs is not None:
            flat_p = probs.t().contiguous().reshape(-1)
            pp = probs.new_zeros((row_ids.numel(),))
            ok = row_ids >= 0
            pp[ok] = flat_p[row_ids[ok]]
        return out, row_ids, pp
    K = routing_map.shape[1]
    flat = routing_map.reshape(-1).to(torch.long)
    slots = torch.nonzero(flat >= 0).reshape(-1)
    order = torch.sort(flat[slots], stable=True).indices
    row_ids = _fit_length(slots[order], num_out_tokens)
    tok = torch.where(row_ids >= 0, row_ids // K, row_ids)
    return _rows_by_token(inp, tok), row_ids


def moe_unpermute(inp, row_id_map, merging_probs=None, restore_shape=None, map_type="mask"):
    """permute_utils.py:157-234: scatter-add of (optionally prob-weighted) rows back to
    token order."""
    if inp.numel() == 0:
        return inp
    if map_type not in ("mask", "index"):
        raise ValueError("map_type should be one of 'mask' or 'index'")
    ok = row_id_map >= 0
    if map_type == "mask":
        if merging_probs is not None:
            T = merging_probs.shape[0]
        elif restore_shape is not None:
            T = restore_shape[0]
        else:
            raise ValueError("restore_shape or merging_probs must be provided for map_type='mask'.")
        flat_p = None if merging_probs is None else merging_probs.t().contiguous().reshape(-1)
        tok = row_id_map[ok] % T
    else:
        if merging_probs is not None:
            T, K = merging_probs.shape
        elif restore_shape is not None:
            T = restore_shape[0]
            K = (int(row_id_map[ok].max()) // max(T, 1) + 1) if bool(ok.any()) else 1
        else:
            T, K = row_id_map.shape[0], 1
        flat_p = None if merging_probs is None else merging_probs.reshape(-1)
        tok = row_id_map[ok] // K
    shape = tuple(restore_shape) if restore_shape is not None else (T, inp.shape[1])
    out = inp.new_zeros(shape)
    rows = inp[ok]
    if flat_p is not None:
        rows = rows * flat_p[row_id_map[ok]].unsqueeze(1)
    out.index_add_(0, tok, rows)
    return out


def moe_sort_chunks_by_index(inp, split_sizes, sorted_index, probs=None):
    """permute_utils.py:237-277: split rows by ``split_sizes``, emit chunks in
    ``sorted_index`` order."""
    if inp.numel() == 0:
        return inp if probs is None else (inp, probs)
    sizes = [int(v) for v in split_sizes.tolist()]
    starts = [sum(sizes[:i]) for i in range(len(sizes))]
    sel = [torch.arange(starts[i], starts[i] + sizes[i]) for i in sorted_index.tolist()]
    rows = torch.cat(sel) if sel else torch.zeros(0, dtype=torch.long)
    if probs is None:
        return inp[rows]
    return inp[rows], probs[rows]


# --------------------------------------------------------------------------- #
# Seeded synthetic inputs of the benchmark configurations (shared by tests/bench).
# --------------------------------------------------------------------------- #

CONFIGS = {
    # name: T, H, E, K, F, dtype, router
    "c1": dict(T=4096, H=1024, E=8, K=2, F=2048, dtype="float32", std=0.02, sigmoid=False, norm=False),
    "c2": dict(T=16384, H=2048, E=128, K=8, F=768, dtype="bfloat16", std=0.02, sigmoid=False, norm=True),
    "c3": dict(T=16384, H=2048, E=128, K=8, F=768, dtype="bfloat16", std=0.02, sigmoid=False, norm=True, zipf=1.2),
    "c4": dict(
        T=8192, H=7168, E=256, K=8, F=2048, dtype="bfloat16", std=0.006, sigmoid=True, norm=True, n_group=8, topk_group=4
    ),
}


def zipf_logit_bias(E: int, s: float, gen: torch.Generator) -> torch.Tensor:
    """``log`` of a Zipf(s) popularity profile laid over a seeded permutation of the
    experts; added to every token's logits it skews the routing."""
    rank = torch.arange(1, E + 1, dtype=torch.float64)
    pop = rank ** (-s)
    pop = pop / pop.sum()
    perm = torch.randperm(E, generator=gen)
    bias = torch.empty(E, dtype=torch.float64)
    bias[perm] = torch.log(pop)
    return bias.float()


def make_config_inputs(name: str, seed: int = 1234, *, scale_tokens: float = 1.0, experts: int | None = None):
    """CPU tensors for one configuration: ``x [T,H]``, ``w1 [E,2F,H]``, ``w2 [E,H,F]``
    ~ N(0, std) cast to the config dtype, ``logits [T,E]`` fp32 ~ N(0,1) (+ Zipf bias)."""
    cfg = dict(CONFIGS[name])
    gen = torch.Generator().manual_seed(seed)
    T = max(1, int(cfg["T"] * scale_tokens))
    E = experts or cfg["E"]
    H, F = cfg["H"], cfg["F"]
    dt = getattr(torch, cfg["dtype"])
    x = (torch.randn(T, H, generator=gen) * cfg["std"]).to(dt)
    w1 = (torch.randn(E, 2 * F, H, generator=gen) * cfg["std"]).to(dt)
    w2 = (torch.randn(E, H, F, generator=gen) * cfg["std"]).to(dt)
    logits = torch.randn(T, E, generator=gen)
    if "zipf" in cfg:
        # skew: a few experts receive >10x the mean load, the least popular almost none
        logits = logits + zipf_logit_bias(E, cfg["zipf"], gen).unsqueeze(0)
    cfg.update(T=T, E=E)
    return cfg, x, w1, w2, logits
