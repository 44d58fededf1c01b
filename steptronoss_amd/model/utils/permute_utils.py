"""TE-style MoE permutation helpers on the gfx950 kernels.

Same names, arguments, return values and errors as the reference's pure-PyTorch helpers
(reference steptronoss/model/utils/permute_utils.py:43-277).  Rows are moved by the library's
row-gather and sorted-segment-sum kernels, the orderings come from its stable sort; torch
supplies device memory and a little index arithmetic on the (small) id vectors.  Like the
reference, functions whose output length depends on the data read one count back to the host.

Differentiable in ``inp`` (the permutation and its transpose are each other's backward) and,
like the reference, in the probabilities: ``merging_probs`` of ``moe_unpermute`` receives the
row dot products, ``probs`` of the ``*_with_probs`` functions the scatter-add of the permuted
probabilities' gradient.
"""

from __future__ import annotations

import torch

from steptronoss_amd import _lib
from steptronoss_amd._lib import call, dtype_code, is_i64, ptr, require_gpu, stream

__all__ = [
    "moe_permute",
    "moe_permute_with_probs",
    "moe_sort_chunks_by_index",
    "moe_sort_chunks_by_index_with_probs",
    "moe_unpermute",
]

_MAX_KEY_BOUND = 1 << 24


# --------------------------------------------------------------------------- kernels
def _sort_by_key(keys: torch.Tensor, key_bound: int):
    """Stable sort of the entries with ``0 <= key < key_bound``: ``(sorted_key, sorted_index,
    n_valid)`` with int32 lists padded to ``keys.numel()`` and the count as a device int32."""
    keys = keys.contiguous()
    n = keys.numel()
    dev = keys.device
    if key_bound > _MAX_KEY_BOUND:
        raise ValueError(f"at most {_MAX_KEY_BOUND} distinct keys are supported")
    sorted_key = torch.empty((n,), device=dev, dtype=torch.int32)
    sorted_index = torch.empty((n,), device=dev, dtype=torch.int32)
    n_valid = torch.zeros((1,), device=dev, dtype=torch.int32)
    nbytes = _lib.load().stm_sort_by_key_workspace_bytes(n, key_bound)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
    call(
        "stm_sort_by_key", ptr(keys), is_i64(keys), n, key_bound, ptr(sorted_key), ptr(sorted_index), ptr(n_valid),
        ptr(ws), nbytes, stream(),
    )  # fmt: skip
    return sorted_key, sorted_index, n_valid


def _gather_rows_raw(x: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """``out[j] = x[idx[j]]`` (zero row where ``idx[j] < 0``); ``x`` is ``[n, ...]``."""
    x = x.contiguous()
    idx = idx.contiguous()
    out = torch.empty((idx.numel(),) + tuple(x.shape[1:]), device=x.device, dtype=x.dtype)
    row_bytes = x.element_size()
    for d in x.shape[1:]:
        row_bytes *= d
    call("stm_gather_rows", ptr(x), ptr(idx), is_i64(idx), ptr(out), idx.numel(), row_bytes, x.shape[0], stream())
    return out


def _scatter_add_rows_raw(rows: torch.Tensor, dest: torch.Tensor, n_out: int, weight=None) -> torch.Tensor:
    """``out[d] = sum_{j: dest[j] == d} weight[j] * rows[j]`` for ``d < n_out`` (fp32 sums in
    ascending ``j``, rounded once); entries with ``dest[j] < 0`` are skipped."""
    rows = rows.contiguous()
    hidden = rows.shape[1]
    out = torch.empty((n_out, hidden), device=rows.device, dtype=rows.dtype)
    if n_out == 0 or hidden == 0:
        return out
    if n_out > _MAX_KEY_BOUND:
        raise ValueError(f"at most {_MAX_KEY_BOUND} output rows are supported")
    sorted_key, sorted_index, _ = _sort_by_key(dest, n_out)
    w = None if weight is None else weight.contiguous()
    call(
        "stm_segment_sum_rows", ptr(rows), ptr(sorted_key), ptr(sorted_index), dest.numel(), 1, ptr(w),
        dtype_code(w.dtype) if w is not None else 0, ptr(out), n_out, hidden, dtype_code(rows.dtype), stream(),
    )  # fmt: skip
    return out


class _GatherRows(torch.autograd.Function):
    """Rows picked by index; the backward adds the row gradients back per source row."""

    @staticmethod
    def forward(ctx, x, idx):
        ctx.save_for_backward(idx)
        ctx.src_shape = tuple(x.shape)
        with torch.cuda.device(x.device):
            return _gather_rows_raw(x, idx)

    @staticmethod
    def backward(ctx, grad_out):
        (idx,) = ctx.saved_tensors
        n_src = ctx.src_shape[0]
        with torch.cuda.device(grad_out.device):
            g = grad_out.contiguous().reshape(idx.numel(), -1)
            return _scatter_add_rows_raw(g, idx, n_src).reshape(ctx.src_shape), None


def _row_dot(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``out[j] = <a[j], b[j]>`` in fp32."""
    a, b = a.contiguous(), b.contiguous()
    out = torch.empty((a.shape[0],), device=a.device, dtype=torch.float32)
    call("stm_row_dot", ptr(a), ptr(b), ptr(out), a.shape[0], a.shape[1], dtype_code(a.dtype), stream())
    return out


class _ScatterAddRows(torch.autograd.Function):
    """Rows added into ``out[dest[j]]`` with an optional per-row weight."""

    @staticmethod
    def forward(ctx, rows, dest, weight, n_out):
        ctx.save_for_backward(dest, weight, rows if weight is not None else None)
        with torch.cuda.device(rows.device):
            return _scatter_add_rows_raw(rows, dest, n_out, weight)

    @staticmethod
    def backward(ctx, grad_out):
        dest, weight, rows = ctx.saved_tensors
        grad_weight = None
        with torch.cuda.device(grad_out.device):
            g = _gather_rows_raw(grad_out.contiguous(), dest)  # zero rows where dest < 0
            if weight is not None:
                if ctx.needs_input_grad[2]:  # d weight[j] = <d out[dest[j]], rows[j]>
                    grad_weight = _row_dot(g, rows).to(weight.dtype)
                g = g * weight.to(g.dtype).unsqueeze(-1)
        return g, None, grad_weight, None


def _float_rows_supported(t: torch.Tensor) -> None:
    if t.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise TypeError("rows must be float32, float16 or bfloat16")


# --------------------------------------------------------------------------- helpers
def _pad_or_trim(indices: torch.Tensor, num_out_tokens: int):
    """reference permute_utils.py:16-29."""
    if num_out_tokens < 0 or num_out_tokens == indices.numel():
        return indices, indices.numel()
    if num_out_tokens < indices.numel():
        return indices[:num_out_tokens], num_out_tokens
    pad = torch.full((num_out_tokens - indices.numel(),), -1, device=indices.device, dtype=indices.dtype)
    return torch.cat([indices, pad], dim=0), num_out_tokens


def _check_permute_args(inp, routing_map, what):
    if routing_map.dim() != 2:
        raise ValueError(f"routing_map must be 2D [num_tokens, {what}]")
    if inp.dim() != 2:
        raise ValueError("inp must be 2D [num_tokens, hidden_size]")
    if inp.size(0) != routing_map.size(0):
        raise ValueError("inp and routing_map must have the same num_tokens")


def _permute_mask_map(inp, routing_map, num_out_tokens, probs):
    """reference permute_utils.py:43-89: rows in expert-major order, ``row_id = e*T + t``."""
    if inp.numel() == 0:
        empty = torch.tensor([], device=inp.device, dtype=torch.long)
        return inp, empty, None if probs is None else probs.new_empty((0,))
    _check_permute_args(inp, routing_map, "num_experts")
    require_gpu(inp, routing_map)
    T, E = routing_map.shape
    with torch.cuda.device(inp.device):
        mask = routing_map.to(torch.bool)
        expert_of = torch.arange(E, device=inp.device, dtype=torch.int32).expand(T, E)
        keys = torch.where(mask, expert_of, torch.full_like(expert_of, -1))  # entry t*E+e -> e or -1
        sorted_key, sorted_index, n_valid = _sort_by_key(keys.reshape(-1), E)
        n = int(n_valid.item())  # the output length depends on the data (the reference's nonzero)
        e_ids = sorted_key[:n].to(torch.long)
        t_ids = sorted_index[:n].to(torch.long) // E
        row_id_map, out_len = _pad_or_trim(e_ids * T + t_ids, num_out_tokens)
        token_ids = torch.where(row_id_map >= 0, row_id_map % T, torch.full_like(row_id_map, -1))
        output = _GatherRows.apply(inp, token_ids)
        permuted_probs = None
        if probs is not None:
            if probs.shape != routing_map.shape:
                raise ValueError("probs must have shape [num_tokens, num_experts]")
            probs_flat = probs.T.contiguous().reshape(-1, 1)
            permuted_probs = _GatherRows.apply(probs_flat, row_id_map).reshape(-1)
    return output, row_id_map, permuted_probs


def _permute_index_map(inp, routing_map, num_out_tokens):
    """reference permute_utils.py:92-126: slots sorted by (expert, flat position)."""
    if inp.numel() == 0:
        return inp, torch.tensor([], device=inp.device, dtype=torch.long)
    _check_permute_args(inp, routing_map, "top_k")
    require_gpu(inp, routing_map)
    _T, top_k = routing_map.shape
    with torch.cuda.device(inp.device):
        flat = routing_map.reshape(-1)
        bound = int(flat.max().item()) + 1 if flat.numel() else 0  # expert count is not an argument
        if bound > 0:
            _key, sorted_index, n_valid = _sort_by_key(flat, bound)
            row_id_map = sorted_index[: int(n_valid.item())].to(torch.long)
        else:
            row_id_map = torch.zeros((0,), device=inp.device, dtype=torch.long)
        row_id_map, _out_len = _pad_or_trim(row_id_map, num_out_tokens)
        token_ids = torch.div(row_id_map, top_k, rounding_mode="floor")  # -1 stays -1
        output = _GatherRows.apply(inp, token_ids)
    return output, row_id_map


def moe_permute(inp, routing_map, num_out_tokens: int = -1, max_token_num: int = -1, map_type: str = "mask"):
    """Permute tokens by ``routing_map`` (reference permute_utils.py:129-143)."""
    del max_token_num
    if map_type == "index":
        return _permute_index_map(inp, routing_map, num_out_tokens)
    if map_type == "mask":
        output, row_id_map, _ = _permute_mask_map(inp, routing_map, num_out_tokens, None)
        return output, row_id_map
    raise ValueError("map_type should be one of 'mask' or 'index'")


def moe_permute_with_probs(inp, probs, routing_map, num_out_tokens: int = -1):
    """Permute tokens and their probabilities (reference permute_utils.py:146-154)."""
    output, row_id_map, permuted_probs = _permute_mask_map(inp, routing_map, num_out_tokens, probs)
    return output, permuted_probs, row_id_map


def moe_unpermute(inp, row_id_map, merging_probs=None, restore_shape=None, map_type: str = "mask", probs=None):
    """Rows added back to token order, optionally weighted (reference permute_utils.py:157-234)."""
    if probs is not None:
        if merging_probs is not None:
            raise ValueError("Both merging_probs and probs are provided. probs is deprecated.")
        merging_probs = probs
    if inp.numel() == 0:
        return inp
    if map_type not in ("mask", "index"):
        raise ValueError("map_type should be one of 'mask' or 'index'")
    require_gpu(inp, row_id_map)
    _float_rows_supported(inp)
    with torch.cuda.device(inp.device):
        if map_type == "mask":
            if merging_probs is not None:
                num_tokens, _ = merging_probs.shape
            elif restore_shape is not None:
                num_tokens = restore_shape[0]
            else:
                raise ValueError("restore_shape or merging_probs must be provided for map_type='mask'.")
            token_ids = torch.where(row_id_map >= 0, row_id_map % max(num_tokens, 1), torch.full_like(row_id_map, -1))
            probs_flat = None if merging_probs is None else merging_probs.T.contiguous().reshape(-1, 1)
        else:
            if merging_probs is not None:
                num_tokens, top_k = merging_probs.shape
            elif restore_shape is not None:
                num_tokens = restore_shape[0]
                valid = row_id_map >= 0
                top_k = int(row_id_map[valid].max().item()) // max(num_tokens, 1) + 1 if bool(valid.any()) else 1
            else:
                num_tokens = row_id_map.size(0)
                top_k = 1
            token_ids = torch.div(row_id_map, top_k, rounding_mode="floor")
            probs_flat = None if merging_probs is None else merging_probs.reshape(-1, 1)
        weights = None
        if probs_flat is not None:
            weights = _GatherRows.apply(probs_flat.contiguous(), row_id_map).reshape(-1)
        hidden = inp.size(1)
        out_rows = restore_shape[0] if restore_shape is not None else num_tokens
        output = _ScatterAddRows.apply(inp, token_ids, weights, out_rows)
        if restore_shape is not None and tuple(restore_shape) != (out_rows, hidden):
            output = output.reshape(restore_shape)
    return output


def _chunk_rows(split_sizes, sorted_index, device):
    if split_sizes.dim() != 1:
        raise ValueError("split_sizes must be 1D")
    if sorted_index.dim() != 1:
        raise ValueError("sorted_index must be 1D")
    sizes = [int(v) for v in split_sizes.tolist()]  # host values, as in the reference (:249-251)
    starts = [0]
    for v in sizes:
        starts.append(starts[-1] + v)
    pieces = [torch.arange(starts[i], starts[i + 1], dtype=torch.long) for i in sorted_index.tolist()]
    rows = torch.cat(pieces) if pieces else torch.zeros((0,), dtype=torch.long)
    return rows.to(device)


def moe_sort_chunks_by_index(inp, split_sizes, sorted_index):
    """Split rows by ``split_sizes`` and emit the chunks in ``sorted_index`` order
    (reference permute_utils.py:237-252)."""
    if inp.numel() == 0:
        return inp
    require_gpu(inp)
    rows = _chunk_rows(split_sizes, sorted_index, inp.device)
    return _GatherRows.apply(inp, rows)


def moe_sort_chunks_by_index_with_probs(inp, probs, split_sizes, sorted_index):
    """As above for rows and their probabilities (reference permute_utils.py:255-277)."""
    if inp.numel() == 0:
        return inp, probs
    if probs.size(0) != inp.size(0):
        raise ValueError("probs and inp must have the same leading dimension")
    require_gpu(inp, probs)
    rows = _chunk_rows(split_sizes, sorted_index, inp.device)
    return _GatherRows.apply(inp, rows), _GatherRows.apply(probs, rows)
