"""fp8 (e4m3, 1x128 block scales) forms of the expert GEMMs on the gfx950 kernels.

The reference has no fp8 path (its grouped GEMMs run in the activations' dtype, reference
steptronoss/model/utils/moe_utils.py:423-453); this module serves the fp8 configuration of the
benchmark: quantise activations and weights with one fp32 scale per row per 128 contraction
elements, then ``grouped_gemm_fp8`` for the forward product and, on the transposed weights,
for dgrad.  The ``_pow2`` pair does the same with power-of-two scales, which the block-scaled
matrix instruction of gfx950 applies in hardware; :class:`Fp8ExpertFFN` strings the pieces into the
forward and dgrad of an expert FFN.
"""

from __future__ import annotations

import torch

from steptronoss_amd import _lib
from steptronoss_amd._lib import call, dtype_code, ptr, require_gpu, stream

BLOCK = 128


def quantize_e4m3_1x128(x: torch.Tensor):
    """``(codes uint8 [..., C], scales float32 [..., ceil(C/128)])`` of the last axis of ``x``."""
    require_gpu(x)
    xc = x.contiguous()
    cols = xc.shape[-1]
    rows = xc.numel() // max(cols, 1)
    codes = torch.empty(xc.shape, device=x.device, dtype=torch.uint8)
    scales = torch.empty(xc.shape[:-1] + ((cols + BLOCK - 1) // BLOCK,), device=x.device, dtype=torch.float32)
    with torch.cuda.device(x.device):
        call("stm_quantize_e4m3_1x128", ptr(xc), dtype_code(xc.dtype), rows, cols, ptr(codes), ptr(scales), stream())
    return codes, scales


def quantize_e4m3_1x128_pow2(x: torch.Tensor):
    """``(codes uint8 [R, C], scales float32 [ceil(C/128), R])`` of a matrix (leading axes
    flattened to ``R``): power-of-two scales, stored block-major, as ``grouped_gemm_fp8_pow2``
    reads them."""
    require_gpu(x)
    xc = x.contiguous()
    cols = xc.shape[-1]
    rows = xc.numel() // max(cols, 1)
    codes = torch.empty(xc.shape, device=x.device, dtype=torch.uint8)
    scales = torch.empty(((cols + BLOCK - 1) // BLOCK, rows), device=x.device, dtype=torch.float32)
    with torch.cuda.device(x.device):
        call("stm_quantize_e4m3_1x128_pow2", ptr(xc), dtype_code(xc.dtype), rows, cols, ptr(codes), ptr(scales), stream())
    return codes, scales


def grouped_gemm_fp8_pow2(a_codes, a_scales, b_codes, b_scales, batch_sizes, out_dtype=torch.bfloat16) -> torch.Tensor:
    """As :func:`grouped_gemm_fp8` on the operands of :func:`quantize_e4m3_1x128_pow2`
    (``a_scales`` ``[K/128, M]``, ``b_scales`` ``[K/128, G*N]``): the scales go into the
    block-scaled matrix instruction, the kernel is the persistent one of the bf16 path.
    ``out_dtype`` bf16 or fp16; at least 4096 rows (``NotImplementedError`` otherwise)."""
    from steptronoss_amd.model.utils.moe_utils import _gemm_workspace, _group_offsets

    dev = require_gpu(a_codes, b_codes, a_scales, b_scales)
    if a_codes.dtype != torch.uint8 or b_codes.dtype != torch.uint8:
        raise TypeError("codes must be uint8 tensors")
    if a_codes.dim() != 2 or b_codes.dim() != 3 or a_codes.shape[1] != b_codes.shape[2]:
        raise ValueError("a must be [M, K] and b [G, N, K]")
    m_cap, k = a_codes.shape
    n_groups, n, _ = b_codes.shape
    if k % BLOCK:
        raise ValueError("the contraction length must be a multiple of 128")
    if a_scales.shape != (k // BLOCK, m_cap) or b_scales.shape != (k // BLOCK, n_groups * n):
        raise ValueError("scales must be [K/128, M] and [K/128, G*N]")
    with torch.cuda.device(dev):
        offsets = _group_offsets(batch_sizes, dev)
        out = torch.zeros((m_cap, n), device=dev, dtype=out_dtype)
        ws = _gemm_workspace(m_cap, n_groups, dev)
        # (normalised copies are bound to names: they must outlive the launch)
        a_c, a_s = a_codes.contiguous(), a_scales.contiguous().float()
        b_c, b_s = b_codes.contiguous(), b_scales.contiguous().float()
        ok = _lib.try_call(
            "stm_grouped_gemm_fp8_pow2", ptr(a_c), ptr(a_s), ptr(b_c), ptr(b_s), ptr(out), ptr(offsets), n_groups, m_cap,
            n, k, dtype_code(out_dtype), ptr(ws), ws.numel(), stream(),
        )  # fmt: skip
    if not ok:
        raise NotImplementedError("grouped_gemm_fp8_pow2: shape or output type outside the persistent kernel")
    return out


def grouped_gemm_fp8_pow2_rows(a_codes, a_scales, b_codes, b_scales, offsets, out_dtype, zero_tail=True) -> torch.Tensor:
    """:func:`grouped_gemm_fp8_pow2` for callers that hold the int32 row offsets ``[G+1]`` on the
    device already (no host round trip); rows past the last group stay zero, or, with
    ``zero_tail=False``, keep whatever the buffer held (for callers that never read them: saves
    a fill of the whole output)."""
    from steptronoss_amd.model.utils.moe_utils import _gemm_workspace

    m_cap, k = a_codes.shape
    n_groups, n, _ = b_codes.shape
    alloc = torch.zeros if zero_tail else torch.empty
    out = alloc((m_cap, n), device=a_codes.device, dtype=out_dtype)
    ws = _gemm_workspace(m_cap, n_groups, a_codes.device)
    call(
        "stm_grouped_gemm_fp8_pow2", ptr(a_codes), ptr(a_scales), ptr(b_codes), ptr(b_scales), ptr(out), ptr(offsets),
        n_groups, m_cap, n, k, dtype_code(out_dtype), ptr(ws), ws.numel(), stream(),
    )  # fmt: skip
    return out


def grouped_gemm_fp8(a_codes, a_scales, b_codes, b_scales, batch_sizes, out_dtype=torch.bfloat16) -> torch.Tensor:
    """``out[rows of g] = dequant(a)[rows of g] @ dequant(b[g])^T`` with ``a`` ``[M, K]`` and ``b``
    ``[G, N, K]`` quantised along ``K`` (a multiple of 128); products and sums in fp32."""
    from steptronoss_amd.model.utils.moe_utils import _gemm_workspace, _group_offsets

    dev = require_gpu(a_codes, b_codes, a_scales, b_scales)
    if a_codes.dtype != torch.uint8 or b_codes.dtype != torch.uint8:
        raise TypeError("codes must be uint8 tensors")
    if a_codes.dim() != 2 or b_codes.dim() != 3 or a_codes.shape[1] != b_codes.shape[2]:
        raise ValueError("a must be [M, K] and b [G, N, K]")
    m_cap, k = a_codes.shape
    n_groups, n, _ = b_codes.shape
    if k % BLOCK:
        raise ValueError("the contraction length must be a multiple of 128")
    if a_scales.shape != (m_cap, k // BLOCK) or b_scales.shape != (n_groups, n, k // BLOCK):
        raise ValueError("scales must be [M, K/128] and [G, N, K/128]")
    with torch.cuda.device(dev):
        offsets = _group_offsets(batch_sizes, dev)
        out = torch.zeros((m_cap, n), device=dev, dtype=out_dtype)
        ws = _gemm_workspace(m_cap, n_groups, dev)
        a_c, a_s = a_codes.contiguous(), a_scales.contiguous().float()
        b_c, b_s = b_codes.contiguous(), b_scales.contiguous().float()
        call(
            "stm_grouped_gemm_fp8", ptr(a_c), ptr(a_s), ptr(b_c), ptr(b_s), ptr(out), ptr(offsets), n_groups, m_cap, n, k,
            dtype_code(out_dtype), ptr(ws), ws.numel(), stream(),
        )  # fmt: skip
    return out


class Fp8ExpertFFN:
    """The expert FFN on e4m3 operands, forward and dgrad (the fp8 benchmark configuration; weight
    gradients stay with the bf16 path).  Weights are quantised once, in both orientations:
    along their own contraction axis for the forward and, transposed, along the other one for
    dgrad.  Activations are quantised on the way into each GEMM; GEMM outputs are bf16 / fp16.

    ``rows`` are already in expert order (``moe_scatter``'s output); ``batch_sizes`` are the
    rows per expert.
    """

    def __init__(self, w1: torch.Tensor, w2: torch.Tensor, swiglu_limit=None):
        self.n_experts, two_f, self.hidden = w1.shape
        self.ffn = two_f // 2
        self.limit = swiglu_limit
        self.w1_q, self.w1_s = quantize_e4m3_1x128_pow2(w1)  # [E, 2F, H] along H
        self.w2_q, self.w2_s = quantize_e4m3_1x128_pow2(w2)  # [E, H, F] along F
        self.w1t_q, self.w1t_s = quantize_e4m3_1x128_pow2(w1.transpose(1, 2).contiguous())  # [E, H, 2F] along 2F
        self.w2t_q, self.w2t_s = quantize_e4m3_1x128_pow2(w2.transpose(1, 2).contiguous())  # [E, F, H] along H

    def forward_rows(self, rows: torch.Tensor, batch_sizes: torch.Tensor):
        """``y = swiglu(rows @ w1^T) @ w2^T`` per expert; returns ``(y, gate_up)``."""
        from steptronoss_amd.model.common.feed_forward import swiglu_fwd_rows

        q, sc = quantize_e4m3_1x128_pow2(rows)
        gate_up = grouped_gemm_fp8_pow2(q, sc, self.w1_q, self.w1_s, batch_sizes, out_dtype=rows.dtype)
        with torch.cuda.device(rows.device):
            h = swiglu_fwd_rows(gate_up, self.limit)
        q, sc = quantize_e4m3_1x128_pow2(h)
        return grouped_gemm_fp8_pow2(q, sc, self.w2_q, self.w2_s, batch_sizes, out_dtype=rows.dtype), gate_up

    def dgrad_rows(self, grad_y: torch.Tensor, gate_up: torch.Tensor, batch_sizes: torch.Tensor) -> torch.Tensor:
        """Gradient of the rows given the gradient of ``y`` (the transposed weights as ``b``)."""
        from steptronoss_amd.model.common.feed_forward import swiglu_bwd_rows

        q, sc = quantize_e4m3_1x128_pow2(grad_y)
        grad_h = grouped_gemm_fp8_pow2(q, sc, self.w2t_q, self.w2t_s, batch_sizes, out_dtype=grad_y.dtype)
        with torch.cuda.device(grad_y.device):
            grad_gate_up = swiglu_bwd_rows(gate_up, grad_h, self.limit)
        q, sc = quantize_e4m3_1x128_pow2(grad_gate_up)
        return grouped_gemm_fp8_pow2(q, sc, self.w1t_q, self.w1t_s, batch_sizes, out_dtype=grad_y.dtype)


def _keepalive():  # the library handle, for callers that only import this module
    return _lib.load()
