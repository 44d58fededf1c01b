"""SwiGLU of the expert FFN on the gfx950 kernels.

Counterpart of ``FeedForwardConfig.activation`` (reference
steptronoss/model/common/feed_forward.py:20-26): ``silu(x[..., :F]) * x[..., F:]`` with an
optional clamp (gate side clamped from above after the SiLU, up side to ``[-limit, limit]``).
"""

from __future__ import annotations

import torch

from steptronoss_amd._lib import call, dtype_code, ptr, require_gpu, stream


def swiglu_fwd_rows(gu: torch.Tensor, swiglu_limit, live_rows: torch.Tensor | None = None) -> torch.Tensor:
    rows, two_f = gu.shape
    f = two_f // 2
    out = torch.empty((rows, f), device=gu.device, dtype=gu.dtype)
    call(
        "stm_swiglu_fwd", ptr(gu), ptr(out), rows, f, ptr(live_rows), int(swiglu_limit is not None),
        float(swiglu_limit or 0.0), dtype_code(gu.dtype), stream(),
    )  # fmt: skip
    return out


def swiglu_bwd_rows(gu: torch.Tensor, grad_out: torch.Tensor, swiglu_limit, live_rows=None) -> torch.Tensor:
    rows, two_f = gu.shape
    f = two_f // 2
    dgu = torch.empty_like(gu)
    call(
        "stm_swiglu_bwd", ptr(gu), ptr(grad_out), ptr(dgu), rows, f, ptr(live_rows), int(swiglu_limit is not None),
        float(swiglu_limit or 0.0), dtype_code(gu.dtype), stream(),
    )  # fmt: skip
    return dgu


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, swiglu_limit):
        dev = require_gpu(x)
        shape = x.shape
        x2 = x.contiguous().reshape(-1, shape[-1])
        ctx.save_for_backward(x2)
        ctx.limit = swiglu_limit
        ctx.shape = shape
        with torch.cuda.device(dev):
            out = swiglu_fwd_rows(x2, swiglu_limit)
        return out.reshape(*shape[:-1], shape[-1] // 2)

    @staticmethod
    def backward(ctx, grad_out):
        (x2,) = ctx.saved_tensors
        with torch.cuda.device(x2.device):
            dgu = swiglu_bwd_rows(x2, grad_out.contiguous().reshape(x2.shape[0], -1), ctx.limit)
        return dgu.reshape(ctx.shape), None


def swiglu(x: torch.Tensor, swiglu_limit=None) -> torch.Tensor:
    """``silu(gate) * up`` over the last dimension split in halves (differentiable)."""
    if x.shape[-1] % 2:
        raise ValueError("the last dimension must be even (gate | up)")
    return _SwiGLU.apply(x, swiglu_limit)


swiglu.is_steptron_swiglu = True
