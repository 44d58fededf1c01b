"""Registers the gfx950 kernels as the ``hip_gfx950`` alternative of the six switchable MoE ops.

The six ops are looked up in a registry of the ``optimizable`` kind by the last component of
their key (``histogram``, ``index_compute``, ``moe_scatter``, ``moe_weighted_gather``,
``grouped_gemm``, ``routed_grouped_ffn``); the alternative is inserted into the registry's
own dict, which is how a backend joins without touching the framework
(reference steptronoss/utils/optimizable.py:44-56, steptronoss/model/utils/moe_utils.py:85-442).
"""

from __future__ import annotations

from steptronoss_amd.model.utils import moe_utils as _ops

BACKEND_NAME = _ops.BACKEND_NAME

BACKEND_OPS = {
    "histogram": _ops.hip_histogram,
    "index_compute": _ops.hip_index_compute,
    "moe_scatter": _ops.hip_moe_scatter,
    "moe_weighted_gather": _ops.hip_moe_weighted_gather,
    "grouped_gemm": _ops.hip_grouped_gemm,
    "routed_grouped_ffn": _ops.hip_routed_grouped_ffn,
}


def register_backend(registry: dict | None = None, name: str = BACKEND_NAME) -> list[str]:
    """Insert the kernels into ``registry`` (default: StepTronOSS's own registry when that
    package is importable, else this package's).  Returns the keys that gained the entry."""
    if registry is None:
        try:
            from steptronoss.model.utils import moe_utils as _  # noqa: F401  (registers the reference ops)
            from steptronoss.utils.optimizable import OPTIMIZABLE_REGISTER as registry
        except Exception:
            from steptronoss_amd.utils.optimizable import OPTIMIZABLE_REGISTER as registry
    touched = []
    for key, meta in registry.items():
        short = key.rsplit(".", 1)[-1]
        if short in BACKEND_OPS and key.rsplit(".", 1)[0].endswith("moe_utils"):
            meta["alternatives"][name] = BACKEND_OPS[short]
            touched.append(key)
    return touched


def enable(set_optimization=None, name: str = BACKEND_NAME) -> None:
    """Select the backend for all six ops through ``set_optimization`` (this package's by
    default).  Note that every ``set_optimization`` call resets ops it does not name."""
    if set_optimization is None:
        from steptronoss_amd.utils.optimizable import set_optimization
    set_optimization(**{short: name for short in BACKEND_OPS})
