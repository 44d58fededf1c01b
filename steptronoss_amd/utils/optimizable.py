"""Registry of switchable implementations: the plugin surface of the MoE hot path.

API-identical counterpart of the reference's ``steptronoss/utils/optimizable.py``
(:14-19 ``OptimizeMeta`` / ``OPTIMIZABLE_REGISTER``, :22-60 ``optimizable``,
:63-103 ``set_optimization``), written from its observable behaviour:

* a decorated function is registered under ``"<module>.<qualname>"``;
* the dict of alternatives handed to the decorator is stored *as the same object*
  (so callers can add entries to it later) and gains a ``"torch_compile"`` entry;
* every call looks the active alternative up at call time and forwards the
  arguments untouched;
* ``set_optimization`` first resets *every* registered function to ``default``,
  then applies the keyword overrides; a function may be named by its last dotted
  component unless two registered functions share it; an unknown function or an
  unknown alternative raises a bare ``KeyError()``.
"""

from __future__ import annotations

import functools
import logging
from collections.abc import Callable
from pprint import pformat
from typing import TypedDict

import torch

log = logging.getLogger("steptronoss_amd.optimizable")


class OptimizeMeta(TypedDict):
    alternatives: dict[str, Callable]
    use_optimize: str | None


OPTIMIZABLE_REGISTER: dict[str, OptimizeMeta] = {}


def optimizable(alternatives: dict[str, Callable] | None = None):
    """Decorator: make ``func`` switchable between itself and ``alternatives``."""

    def decorate(func: Callable):
        module = getattr(func, "__module__", "UnknownModule")
        name = getattr(func, "__qualname__", func.__name__)
        key = f"{module}.{name}"
        table = alternatives if alternatives else {}
        table["torch_compile"] = torch.compile(func)
        OPTIMIZABLE_REGISTER[key] = OptimizeMeta(alternatives=table, use_optimize=None)

        @functools.wraps(func)
        def dispatch(*args, **kwargs):
            chosen = OPTIMIZABLE_REGISTER[key]["use_optimize"]
            if chosen:
                return OPTIMIZABLE_REGISTER[key]["alternatives"][chosen](*args, **kwargs)
            return func(*args, **kwargs)

        return dispatch

    return decorate


def _short_names() -> dict[str, str]:
    names: dict[str, str | None] = {}
    for key in OPTIMIZABLE_REGISTER:
        short = key.rsplit(".", 1)[-1]
        names[short] = None if short in names else key  # ambiguous short names are disabled
        names[key] = key
    return {k: v for k, v in names.items() if v is not None}


def set_optimization(default=None, **kwargs):
    """Select the active alternative of registered functions.

    ``default`` is applied to *all* registered functions first (so naming one
    function switches every other one back to ``default``); then each
    ``name=alternative`` (``None`` = the function's own body) is applied.
    """
    names = _short_names()
    for meta in OPTIMIZABLE_REGISTER.values():
        meta["use_optimize"] = default
    for name, choice in kwargs.items():
        if name not in names:
            log.error("Cannot find Func %s in optimizable register! Availables: \n%s", name, pformat(names))
            raise KeyError()
        meta = OPTIMIZABLE_REGISTER[names[name]]
        if choice is not None and choice not in meta["alternatives"]:
            log.error("Func %s has no alter named %s! Availables: \n%s", name, choice, pformat(meta["alternatives"]))
            raise KeyError()
        meta["use_optimize"] = choice
    active = "\n".join(f"{k} -> {m['use_optimize']}" for k, m in OPTIMIZABLE_REGISTER.items() if m["use_optimize"])
    log.info("Optimization set: \n%s", active)
