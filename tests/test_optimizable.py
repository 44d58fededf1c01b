"""Behaviour of the plugin registry, one fact per test (reference
steptronoss/utils/optimizable.py:22-103)."""

import pytest

from steptronoss_amd import backend  # (registers this package's own six ops on import)
from steptronoss_amd.utils import optimizable as opt


@pytest.fixture
def registry():
    saved = dict(opt.OPTIMIZABLE_REGISTER)
    opt.OPTIMIZABLE_REGISTER.clear()
    yield opt.OPTIMIZABLE_REGISTER
    opt.OPTIMIZABLE_REGISTER.clear()
    opt.OPTIMIZABLE_REGISTER.update(saved)


def _make(name="f", alts=None):
    def body(x):
        return ("base", x)

    body.__qualname__ = name
    body.__module__ = "pkg.mod"
    return opt.optimizable(alts)(body)


def test_key_is_module_dot_qualname_and_torch_compile_is_added(registry):
    alts = {"fast": lambda x: ("fast", x)}
    _make("f", alts)
    assert list(registry) == ["pkg.mod.f"]
    assert registry["pkg.mod.f"]["alternatives"] is alts  # the caller's dict object itself
    assert set(alts) == {"fast", "torch_compile"}
    assert registry["pkg.mod.f"]["use_optimize"] is None


def test_dispatch_looks_up_at_call_time(registry):
    f = _make("f", {"fast": lambda x: ("fast", x)})
    assert f(1) == ("base", 1)
    opt.set_optimization(f="fast")
    assert f(2) == ("fast", 2)
    registry["pkg.mod.f"]["alternatives"]["late"] = lambda x: ("late", x)  # added after decoration
    opt.set_optimization(f="late")
    assert f(3) == ("late", 3)
    opt.set_optimization(f=None)
    assert f(4) == ("base", 4)


def test_every_call_resets_unnamed_functions_to_default(registry):
    f = _make("f", {"fast": lambda x: "ff"})
    g = _make("g", {"fast": lambda x: "gf"})
    opt.set_optimization(f="fast", g="fast")
    opt.set_optimization(g="fast")  # f silently falls back to its own body
    assert f(0) == ("base", 0) and g(0) == "gf"
    opt.set_optimization(default="fast")
    assert f(0) == "ff" and g(0) == "gf"


def test_full_key_and_short_name(registry):
    f = _make("f", {"fast": lambda x: "ff"})
    opt.set_optimization(**{"pkg.mod.f": "fast"})
    assert f(0) == "ff"


def test_ambiguous_short_name_is_disabled(registry):
    _make("f", {"fast": lambda x: "a"})

    def other(x):
        return "other"

    other.__qualname__ = "f"
    other.__module__ = "pkg.other"
    opt.optimizable({"fast": lambda x: "b"})(other)
    with pytest.raises(KeyError):
        opt.set_optimization(f="fast")
    opt.set_optimization(**{"pkg.other.f": "fast"})


def test_unknown_function_or_alternative_raises_bare_keyerror(registry):
    _make("f", {"fast": lambda x: "ff"})
    with pytest.raises(KeyError) as e1:
        opt.set_optimization(nope="fast")
    assert e1.value.args == ()
    with pytest.raises(KeyError) as e2:
        opt.set_optimization(f="nope")
    assert e2.value.args == ()


def test_arguments_are_forwarded_unchanged(registry):
    seen = {}

    def alt(*a, **k):
        seen["a"], seen["k"] = a, k
        return 7

    f = _make("f", {"alt": alt})
    opt.set_optimization(f="alt")
    assert f(1, 2, z=3) == 7 and seen == {"a": (1, 2), "k": {"z": 3}}


def test_register_backend_joins_a_registry_keyed_like_the_reference(registry):
    """The reference's six ops live under ``steptronoss.model.utils.moe_utils.<op>``, each with its
    own alternatives, absent optional backends registered as ``None``
    (reference moe_utils.py:3-58, 85-89, 435-442).  register_backend adds ``hip_gfx950`` to exactly
    those six dicts (the caller's own dict objects), touches nothing else, and set_optimization
    then dispatches to the inserted callables."""
    ref_alts = {
        "histogram": {"triton": None},
        "index_compute": {"triton": None},
        "routed_grouped_ffn": {"fused": None},
        "moe_weighted_gather": {"triton": None},
        "moe_scatter": {"triton": None},
        "grouped_gemm": {"nv_grouped_gemm": None, "triton_grouped_gemm": None, "npu_gmm": None, "function_imple": lambda *a, **k: "fi"},
    }  # fmt: skip
    wrapped = {}
    for name, alts in ref_alts.items():
        def body(*a, _name=name, **k):
            return ("baseline", _name)

        body.__qualname__ = name
        body.__module__ = "steptronoss.model.utils.moe_utils"
        wrapped[name] = opt.optimizable(alts)(body)
    # an op of the same short name elsewhere, and an unrelated op in the same module: left alone
    def stray(*a, **k):
        return "stray"

    stray.__qualname__ = "histogram"
    stray.__module__ = "steptronoss.data.stats"
    stray_alts = {}
    opt.optimizable(stray_alts)(stray)
    def gate(*a, **k):
        return "gate"

    gate.__qualname__ = "MoEGateFunction"
    gate.__module__ = "steptronoss.model.utils.moe_utils"
    gate_alts = {}
    opt.optimizable(gate_alts)(gate)

    touched = backend.register_backend(registry)
    assert sorted(touched) == sorted(f"steptronoss.model.utils.moe_utils.{n}" for n in ref_alts)
    for name, alts in ref_alts.items():
        assert alts[backend.BACKEND_NAME] is backend.BACKEND_OPS[name]  # inserted into the caller's dict
        assert registry[f"steptronoss.model.utils.moe_utils.{name}"]["alternatives"] is alts
    assert backend.BACKEND_NAME not in stray_alts and backend.BACKEND_NAME not in gate_alts
    assert ref_alts["grouped_gemm"]["nv_grouped_gemm"] is None  # absent backends stay as they were

    # dispatch through the registry: full keys (the short name "histogram" is ambiguous here)
    calls = []
    for name in ref_alts:
        ref_alts[name][backend.BACKEND_NAME] = lambda *a, _n=name, **k: calls.append(_n) or ("hip", _n)
    opt.set_optimization(**{f"steptronoss.model.utils.moe_utils.{n}": backend.BACKEND_NAME for n in ref_alts})
    for name, fn in wrapped.items():
        assert fn(1, 2) == ("hip", name)
    assert calls == list(ref_alts)
    opt.set_optimization(grouped_gemm="function_imple")  # resets the other five to their baselines
    assert wrapped["grouped_gemm"]() == "fi" and wrapped["moe_scatter"]() == ("baseline", "moe_scatter")
    with pytest.raises(KeyError):
        opt.set_optimization(histogram=backend.BACKEND_NAME)  # two registered functions share the short name
