"""Behaviour of the plugin registry, one fact per test (reference
steptronoss/utils/optimizable.py:22-103)."""

import pytest

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
