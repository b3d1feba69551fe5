"""
Drop-in surface: every class, method, parameter name, property and module function that a caller of the
reference's `culsh` package can name exists here under the same name (extra, optional parameters are
allowed).  The expected names are fixtures written from the text of the reference's files by
tests/golden/make_surface.py (python/culsh/_culsh_core.pyi:22-301, python/culsh/*.py).
"""

import inspect
import json
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


def _check_callable(owner, fn, spec):
    sig = inspect.signature(fn)
    names = [p for p in sig.parameters if p not in ("self", "cls")]
    have_var_kw = any(p.kind is inspect.Parameter.VAR_KEYWORD for p in sig.parameters.values())
    # the reference's parameters, in its order, lead ours; anything we add comes after and has a default
    want = spec["params"]
    assert len(names) >= len(want), f"{owner}: takes {names}, the reference {want}"
    for position, (have, ref) in enumerate(zip(names, want)):
        # `argN` in the stub marks a positional-only parameter of the binding: its position is the contract
        if not re.fullmatch(r"arg\d+", ref):
            assert have == ref, f"{owner}: parameter {position} is {have!r}, the reference names it {ref!r}"
    for extra in names[len(want):]:
        p = sig.parameters[extra]
        assert p.default is not inspect.Parameter.empty or p.kind in (
            inspect.Parameter.VAR_POSITIONAL, inspect.Parameter.VAR_KEYWORD), f"{owner}: extra parameter {extra} has no default"
    for kw in spec["kwonly"]:
        assert kw in sig.parameters or have_var_kw, f"{owner}: keyword {kw} missing"
    required_here = [n for n in names if sig.parameters[n].default is inspect.Parameter.empty
                     and sig.parameters[n].kind in (inspect.Parameter.POSITIONAL_ONLY, inspect.Parameter.POSITIONAL_OR_KEYWORD)]
    assert len(required_here) <= len(spec["required"]), f"{owner}: requires {required_here}, the reference only {spec['required']}"


def _check_class(cls, spec, where):
    for name, mspec in spec["methods"].items():
        assert hasattr(cls, name), f"{where}.{cls.__name__} lacks {name}"
        raw = inspect.getattr_static(cls, name)
        if name in spec["static"]:
            assert isinstance(raw, (staticmethod, classmethod)), f"{where}.{cls.__name__}.{name} must be callable on the class"
        _check_callable(f"{where}.{cls.__name__}.{name}", getattr(cls, name), mspec)
    for prop in spec["properties"]:
        assert isinstance(inspect.getattr_static(cls, prop), property), f"{where}.{cls.__name__}.{prop} must be a property"


def test_core_module_surface():
    from culsh_amd import _culsh_core as core

    want = _load("core_surface.json")
    for cname, spec in want["classes"].items():
        assert hasattr(core, cname), f"_culsh_core lacks {cname}"
        _check_class(getattr(core, cname), spec, "_culsh_core")


@pytest.mark.parametrize("module", ["rp_lsh", "pstable_lsh", "minhash_lsh", "utils"])
def test_python_api_surface(module):
    import importlib

    want = _load("api_surface.json")["modules"][module]
    mod = importlib.import_module(f"culsh_amd.{module}")
    for cname, spec in want["classes"].items():
        assert hasattr(mod, cname), f"{module} lacks {cname}"
        _check_class(getattr(mod, cname), spec, module)
    for fname, fspec in want["functions"].items():
        assert hasattr(mod, fname), f"{module} lacks {fname}"
        _check_callable(f"{module}.{fname}", getattr(mod, fname), fspec)


def test_reference_import_name_resolves_to_this_package():
    import culsh
    import culsh_amd
    from culsh import RPLSH, MinHashLSH, PStableLSH  # noqa: F401
    from culsh._culsh_core import Candidates, RPLSHCore  # noqa: F401
    from culsh.rp_lsh import RPLSHModel
    from culsh.utils import compute_recall  # noqa: F401

    want = _load("api_surface.json")
    assert sorted(culsh.__all__) == sorted(want["__all__"])
    for name in want["__all__"]:
        assert getattr(culsh, name) is getattr(culsh_amd, name)
    assert RPLSHModel is culsh_amd.RPLSHModel
    assert culsh.__version__ == culsh_amd.__version__
