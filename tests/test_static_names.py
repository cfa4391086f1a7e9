"""Every global name a function of the package loads must exist: in its module after import, or
among the builtins.  (A misspelt or never-imported name on a rarely taken branch otherwise
shows up as a NameError in the middle of a search.)"""
import builtins
import dis
import importlib
import os
import types

import pytest

import superscaler_amd

MODULES = sorted(f[:-3] for f in os.listdir(superscaler_amd.__path__[0]) if f.endswith(".py") and f != "__init__.py")
EXTRA = ["bench", "__graft_entry__"]


def _global_loads(code):
    for ins in dis.get_instructions(code):
        if ins.opname in ("LOAD_GLOBAL", "LOAD_NAME"):
            yield ins.argval, code.co_name, ins.starts_line
    for c in code.co_consts:
        if isinstance(c, types.CodeType):
            yield from _global_loads(c)


def _missing(mod):
    with open(mod.__file__) as f:
        code = compile(f.read(), mod.__file__, "exec")
    bad = []
    for name, where, _ in _global_loads(code):
        if not hasattr(mod, name) and not hasattr(builtins, name):
            bad.append((name, where))
    return sorted(set(bad))


@pytest.mark.parametrize("name", MODULES)
def test_package_module_has_no_undefined_global(name):
    mod = importlib.import_module(f"superscaler_amd.{name}")
    assert _missing(mod) == []


@pytest.mark.parametrize("name", EXTRA)
def test_root_script_has_no_undefined_global(name):
    mod = importlib.import_module(name)
    assert os.path.dirname(mod.__file__) == os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    assert _missing(mod) == []
