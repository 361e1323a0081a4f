"""The repository's entry points: smoke() runs as a GPU test so that a change
of the planner (a workspace it now asks for, another kernel it picks) shows
here and not only where smoke() is run by itself."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def entry():
    spec = importlib.util.spec_from_file_location(
        "__graft_entry__", os.path.join(ROOT, "__graft_entry__.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_entry_points_exist():
    mod = entry()
    assert callable(mod.build) and callable(mod.smoke)


@pytest.mark.gpu
def test_smoke(capsys):
    entry().smoke()
    assert "smoke ok" in capsys.readouterr().out
