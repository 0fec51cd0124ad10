"""CPU-side checks of the drop-in boundary: the built library loads and exports every symbol that
include/cattle_hip.h declares. No compute call is made (there is no GPU here)."""
import ctypes
import importlib
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pkg = importlib.import_module("c-attl3_amd")


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "cattle_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cattle_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert _declared_symbols() == sorted(pkg.EXPORTS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(pkg.LIB_PATH):
        pytest.skip("libcattle_hip.so not built yet (run __graft_entry__.build())")
    lib = ctypes.CDLL(pkg.LIB_PATH)
    for name in _declared_symbols():
        assert hasattr(lib, name), name


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    binding = importlib.import_module("c-attl3_amd.binding")
    monkeypatch.setattr(binding, "_lib", None)
    monkeypatch.setattr(binding, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(pkg.CattleHipError):
        binding.lib()
