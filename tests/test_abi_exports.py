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


class _FakeTensor(object):
    """Stands in for a DeviceTensor: the wrapper's checks read shape and dtype only and must fire before any call."""

    def __init__(self, shape, dtype="float32"):
        import numpy as np
        self.shape, self.dtype, self.ptr = tuple(shape), np.dtype(dtype), None


@pytest.mark.parametrize("what, kw", [
    ("weights rows", dict(weights=_FakeTensor((26, 8)))),
    ("bias shape", dict(bias=_FakeTensor((8, 1)))),
    ("out extent", dict(out=_FakeTensor((4, 6, 5, 8)))),
    ("out filters", dict(out=_FakeTensor((4, 6, 6, 7)))),
    ("out dtype", dict(out=_FakeTensor((4, 6, 6, 8), "float64"))),
    ("weights dtype", dict(weights=_FakeTensor((27, 8), "float64"))),
    ("rank", dict(x=_FakeTensor((4, 6, 6)))),
    ("receptor larger than input", dict(receptor_height=9)),
])
def test_noalloc_wrapper_refuses_mismatched_buffers(monkeypatch, what, kw):
    """The C entry point takes raw addresses: the Python wrapper is where extents can be checked. Every mismatch must be
    refused before the library is called (the library is replaced by an object that fails on any use)."""
    binding = importlib.import_module("c-attl3_amd.binding")

    class Untouchable(object):
        def __getattr__(self, name):
            raise AssertionError("the library was called: " + name)

    monkeypatch.setattr(binding, "_lib", Untouchable())
    args = dict(x=_FakeTensor((4, 6, 6, 3)), weights=_FakeTensor((27, 8)), bias=_FakeTensor((1, 8)), out=_FakeTensor((4, 6, 6, 8)))
    geom = {}
    for k, v in kw.items():
        (args if k in args else geom)[k] = v
    with pytest.raises(ValueError):
        binding.conv_forward_noalloc(args["x"], args["weights"], args["bias"], args["out"], **geom)
