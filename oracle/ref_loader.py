"""Loads ``oracle/_ref/_optimized_transducer.so`` (TEST INFRASTRUCTURE ONLY).

That shared object is the reference's own CPU path (cpu.cc, transducer-loss.cc
and the pybind11 module of optimized_transducer/python/csrc/optimized_transducer.cc)
compiled by ``make -C oracle ref``.  It exists only where that recipe has been
run; ``load()`` returns None elsewhere.
"""
import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_ref", "_optimized_transducer.so")
_mod = None


def available():
    return os.path.exists(_PATH)


def load():
    """The compiled reference module, or None when it has not been built."""
    global _mod
    if _mod is None and available():
        import torch  # noqa: F401  (the module links against libtorch)
        spec = importlib.util.spec_from_file_location("_optimized_transducer", _PATH)
        _mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_mod)
    return _mod
