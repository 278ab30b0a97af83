"""little-gemma verify step for MI355X: Python-side plumbing.

The product is the C-ABI HIP library (csrc/liblg_hip.so, declared in include/lg_hip.h)
and the C host layer (host/).  This package only loads those libraries through ctypes
for the tests, the smoke check and the benchmark; it contains no compute and no CPU
fallback: every call fails loudly if the HIP library is missing.

The directory name contains a hyphen, so import it with
``importlib.import_module("little-gemma_amd")``.
"""
from . import hostlib, synth  # noqa: F401
from .hiplib import HipBackend, load_hip, HipError  # noqa: F401
