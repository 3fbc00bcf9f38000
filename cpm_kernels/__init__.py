"""Drop-in name for the reference package: ``import cpm_kernels.kernels as ck`` and
``import cpm_kernels.torch as ct`` resolve to the MI355X implementation in cpm_kernels_amd.
``library``, ``device`` and ``kernels`` are the very same module objects (aliased in
``sys.modules``); ``cpm_kernels.torch`` re-exports ``cpm_kernels_amd.torch`` on first import."""
import importlib
import sys

from cpm_kernels_amd import *  # noqa: F401,F403

for _sub in ("library", "device", "kernels"):
    _mod = importlib.import_module("cpm_kernels_amd." + _sub)
    sys.modules[__name__ + "." + _sub] = _mod
    globals()[_sub] = _mod
