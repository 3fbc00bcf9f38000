"""Loader for the C-ABI shared library, mirroring the behaviour of the reference's generic
``Lib`` class (cpm_kernels/library/base.py:41-96):

* a library that cannot be found does not break ``import``: every bound function becomes a
  stub that raises ``RuntimeError("Library ... is not initialized")`` when called;
* a symbol that is missing from a found library raises ``AttributeError`` when called and
  logs a warning at bind time.

Search order: ``$CPMK_LIBRARY`` (explicit file), the in-tree build
``cpm_kernels_amd/lib/libcpmk_hip.so``, then the system linker path.

One process must use one HIP runtime: a ``hipStream_t`` or device pointer made by one copy of
``libamdhip64`` means nothing to another, and a second copy that initialises after the first
finds no usable device.  PyTorch-ROCm wheels ship their own ``libamdhip64.so`` and load it by
path, so if this library were loaded first it would pull in the system copy and the two would
coexist.  ``preload_torch_hip_runtime()`` therefore maps PyTorch's copy first (when PyTorch is
installed and ships one); the ``NEEDED libamdhip64.so.N`` of ``libcpmk_hip.so`` then binds to it
by soname, and a later ``import torch`` finds the very same file already loaded.
"""
import ctypes
import ctypes.util
import logging
import os
import sys
from functools import wraps
from typing import Callable, TypeVar

logger = logging.getLogger(__name__)
LibCall = TypeVar("LibCall")

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


_preloaded = False


def preload_torch_hip_runtime():
    """Map the HIP runtime bundled with PyTorch (if any) before anything links the system one."""
    global _preloaded
    if _preloaded or "torch" in sys.modules:      # torch imported: its runtime is already mapped
        _preloaded = True
        return None
    _preloaded = True
    try:
        import importlib.util
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        return None
    if spec is None or not spec.submodule_search_locations:
        return None
    cand = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
    if not os.path.exists(cand):
        return None
    try:
        ctypes.CDLL(cand, mode=ctypes.RTLD_GLOBAL)
        return cand
    except OSError as e:
        logger.warning("Could not preload %s: %s", cand, e)
        return None


def find_lib(name: str):
    explicit = os.environ.get("CPMK_LIBRARY")
    if explicit:
        return explicit if os.path.exists(explicit) else None
    in_tree = os.path.join(_PKG_DIR, "lib", "lib%s.so" % name)
    if os.path.exists(in_tree):
        return in_tree
    return ctypes.util.find_library(name)


class Lib:
    def __init__(self, name: str, path=None):
        self._name = name
        self._path = path if path is not None else find_lib(name)
        self._lib = None
        self._load_error = None
        if self._path is not None:
            preload_torch_hip_runtime()
            try:
                self._lib = ctypes.CDLL(self._path)
            except OSError as e:          # e.g. libamdhip64.so missing on this host
                self._load_error = str(e)
                logger.warning("Could not load %s: %s", self._path, e)

    @property
    def path(self):
        return self._path

    @property
    def loaded(self) -> bool:
        return self._lib is not None

    def bind(self, name, arg_types, ret_type) -> Callable[[LibCall], LibCall]:
        if self._lib is None:
            def decorator(f):
                @wraps(f)
                def wrapper(*args, **kwargs):
                    raise RuntimeError("Library %s is not initialized" % self._name)
                return wrapper
            return decorator
        try:
            func = getattr(self._lib, name)
        except AttributeError:
            def decorator(f):
                @wraps(f)
                def wrapper(*args, **kwargs):
                    raise AttributeError("%s: undefined symbol: %s" % (self._path, name))
                return wrapper
            logger.warning("Symbol %s not found in %s", name, self._path)
            return decorator
        func.argtypes = arg_types
        func.restype = ret_type
        setattr(self, name, func)

        def decorator(f):
            @wraps(f)
            def wrapper(*args, **kwargs):
                return f(*args, **kwargs)
            return wrapper
        return decorator
