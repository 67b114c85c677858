"""Locating and loading the package's native libraries.

Every library is built in-tree (see ``orion_amd/csrc/Makefile``) and loaded by
absolute path.  There is no fallback: a missing library raises, because a
silent CPU path would invalidate every parity and performance claim.
"""

import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))

KERNELS_LIB = os.path.join(PKG_DIR, "liborion_kernels.so")
POLICY_LIB = os.path.join(PKG_DIR, "liborion_policy.so")
CAPTURE_LIB = os.path.join(PKG_DIR, "libinttemp.so")
SCHEDULER_LIB = os.path.join(PKG_DIR, "scheduler_eval.so")
# loaded by libinttemp.so itself, at run time (csrc/capture/tls_fresh.h)
TLS_HELPER_LIB = os.path.join(PKG_DIR, "liborion_tlsfresh.so")


class NativeLibraryMissing(RuntimeError):
    pass


_cache = {}


def load(path, mode=ctypes.DEFAULT_MODE):
    """``ctypes.CDLL`` of an in-tree library; raises if it has not been built."""
    lib = _cache.get(path)
    if lib is not None:
        return lib
    if not os.path.exists(path):
        raise NativeLibraryMissing(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; "
            f"g.build()'` (or `make -C orion_amd/csrc`) first")
    lib = ctypes.CDLL(path, mode=mode)
    _cache[path] = lib
    return lib


def loaded(path):
    """The handle ``load`` returned for ``path``, or None."""
    return _cache.get(path)


def unload(path):
    """Closes a library loaded here; its handle must not be used afterwards."""
    lib = _cache.pop(path, None)
    if lib is not None:
        import _ctypes
        _ctypes.dlclose(lib._handle)
