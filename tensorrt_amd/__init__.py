"""MI355X-native BERT encoder plugins (embLayerNorm, skipLayerNorm, QKV-to-context).

The product is ``lib/libtrtamd_bert_plugins.so``: hand-written gfx950 kernels behind a C ABI
(``include/trtamd_bert_kernels.h``) and the IPluginV3 host classes registered under the reference's
plugin names.  This package is the thin Python side: it locates and loads that library and exposes
ctypes bindings (``tensorrt_amd.capi``) plus a plugin-level driver (``tensorrt_amd.plugin``).
There is no CPU fallback: if the library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os

__all__ = ["library_path", "load_library", "LibraryNotBuilt"]

_ROOT = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_ROOT, "lib", "libtrtamd_bert_plugins.so")
_handle = None


class LibraryNotBuilt(RuntimeError):
    pass


def library_path() -> str:
    return _LIB


def load_library() -> ctypes.CDLL:
    """dlopen the plugin library (once).  Raises LibraryNotBuilt when it has not been compiled."""
    global _handle
    if _handle is None:
        if not os.path.exists(_LIB):
            raise LibraryNotBuilt(
                f"{_LIB} is missing: run `python -m tensorrt_amd.build` (needs hipcc); there is no fallback path")
        _handle = ctypes.CDLL(_LIB, mode=ctypes.RTLD_GLOBAL)
    return _handle
