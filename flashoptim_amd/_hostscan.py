"""Loader of the optional C++ helper that validates cached launch plans (flashoptim_amd/hostscan/fo_hostscan.cpp).

``scan`` and ``same_objects`` are None when the module has not been built (``make -C flashoptim_amd/hostscan``) or
was built against another torch: the optimizer then walks its parameters in Python, 0.25 us per parameter instead of
0.06.  Host-side bookkeeping only; the step itself has no fallback (flashoptim_amd/_native.py).
``FLASHOPTIM_NO_HOSTSCAN=1`` keeps the Python walk.
"""

from __future__ import annotations

import importlib.util
import os

scan = None
same_objects = None

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "_fo_hostscan.so")


def _load() -> None:
    global scan, same_objects
    if os.environ.get("FLASHOPTIM_NO_HOSTSCAN", "").strip() not in ("", "0") or not os.path.exists(_PATH):
        return
    try:
        spec = importlib.util.spec_from_file_location("_fo_hostscan", _PATH)
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
    except (ImportError, OSError):  # built against another torch or python: keep the Python walk
        return
    scan, same_objects = module.scan, module.same_objects


def library_path() -> str:
    return _PATH


_load()
