"""Loader of ``valora_amd/_binding.so``, the torch extension module with the reference's op entry points
(``csrc/binding.cpp``).  There is no Python or CPU stand-in: a missing module is an error."""
from __future__ import annotations

import os

import torch  # noqa: F401  (the extension links against the torch libraries this import loads)

from . import _lib

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_binding.so")
if not os.path.exists(_PATH):
    raise ImportError(f"{_PATH} is missing: build it with `python -m valora_amd._build` "
                      "(hipcc --offload-arch=gfx950 for libmlora.so, g++ for the binding); there is no fallback path")
_lib.lib()          # libmlora.so first, by its path, so that the extension's dependency resolves to this very file
from . import _binding as binding  # noqa: E402
