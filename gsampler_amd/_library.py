"""Loads the C++ operator library (libgs.so) into torch.  There is no fallback:
a missing library is an import error that says how to build it."""
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "lib", "libgs.so")
_loaded = False


def load() -> None:
    global _loaded
    if _loaded:
        return
    if not os.path.exists(SO_PATH):
        raise ImportError(
            f"{SO_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; "
            "g.build()'` (make -C gsampler_amd/csrc && python gsampler_amd/csrc/host/build.py)")
    torch.classes.load_library(SO_PATH)
    _loaded = True
