"""Loads the in-tree PyTorch extension ``selective_scan_cuda_oflex`` (vmamba_amd/csrc/torch_ext.cpp).

The reference decides at import time which selective-scan backend it has by trying
``import selective_scan_cuda_oflex`` (classification/models/csms6s.py:9-14).  ``install()`` makes that import
resolve to this package's HIP-backed shim, so unmodified reference code picks it up.
"""
import importlib
import importlib.util
import os
import sys

from .build import torch_ext_path

MODULE_NAME = "selective_scan_cuda_oflex"


def load():
    """Import and return the extension module; raises ImportError when it has not been built."""
    if MODULE_NAME in sys.modules:
        return sys.modules[MODULE_NAME]
    path = torch_ext_path()
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python -m vmamba_amd.build`")
    import torch  # noqa: F401  (the extension links against libtorch)
    spec = importlib.util.spec_from_file_location(MODULE_NAME, path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def install():
    """Register the module under its reference name so that ``import selective_scan_cuda_oflex`` finds it."""
    module = load()
    sys.modules[MODULE_NAME] = module
    return module
