"""Loader of the PyTorch-ROCm extension (``csrc/torch_binding.cpp`` -> ``_torchgt_ext.so``): the
``torch.ops.torchgt.*`` operators with C++ autograd functions over the C ABI.  There is no fallback: a
missing extension raises with the build command."""
import os

import torch

from . import _lib

HERE = os.path.dirname(os.path.abspath(__file__))
EXT_PATH = os.path.join(HERE, "_torchgt_ext.so")
_loaded = False


def ops():
    """``torch.ops.torchgt`` with the extension loaded."""
    global _loaded
    if not _loaded:
        _lib.lib()                      # libtorchgt_hip.so first: the extension links against it
        if not os.path.exists(EXT_PATH):
            raise RuntimeError(f"{EXT_PATH} is not built; run `python -m torchgt_amd.build` "
                               "(there is no Python fallback for the operators)")
        torch.ops.load_library(EXT_PATH)
        _loaded = True
    return torch.ops.torchgt
