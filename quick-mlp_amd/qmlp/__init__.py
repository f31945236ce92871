"""QuickMLP for MI355X: fused input encodings + fp16 MLP as run-time generated HIP kernels.

Mirrors the Python package of the reference (src_py/qmlp/__init__.py:1-14).
"""
from ._version import __version__
from .activation import FusedActivation
from .encoding import FusedEncoding
from .network import FusedNetwork, SimulatedNetwork, copy_torch_to_fused
from . import pullpush   # qmlp.pullpush.pullpush(mask, data), like the reference's module
from .classes import Activation, Encoding, Network, QuickMLP
from ._lib import QmlpError, set_kernel_cache_dir, set_log_level


_torch_classes = None


def load_library():
    """Registers the torch custom classes ``torch.classes.qmlp_cu.{QuickMLP, Network, Encoding,
    Activation, utils}`` (like ``load_library`` of the reference, src_py/qmlp/import_library.py:5-39)
    and returns that namespace. The modules of this package do not need them (they call the C ABI
    directly); scripted or traced modules that are to be saved with TorchScript do."""
    global _torch_classes
    if _torch_classes is None:
        import os
        import torch
        from . import _lib
        path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libqmlp_torch.so")
        if not os.path.exists(path):
            raise ImportError("%s has not been built: make -C quick-mlp_amd/csrc/torch (or __graft_entry__.build())" % path)
        torch.classes.load_library(path)
        _torch_classes = torch.classes.qmlp_cu
    return _torch_classes


__all__ = [
    "__version__", "load_library", "FusedActivation", "FusedEncoding", "FusedNetwork", "SimulatedNetwork",
    "copy_torch_to_fused", "pullpush", "Activation", "Encoding", "Network", "QuickMLP", "QmlpError",
    "set_kernel_cache_dir", "set_log_level"]
