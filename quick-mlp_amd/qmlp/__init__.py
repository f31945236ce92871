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


def load_library():
    """Kept for API compatibility: the native library is loaded when the package is imported."""
    from . import _lib
    return _lib.LIB_PATH


__all__ = [
    "__version__", "load_library", "FusedActivation", "FusedEncoding", "FusedNetwork", "SimulatedNetwork",
    "copy_torch_to_fused", "pullpush", "Activation", "Encoding", "Network", "QuickMLP", "QmlpError",
    "set_kernel_cache_dir", "set_log_level"]
