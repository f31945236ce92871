"""ctypes binding of libqmlp.so (the C ABI declared in include/qmlp_capi.h).

There is no fallback: if the native library is missing, importing this module fails.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libqmlp.so")
DEFAULT_CACHE_DIR = os.path.join(os.path.dirname(_HERE), ".kernel_cache")

QMLP_FLOAT, QMLP_HALF, QMLP_DOUBLE = 0, 1, 2
QMLP_INFERENCE, QMLP_GRADIENTS = 0, 1
GRADIENTS_INPUT, GRADIENTS_NETWORK_WEIGHTS, GRADIENTS_INPUT_ENCODINGS = 1, 2, 4


class QmlpError(RuntimeError):
    """An error reported by the native library (configuration, shape/type or device)."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


class TensorDesc(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("precision", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("sizes", ctypes.c_int32 * 4), ("strides", ctypes.c_int32 * 4)]


if not os.path.exists(LIB_PATH):
    raise ImportError(
        "The native QuickMLP library %s has not been built. Build it with "
        "`make -C quick-mlp_amd/csrc` (or __graft_entry__.build())." % LIB_PATH)

lib = ctypes.CDLL(LIB_PATH)
lib.qmlp_last_error.restype = ctypes.c_char_p
lib.qmlp_free_string.argtypes = [ctypes.c_void_p]
lib.qmlp_free_string.restype = None

_P = ctypes.POINTER
_TD = _P(TensorDesc)
_vp = ctypes.c_void_p
_ci = ctypes.c_int
_pi = _P(ctypes.c_int)
_pstr = _P(ctypes.c_void_p)   # char** returned strings (freed with qmlp_free_string)

_SIGNATURES = {
    "qmlp_is_gpu_available": [_pi],
    "qmlp_set_log_level": [ctypes.c_char_p],
    "qmlp_set_compile_debug_mode": [_ci],
    "qmlp_is_compile_debug_mode": [_pi],
    "qmlp_set_kernel_cache_dir": [ctypes.c_char_p],
    "qmlp_kernel_cache_stats": [_pi, _pi],
    "qmlp_kernel_compiler_stats": [_pi, _pi],
    "qmlp_network_create": [ctypes.c_char_p, ctypes.c_char_p, _P(_vp)],
    "qmlp_network_destroy": [_vp],
    "qmlp_network_channels_in": [_vp, _pi],
    "qmlp_network_channels_out": [_vp, _pi],
    "qmlp_network_num_layers": [_vp, _pi],
    "qmlp_network_num_encodings": [_vp, _pi],
    "qmlp_network_encoding": [_vp, _ci, _P(_vp)],
    "qmlp_network_parameter_count": [_vp, _pi],
    "qmlp_network_parameter_precision": [_vp, _ci, _pi],
    "qmlp_network_matrix_size": [_pi],
    "qmlp_network_warp_size": [_pi],
    "qmlp_network_max_shared_memory_bytes": [_pi],
    "qmlp_network_is_parallel_streams": [_vp, _pi],
    "qmlp_network_set_parallel_streams": [_vp, _ci],
    "qmlp_network_set_parameter": [_vp, _TD, _ci],
    "qmlp_network_initialize_inference_parameters": [_vp, ctypes.c_uint32],
    "qmlp_network_parameter_view": [_vp, _ci, _ci, _vp, _ci, _TD],
    "qmlp_network_inference": [_vp, _TD, _TD, _vp],
    "qmlp_network_inference_noalloc": [_vp, _TD, _TD, _vp],
    "qmlp_network_forward_memory": [_vp, _ci, _ci, _P(ctypes.c_size_t)],
    "qmlp_network_forward": [_vp, _TD, _TD, _vp, _vp],
    "qmlp_network_zero_gradients": [_vp],
    "qmlp_network_adjoint_memory": [_vp, _ci, _ci, _P(ctypes.c_size_t)],
    "qmlp_network_adjoint": [_vp, _TD, _TD, _ci, _TD, _vp, _vp, _vp],
    "qmlp_network_clear_cached_kernels": [_vp],
    "qmlp_network_precompile": [_vp, _ci],
    "qmlp_network_prepare": [_vp, _ci, _ci],
    "qmlp_network_generated_source": [_vp, ctypes.c_char_p, _ci, _pstr],
    "qmlp_encoding_create": [ctypes.c_char_p, _P(_vp)],
    "qmlp_encoding_destroy": [_vp],
    "qmlp_encoding_to_json": [_vp, _pstr],
    "qmlp_encoding_id": [_vp, _pstr],
    "qmlp_encoding_max_input_channel": [_vp, _pi],
    "qmlp_encoding_num_output_channels": [_vp, _pi],
    "qmlp_encoding_has_parameters": [_vp, _pi],
    "qmlp_encoding_parameter_count": [_vp, _pi],
    "qmlp_encoding_parameter_precision": [_vp, _ci, _pi],
    "qmlp_encoding_set_parameter": [_vp, _TD, _ci],
    "qmlp_encoding_zero_gradients": [_vp],
    "qmlp_encoding_forward": [_vp, _TD, _TD, _vp, _TD],
    "qmlp_encoding_adjoint": [_vp, _TD, _TD, _TD, _vp, _TD, _TD, _ci],
    "qmlp_encoding_hashgrid_levels": [_vp, _ci, _pi, _pi, _pi, _pi, _pi],
    "qmlp_encoding_hashgrid_corners": [_vp, _TD, _vp, _vp, _vp],
    "qmlp_encoding_hashgrid_trace": [_vp, _TD, _ci, _vp, _vp, _vp],
    "qmlp_encoding_precompile": [_vp, _ci],
    "qmlp_activation_create": [ctypes.c_char_p, _P(_vp)],
    "qmlp_activation_destroy": [_vp],
    "qmlp_activation_to_json": [_vp, _pstr],
    "qmlp_activation_forward": [_vp, _TD, _TD, _vp],
    "qmlp_activation_adjoint": [_vp, _TD, _TD, _TD, _vp],
    "qmlp_activation_precompile": [_vp],
    "qmlp_utils_pullpush_forward": [_TD, _TD, _TD, _vp],
    "qmlp_utils_pullpush_adjoint": [_TD, _TD, _TD, _TD, _TD, _vp],
    "qmlp_utils_pullpush_precompile": [_ci],
}
for _name, _args in _SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.argtypes = _args
    _fn.restype = ctypes.c_int


def check(rc):
    if rc != 0:
        raise QmlpError(rc, lib.qmlp_last_error().decode("utf-8", "replace"))


def get_int(fn, *args):
    v = ctypes.c_int()
    check(fn(*args, ctypes.byref(v)))
    return v.value


def get_string(fn, *args):
    p = ctypes.c_void_p()
    check(fn(*args, ctypes.byref(p)))
    try:
        return ctypes.string_at(p.value).decode("utf-8")
    finally:
        lib.qmlp_free_string(p)


_PRECISION_OF = {torch.float32: QMLP_FLOAT, torch.float16: QMLP_HALF, torch.float64: QMLP_DOUBLE}
DTYPE_OF = {QMLP_FLOAT: torch.float32, QMLP_HALF: torch.float16, QMLP_DOUBLE: torch.float64}


# one pack call per descriptor: field-by-field assignment of a ctypes structure costs more than
# the launch of a small kernel
_PACK = {n: __import__("struct").Struct("<Qii%di%dx%di%dx" % (n, 4 * (4 - n), n, 4 * (4 - n))) for n in range(1, 5)}


def desc(t):
    """Tensor descriptor of a torch tensor (None -> undefined tensor)."""
    if t is None:
        return TensorDesc()
    n = t.dim()
    if t.dtype not in _PRECISION_OF:
        raise TypeError("unsupported dtype %s" % t.dtype)
    if n < 1 or n > 4:
        raise ValueError("tensors must have 1 to 4 dimensions")
    return TensorDesc.from_buffer_copy(_PACK[n].pack(t.data_ptr(), _PRECISION_OF[t.dtype], n, *t.shape, *t.stride()))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device=None):
    """Handle of torch's current HIP stream as a void*."""
    if _raw_stream is not None and isinstance(device, torch.device) and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))      # no Stream object: this sits on every call
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def set_log_level(level):
    check(lib.qmlp_set_log_level(level.encode()))


def set_kernel_cache_dir(path):
    check(lib.qmlp_set_kernel_cache_dir((path or "").encode()))


def kernel_cache_stats():
    a, b = ctypes.c_int(), ctypes.c_int()
    check(lib.qmlp_kernel_cache_stats(ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def kernel_compiler_stats():
    """(whether the offline compiler of the installed ROCm takes the kernels that ask for it, how many it compiled so far)"""
    a, b = ctypes.c_int(), ctypes.c_int()
    check(lib.qmlp_kernel_compiler_stats(ctypes.byref(a), ctypes.byref(b)))
    return bool(a.value), b.value


set_kernel_cache_dir(os.environ.get("QMLP_CACHE_DIR", DEFAULT_CACHE_DIR))
