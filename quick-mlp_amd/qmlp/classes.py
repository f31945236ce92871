"""Python counterparts of the custom classes the reference registers as
``torch.classes.qmlp_cu.{QuickMLP, Network, Encoding, Activation}``
(src_cpp/pytorch-bindings/src/bindings.cpp:102-122, bind_network.cpp:346-411,
bind_encoding.cpp:165-197, bind_activation.cpp:80-98), same method names and
argument meaning, implemented on the C ABI of libqmlp.so. torch only provides
device memory, the current stream and autograd bookkeeping here.
"""
import ctypes
import json
import threading

import torch

from . import _lib
from ._lib import (GRADIENTS_INPUT, GRADIENTS_INPUT_ENCODINGS, GRADIENTS_NETWORK_WEIGHTS,
                   QMLP_GRADIENTS, QMLP_INFERENCE, check, current_stream, desc, lib)


def _device_of(t):
    if not t.is_cuda:
        raise RuntimeError("QuickMLP tensors must live on the GPU")
    return t.device


def _create_output(input, channels):
    if input.dim() != 2:
        raise RuntimeError("input must be a tensor with 2 dimensions (batch, channels)")
    return torch.empty((input.shape[0], channels), dtype=input.dtype, device=input.device)


class QuickMLP:
    """Global settings (bindings.cpp:104-113)."""

    @staticmethod
    def set_compile_debug_mode(enable):
        check(lib.qmlp_set_compile_debug_mode(1 if enable else 0))

    @staticmethod
    def is_compile_debug_mode():
        return bool(_lib.get_int(lib.qmlp_is_compile_debug_mode))

    @staticmethod
    def set_log_level(level):
        _lib.set_log_level(level)

    @staticmethod
    def is_cuda_available():
        return bool(_lib.get_int(lib.qmlp_is_gpu_available))

    is_gpu_available = is_cuda_available


# ---------------------------------------------------------------------------- activation
class _ActivationFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, activ):
        ctx.save_for_backward(input)
        ctx.activ = activ
        return activ.inference(input)

    @staticmethod
    def backward(ctx, grad_output):
        (input,) = ctx.saved_tensors
        return ctx.activ.adjoint(input, grad_output.contiguous()), None


class Activation:
    """A built-in activation id or an inline JSON specification; half tensors only."""

    def __init__(self, cfg):
        self._cfg = cfg
        self._handle = ctypes.c_void_p()
        check(lib.qmlp_activation_create(cfg.encode(), ctypes.byref(self._handle)))

    def __del__(self):
        if getattr(self, "_handle", None):
            lib.qmlp_activation_destroy(self._handle)
            self._handle = None

    def cfg(self):
        return self._cfg

    def to_json(self):
        return _lib.get_string(lib.qmlp_activation_to_json, self._handle)

    def precompile(self):
        """Compiles the standalone kernels into the kernel cache; needs no GPU."""
        check(lib.qmlp_activation_precompile(self._handle))

    def inference(self, input):
        _device_of(input)
        output = torch.empty_like(input)
        check(lib.qmlp_activation_forward(self._handle, desc(input), desc(output), current_stream(input.device)))
        return output

    def adjoint(self, input, adj_output):
        adj_input = torch.empty_like(input)
        check(lib.qmlp_activation_adjoint(self._handle, desc(input), desc(adj_output), desc(adj_input),
                                          current_stream(input.device)))
        return adj_input

    def forward(self, input):
        return _ActivationFunction.apply(input, self)

    def __getstate__(self):
        return self._cfg

    def __setstate__(self, state):
        self.__init__(state)


# ---------------------------------------------------------------------------- encoding
class _EncodingFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, enc):
        ctx.save_for_backward(input)
        ctx.enc = enc
        return enc.inference(input)

    @staticmethod
    def backward(ctx, grad_output):
        (input,) = ctx.saved_tensors
        return ctx.enc.adjoint(input, grad_output.contiguous()), None


class _EncodingFunctionWithParameter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, parameter, enc):
        ctx.save_for_backward(input, parameter)
        ctx.enc = enc
        ctx.flags = (1 if input.requires_grad else 0) | (2 if parameter.requires_grad else 0)
        return enc.inference_with_parameter(input, parameter)

    @staticmethod
    def backward(ctx, grad_output):
        input, parameter = ctx.saved_tensors
        if ctx.flags == 0:
            return None, None, None
        gi, gp = ctx.enc.adjoint_with_parameter_and_flags(input, parameter, grad_output.contiguous(), ctx.flags)
        return (gi if ctx.flags & 1 else None), (gp if ctx.flags & 2 else None), None


class Encoding:
    """One input encoding, standalone (fp32 in, fp32 out)."""

    def __init__(self, cfg=None, _borrowed=None, _owner=None):
        self._owner = _owner          # keeps the network alive for borrowed handles
        self._borrowed = _borrowed is not None
        if _borrowed is not None:
            self._handle = _borrowed
            self._cfg = self.to_json()
        else:
            self._cfg = cfg
            self._handle = ctypes.c_void_p()
            check(lib.qmlp_encoding_create(cfg.encode(), ctypes.byref(self._handle)))

    def __del__(self):
        if getattr(self, "_handle", None) and not self._borrowed:
            lib.qmlp_encoding_destroy(self._handle)
        self._handle = None

    def cfg(self):
        return self._cfg

    def to_json(self):
        return _lib.get_string(lib.qmlp_encoding_to_json, self._handle)

    def id(self):
        return _lib.get_string(lib.qmlp_encoding_id, self._handle)

    def max_input_channel(self):
        return _lib.get_int(lib.qmlp_encoding_max_input_channel, self._handle)

    def num_output_channels(self):
        return _lib.get_int(lib.qmlp_encoding_num_output_channels, self._handle)

    def has_parameters(self):
        # fixed by the specification: asked once (this sits on the per-call path of the network)
        if getattr(self, "_has_parameters", None) is None:
            self._has_parameters = bool(_lib.get_int(lib.qmlp_encoding_has_parameters, self._handle))
        return self._has_parameters

    def num_parameters(self):
        return _lib.get_int(lib.qmlp_encoding_parameter_count, self._handle)

    def parameter_dtype(self, gradients=False):
        p = _lib.get_int(lib.qmlp_encoding_parameter_precision, self._handle,
                         QMLP_GRADIENTS if gradients else QMLP_INFERENCE)
        return _lib.DTYPE_OF[p]

    def create_inference_parameters(self, device="cuda"):
        if not self.has_parameters():
            raise RuntimeError("the encoding has no parameters")
        return torch.empty((self.num_parameters(),), dtype=self.parameter_dtype(False), device=device)

    def create_gradient_parameters(self, device="cuda"):
        if not self.has_parameters():
            raise RuntimeError("the encoding has no parameters")
        return torch.empty((self.num_parameters(),), dtype=self.parameter_dtype(True), device=device)

    def set_parameter(self, tensor, gradients=False):
        if not gradients:
            # binding the same memory again changes nothing: skipped, this sits on every call of a network
            key = None if tensor is None else (tensor.data_ptr(), tensor.numel(), tensor.dtype)
            if key is not None and key == getattr(self, "_bound_inference", None):
                return
            self._bound_inference = key
        check(lib.qmlp_encoding_set_parameter(self._handle, desc(tensor),
                                              QMLP_GRADIENTS if gradients else QMLP_INFERENCE))

    def precompile(self, adjoint_mode=3):
        """Compiles the standalone kernels into the kernel cache (needs no GPU)."""
        check(lib.qmlp_encoding_precompile(self._handle, int(adjoint_mode)))

    def hashgrid_levels(self):
        """[(resolution, hashed, memory_offset, hash_grid_size)] of a HashGrid encoding."""
        n = ctypes.c_int()
        cap = 64
        arrs = [(ctypes.c_int * cap)() for _ in range(4)]
        check(lib.qmlp_encoding_hashgrid_levels(self._handle, cap, ctypes.byref(n), *arrs))
        off, res, hs, hashed = arrs
        return [(res[l], bool(hashed[l]), off[l], hs[l]) for l in range(n.value)]

    def hashgrid_corners(self, input, mode=0):
        """Device-computed table offsets and weights, shape (N, levels, 2^dim). mode 0: the index
        function; 1: what the gathers of the fused forward kernels use (bind a table first);
        2: what the gradient scatter of the fused backward kernel adds to; 3: what the gradient
        records of large batches (sums per slice of the table) stand for; 4: the elements behind the
        sums of the column kernel (single dense levels whose batches train sorted by slab)."""
        if input is None:      # compile the kernel of this mode into the kernel cache, nothing runs
            check(lib.qmlp_encoding_hashgrid_trace(self._handle, None, int(mode), None, None, None))
            return None
        levels = self.hashgrid_levels()
        dim = int(json.loads(self.to_json())["n_in"])
        n = input.shape[0]
        idx = torch.full((n, len(levels), 1 << dim), -1, dtype=torch.int32, device=input.device)
        w = torch.full((n, len(levels), 1 << dim), float("nan"), dtype=torch.float32, device=input.device)
        check(lib.qmlp_encoding_hashgrid_trace(self._handle, desc(input), int(mode), idx.data_ptr(), w.data_ptr(),
                                               current_stream(input.device)))
        return idx, w

    def inference(self, input):
        if self.has_parameters():
            raise RuntimeError("Encoding has parameters, call the variation of 'inference' with parameters")
        _device_of(input)
        output = _create_output(input, self.num_output_channels())
        check(lib.qmlp_encoding_forward(self._handle, desc(input), desc(output), current_stream(input.device), None))
        return output

    def inference_with_parameter(self, input, parameter_forward):
        if not self.has_parameters():
            raise RuntimeError("Encoding doesn't have parameters, call the variation of 'inference' without parameters")
        _device_of(input)
        output = _create_output(input, self.num_output_channels())
        check(lib.qmlp_encoding_forward(self._handle, desc(input), desc(output), current_stream(input.device),
                                        desc(parameter_forward)))
        # the native call binds the table for its own duration and leaves the encoding unbound
        self._bound_inference = None
        return output

    def adjoint(self, input, adj_output):
        if self.has_parameters():
            raise RuntimeError("Encoding has parameters, call the variation of 'adjoint' with parameters")
        adj_input = torch.zeros_like(input)
        check(lib.qmlp_encoding_adjoint(self._handle, desc(input), desc(adj_output), desc(adj_input),
                                        current_stream(input.device), None, None, 3))
        return adj_input

    def adjoint_with_parameter(self, input, parameter_forward, adj_output):
        return self.adjoint_with_parameter_and_flags(input, parameter_forward, adj_output, 3)

    def adjoint_with_parameter_and_flags(self, input, parameter_forward, adj_output, flags):
        if not self.has_parameters():
            raise RuntimeError("Encoding doesn't have parameters, call the variation of 'adjoint' without parameters")
        adj_input = torch.zeros_like(input)
        adj_param = torch.zeros(parameter_forward.shape, dtype=self.parameter_dtype(True),
                                device=parameter_forward.device)
        check(lib.qmlp_encoding_adjoint(self._handle, desc(input), desc(adj_output), desc(adj_input),
                                        current_stream(input.device), desc(parameter_forward), desc(adj_param),
                                        int(flags)))
        self._bound_inference = None   # as in inference_with_parameter
        return adj_input, adj_param.to(parameter_forward.dtype)

    def forward(self, input):
        if self.has_parameters():
            raise RuntimeError("Encoding has parameters, call the variation of 'forward' with parameters")
        return _EncodingFunction.apply(input, self)

    def forward_with_parameter(self, input, parameter):
        if not self.has_parameters():
            raise RuntimeError("Encoding doesn't have parameters, call the variation of 'forward' without parameters")
        return _EncodingFunctionWithParameter.apply(input, parameter, self)

    def __getstate__(self):
        return self._cfg

    def __setstate__(self, state):
        self.__init__(state)


# ---------------------------------------------------------------------------- network
class _NetworkFunction(torch.autograd.Function):
    """Differentiable fused forward (bind_network.cpp:189-319)."""

    @staticmethod
    def forward(ctx, net, flags, input, network_parameters, *encoding_parameters):
        ctx.net = net
        ctx.flags = flags
        ctx.param_dtype = network_parameters.dtype
        np16 = network_parameters if network_parameters.dtype == torch.float16 else network_parameters.to(torch.float16)
        nbytes = net.forward_memory(input.shape[0], flags)
        tmp_forward = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=input.device)
        output = _create_output(input, net.channels_out())
        with net._mutex:
            net._set_network_parameters(np16, encoding_parameters)
            check(lib.qmlp_network_forward(net._handle, desc(input), desc(output),
                                           ctypes.c_void_p(tmp_forward.data_ptr()), current_stream(input.device)))
        ctx.save_for_backward(input, np16, tmp_forward, *encoding_parameters)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        net, flags = ctx.net, ctx.flags
        input, np16, tmp_forward = ctx.saved_tensors[:3]
        encoding_parameters = ctx.saved_tensors[3:]
        grad_output = grad_output.contiguous()
        adj_input = torch.zeros_like(input) if flags & GRADIENTS_INPUT else None
        adj_network = None
        adj_encodings = [None] * len(encoding_parameters)
        with net._mutex:
            net._set_network_parameters(np16, encoding_parameters)
            if flags & GRADIENTS_NETWORK_WEIGHTS:
                adj_network = torch.zeros(np16.shape, dtype=torch.float32, device=np16.device)
                check(lib.qmlp_network_set_parameter(net._handle, desc(adj_network), QMLP_GRADIENTS))
            if flags & GRADIENTS_INPUT_ENCODINGS:
                for i, p in enumerate(encoding_parameters):
                    enc = net.encoding(i)
                    # the kernel adds the gradients of every encoding with parameters: a frozen one
                    # gets a zero tensor as well, which is dropped below (bind_network.cpp:277-290)
                    if enc.has_parameters():
                        adj_encodings[i] = torch.zeros(p.shape, dtype=enc.parameter_dtype(True), device=p.device)
                        enc.set_parameter(adj_encodings[i], gradients=True)
            nbytes = net.adjoint_memory(input.shape[0], flags)
            tmp_adjoint = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=input.device)
            check(lib.qmlp_network_adjoint(net._handle, desc(input), desc(grad_output), flags, desc(adj_input),
                                           ctypes.c_void_p(tmp_forward.data_ptr()),
                                           ctypes.c_void_p(tmp_adjoint.data_ptr()), current_stream(input.device)))
            # do not leave dangling gradient bindings behind
            check(lib.qmlp_network_set_parameter(net._handle, None, QMLP_GRADIENTS))
            for i, g in enumerate(adj_encodings):
                if g is not None:
                    net.encoding(i).set_parameter(None, gradients=True)
        if adj_network is not None:
            adj_network = adj_network.to(ctx.param_dtype)
        adj_encodings = [g.to(p.dtype) if g is not None and ctx.needs_input_grad[4 + i] else None
                         for i, (g, p) in enumerate(zip(adj_encodings, encoding_parameters))]
        return (None, None, adj_input, adj_network, *adj_encodings)


class Network:
    """The fused network of a JSON configuration (bind_network.h:16-95)."""

    def __init__(self, cfg, parent="."):
        self._cfg = cfg
        self._parent = parent
        self._mutex = threading.Lock()
        self._handle = ctypes.c_void_p()
        check(lib.qmlp_network_create(cfg.encode(), parent.encode(), ctypes.byref(self._handle)))
        self._encodings = {}

    def __del__(self):
        if getattr(self, "_handle", None):
            lib.qmlp_network_destroy(self._handle)
            self._handle = None

    def cfg(self):
        return self._cfg

    def parent(self):
        return self._parent

    @staticmethod
    def MatrixSize():
        return _lib.get_int(lib.qmlp_network_matrix_size)

    @staticmethod
    def WarpSize():
        return _lib.get_int(lib.qmlp_network_warp_size)

    @staticmethod
    def MaxSharedMemoryBytes():
        return _lib.get_int(lib.qmlp_network_max_shared_memory_bytes)

    def is_parallel_streams(self):
        return bool(_lib.get_int(lib.qmlp_network_is_parallel_streams, self._handle))

    def set_parallel_streams(self, enabled):
        check(lib.qmlp_network_set_parallel_streams(self._handle, 1 if enabled else 0))

    def num_encodings(self):
        if getattr(self, "_num_encodings", None) is None:
            self._num_encodings = _lib.get_int(lib.qmlp_network_num_encodings, self._handle)
        return self._num_encodings

    def encoding(self, idx):
        if idx not in self._encodings:
            h = ctypes.c_void_p()
            check(lib.qmlp_network_encoding(self._handle, idx, ctypes.byref(h)))
            self._encodings[idx] = Encoding(_borrowed=h, _owner=self)
        return self._encodings[idx]

    def channels_in(self):
        return _lib.get_int(lib.qmlp_network_channels_in, self._handle)

    def channels_out(self):
        if getattr(self, "_channels_out", None) is None:
            self._channels_out = _lib.get_int(lib.qmlp_network_channels_out, self._handle)
        return self._channels_out

    def num_layers(self):
        return _lib.get_int(lib.qmlp_network_num_layers, self._handle)

    def num_network_parameters(self):
        return _lib.get_int(lib.qmlp_network_parameter_count, self._handle)

    def create_inference_parameters(self, device="cuda"):
        """Uninitialized fp16 tensor of shape (num_network_parameters(),)."""
        return torch.empty((self.num_network_parameters(),), dtype=torch.float16, device=device)

    def initialize_inference_parameters(self, dst):
        """Default (torch.nn.Linear style) initialization of the fp16 tensor 'dst'."""
        with self._mutex:
            check(lib.qmlp_network_set_parameter(self._handle, desc(dst), QMLP_INFERENCE))
            self._bound_inference = (dst.data_ptr(), dst.numel(), dst.dtype)
            seed = int(torch.randint(2 ** 31 - 1, (1,)).item())
            check(lib.qmlp_network_initialize_inference_parameters(self._handle, seed))

    def parameter_view(self, layer, bias, parameters):
        """Read-write view of the weight matrix / bias vector of 'layer' inside 'parameters'."""
        if parameters.dtype not in (torch.float32, torch.float16):
            raise RuntimeError("parameters must be float or half")
        if parameters.dim() != 1 or parameters.shape[0] != self.num_network_parameters():
            raise RuntimeError("The tensor must be of shape (num_parameters, )")
        view = _lib.TensorDesc()
        prec = _lib.QMLP_FLOAT if parameters.dtype == torch.float32 else _lib.QMLP_HALF
        check(lib.qmlp_network_parameter_view(self._handle, int(layer), 1 if bias else 0,
                                              ctypes.c_void_p(parameters.data_ptr()), prec, ctypes.byref(view)))
        if view.ndim == 0:
            return None
        offset = (view.data - parameters.data_ptr()) // parameters.element_size()
        sizes = [view.sizes[i] for i in range(view.ndim)]
        strides = [view.strides[i] for i in range(view.ndim)]
        return torch.as_strided(parameters, sizes, strides, parameters.storage_offset() + offset)

    def forward_memory(self, num_elements, flags):
        n = ctypes.c_size_t()
        check(lib.qmlp_network_forward_memory(self._handle, int(num_elements), int(flags), ctypes.byref(n)))
        return n.value

    def adjoint_memory(self, num_elements, flags):
        n = ctypes.c_size_t()
        check(lib.qmlp_network_adjoint_memory(self._handle, int(num_elements), int(flags), ctypes.byref(n)))
        return n.value

    def precompile(self, adjoint_flags=7):
        check(lib.qmlp_network_precompile(self._handle, int(adjoint_flags)))

    def prepare(self, num_elements, adjoint_flags=0):
        """Loads the kernels and allocates the workspace that calls on a batch of this size need,
        so that those calls only enqueue kernels (e.g. under graph capture)."""
        check(lib.qmlp_network_prepare(self._handle, int(num_elements), int(adjoint_flags)))

    def generated_source(self, kind, adjoint_flags=0):
        return _lib.get_string(lib.qmlp_network_generated_source, self._handle, kind.encode(), int(adjoint_flags))

    def _set_network_parameters(self, network_parameters, encoding_parameters):
        if network_parameters is not None:
            key = (network_parameters.data_ptr(), network_parameters.numel(), network_parameters.dtype)
            if key != getattr(self, "_bound_inference", None):
                check(lib.qmlp_network_set_parameter(self._handle, desc(network_parameters), QMLP_INFERENCE))
                self._bound_inference = key
        m = min(len(encoding_parameters), self.num_encodings())
        for i in range(m):
            p = encoding_parameters[i]
            enc = self.encoding(i)
            if p is not None and enc.has_parameters():
                enc.set_parameter(p, gradients=False)

    def inference(self, input, network_parameters, encoding_parameters=()):
        _device_of(input)
        output = _create_output(input, self.channels_out())
        np16 = network_parameters if network_parameters.dtype == torch.float16 else network_parameters.to(torch.float16)
        with self._mutex:
            self._set_network_parameters(np16, list(encoding_parameters))
            check(lib.qmlp_network_inference(self._handle, desc(input), desc(output), current_stream(input.device)))
        return output

    def inference_noalloc(self, input, output, network_parameters, encoding_parameters=()):
        """inference() into a tensor of the caller through the entry point of the C ABI that
        allocates no device memory (for code under HIP graph capture and the like): the kernels must
        have been loaded by an inference() call on a batch of the same size, the parameters are
        fp16 already, and a batch that is ordered by grid slab has to fit the library's static
        48 MiB workspace. Calls that overlap on one GPU race on that workspace."""
        _device_of(input)
        if network_parameters.dtype != torch.float16:
            raise RuntimeError("inference_noalloc takes fp16 network parameters (a conversion would allocate)")
        with self._mutex:
            self._set_network_parameters(network_parameters, list(encoding_parameters))
            check(lib.qmlp_network_inference_noalloc(self._handle, desc(input), desc(output), current_stream(input.device)))
        return output

    def forward_raw(self, input, network_parameters, encoding_parameters=(), flags=7):
        """forward() of the C ABI without autograd: returns (output, tmp_forward)."""
        _device_of(input)
        output = _create_output(input, self.channels_out())
        nbytes = self.forward_memory(input.shape[0], flags)
        tmp_forward = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=input.device)
        with self._mutex:
            self._set_network_parameters(network_parameters, list(encoding_parameters))
            check(lib.qmlp_network_forward(self._handle, desc(input), desc(output),
                                           ctypes.c_void_p(tmp_forward.data_ptr()), current_stream(input.device)))
        return output, tmp_forward

    def adjoint_raw(self, input, adj_output, flags, tmp_forward, network_parameters, encoding_parameters=(),
                    grad_network=None, grad_encodings=None, adj_input=None):
        """adjoint() of the C ABI without autograd. Gradient tensors that are passed in are
        accumulated into (+=); missing ones are created zero-filled.
        Returns (adj_input, grad_network, grad_encodings)."""
        encoding_parameters = list(encoding_parameters)
        if flags & GRADIENTS_INPUT and adj_input is None:
            adj_input = torch.zeros_like(input)
        if flags & GRADIENTS_NETWORK_WEIGHTS and grad_network is None:
            grad_network = torch.zeros((self.num_network_parameters(),), dtype=torch.float32, device=input.device)
        if grad_encodings is None:
            grad_encodings = [None] * self.num_encodings()
        grad_encodings = list(grad_encodings)
        if flags & GRADIENTS_INPUT_ENCODINGS:
            for i in range(self.num_encodings()):
                enc = self.encoding(i)
                if enc.has_parameters() and grad_encodings[i] is None:
                    grad_encodings[i] = torch.zeros((enc.num_parameters(),), dtype=torch.float32, device=input.device)
        nbytes = self.adjoint_memory(input.shape[0], flags)
        tmp_adjoint = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=input.device)
        with self._mutex:
            self._set_network_parameters(network_parameters, encoding_parameters)
            if flags & GRADIENTS_NETWORK_WEIGHTS:
                check(lib.qmlp_network_set_parameter(self._handle, desc(grad_network), QMLP_GRADIENTS))
            if flags & GRADIENTS_INPUT_ENCODINGS:
                for i, g in enumerate(grad_encodings):
                    if g is not None:
                        self.encoding(i).set_parameter(g, gradients=True)
            check(lib.qmlp_network_adjoint(self._handle, desc(input), desc(adj_output), int(flags),
                                           desc(adj_input if flags & GRADIENTS_INPUT else None),
                                           ctypes.c_void_p(tmp_forward.data_ptr()),
                                           ctypes.c_void_p(tmp_adjoint.data_ptr()), current_stream(input.device)))
            check(lib.qmlp_network_set_parameter(self._handle, None, QMLP_GRADIENTS))
            for i, g in enumerate(grad_encodings):
                if g is not None and self.encoding(i).has_parameters():
                    self.encoding(i).set_parameter(None, gradients=True)
        return adj_input, grad_network, grad_encodings

    def forward(self, input, network_parameters, encoding_parameters=()):
        """Differentiable forward pass; gradients flow to every argument that requires them."""
        encoding_parameters = list(encoding_parameters)
        flags = 0
        if input.requires_grad:
            flags |= GRADIENTS_INPUT
        if network_parameters is not None and network_parameters.requires_grad:
            flags |= GRADIENTS_NETWORK_WEIGHTS
        for i, t in enumerate(encoding_parameters):
            if t is not None and t.requires_grad and i < self.num_encodings() and self.encoding(i).has_parameters():
                flags |= GRADIENTS_INPUT_ENCODINGS
        if flags == 0 or not torch.is_grad_enabled():
            return self.inference(input, network_parameters, encoding_parameters)
        # encodings without parameters get a placeholder so that positions line up
        filled = []
        for i in range(self.num_encodings()):
            p = encoding_parameters[i] if i < len(encoding_parameters) else None
            if p is None or not self.encoding(i).has_parameters():
                p = torch.zeros((1,), device=input.device)
            filled.append(p)
        return _NetworkFunction.apply(self, flags, input, network_parameters, *filled)

    def __getstate__(self):
        return (self._cfg, self._parent)

    def __setstate__(self, state):
        self.__init__(*state)
