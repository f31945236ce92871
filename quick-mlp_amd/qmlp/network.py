import json
import warnings

import torch

from .activation import FusedActivation
from .classes import Network
from .encoding import FusedEncoding


class FusedNetwork(torch.nn.Module):
    """A fully fused coordinate MLP: input encodings, linear layers and activations in
    one generated kernel per pass.

    Mirrors src_py/qmlp/network.py:12-159 of the reference. Differences, on purpose:
    the parameters of the encodings are real module parameters that reach the kernel
    (the reference passes an empty list), and the static size queries work.
    """

    def __init__(self, cfg: str, parent: str = ".", weight_dtype=torch.float16, device="cuda", scriptable: bool = False):
        """
        :param cfg: the network specification as a JSON string
        :param parent: folder relative to which activation files named in the
            specification are resolved
        :param weight_dtype: dtype of the master weights (float32 for training with
            optimizers that cannot step fp16 tensors)
        :param scriptable: hold the torch custom class ``torch.classes.qmlp_cu.Network`` instead of
            the ctypes mirror, so that the module can be traced and saved with TorchScript like the
            reference's module (same kernels and numbers either way)
        """
        super().__init__()
        self._cfg = cfg
        self._parent = parent
        self._scriptable = scriptable
        if scriptable:
            from . import load_library
            self._network = load_library().Network(cfg, parent)
        else:
            self._network = Network(cfg, parent)
        # plain integers: a traced forward() may not call integer methods of the custom class
        self._channels_in = self._network.channels_in()
        self._num_output_channels = self._network.channels_out()
        self._num_layers = self._network.num_layers()

        weights = (self._network.create_inference_parameters().to(device) if scriptable
                   else self._network.create_inference_parameters(device))
        self._network.initialize_inference_parameters(weights)
        self.weights = torch.nn.Parameter(weights.to(weight_dtype), requires_grad=True)

        self._num_encodings = self._network.num_encodings()
        self._max_input_channel = 0
        self._encodings = []
        params = []
        for i in range(self._num_encodings):
            e = self._network.encoding(i)
            self._encodings.append(e)
            self._max_input_channel = max(self._max_input_channel, e.max_input_channel())
            if e.has_parameters():
                p = e.create_inference_parameters().to(device) if scriptable else e.create_inference_parameters(device)
                torch.zero_(p)
                params.append(torch.nn.Parameter(p, requires_grad=True))
            else:
                params.append(torch.nn.Parameter(torch.zeros((1,), device=device), requires_grad=False))
        self.encoding_parameters = torch.nn.ParameterList(params)

    @staticmethod
    def MatrixSize() -> int:
        """Layer widths are padded to multiples of this value."""
        return Network.MatrixSize()

    @staticmethod
    def WarpSize() -> int:
        """Points per wavefront tile; batches are padded internally to a multiple of it."""
        return Network.WarpSize()

    @staticmethod
    def MaxSharedMemoryBytes() -> int:
        """LDS bytes available to one workgroup."""
        return Network.MaxSharedMemoryBytes()

    def is_parallel_streams(self) -> bool:
        return self._network.is_parallel_streams()

    def set_parallel_streams(self, v: bool):
        """Run the per-layer weight-gradient kernels on separate streams."""
        self._network.set_parallel_streams(v)

    def num_encodings(self) -> int:
        return self._num_encodings

    def encoding(self, index: int) -> FusedEncoding:
        return FusedEncoding(self._encodings[index])

    def channels_in(self) -> int:
        return self._channels_in

    def channels_out(self) -> int:
        return self._num_output_channels

    def num_layers(self) -> int:
        return self._num_layers

    def num_output_channels(self) -> int:
        return self._num_output_channels

    def get_weight(self, layer: int, bias: bool, grad: bool) -> torch.Tensor:
        """Copy of the (padded) weight matrix or bias vector of a layer, or of its gradient."""
        p = self.weights.grad if grad else self.weights.data
        t = self._network.parameter_view(layer, bias, p)
        return torch.clone(t.detach())

    def set_weight(self, layer: int, bias: bool, grad: bool, value: torch.Tensor):
        p = self.weights.grad if grad else self.weights.data
        t = self._network.parameter_view(layer, bias, p)
        assert value.shape == t.shape, (value.shape, t.shape)
        assert value.dtype == t.dtype
        t.copy_(value)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        assert x.dim() == 2
        assert x.shape[1] == self.channels_in()
        if self.weights.requires_grad and self.weights.dtype == torch.float16 and torch.is_grad_enabled():
            warnings.warn("Training a network with 16-bit master weights: the gradient tensor is 16-bit as well, "
                          "which most optimizers cannot handle. Pass weight_dtype=torch.float32 to the constructor.")
        return self._network.forward(x, self.weights, list(self.encoding_parameters))

    def __getstate__(self):
        state = super().__getstate__() if hasattr(super(), "__getstate__") else self.__dict__.copy()
        state = dict(state)
        state["_encodings"] = None      # handles into the native network: taken again after unpickling
        return state

    def __setstate__(self, state):
        # pickling rebuilds the native network from its specification; take the encodings from
        # the rebuilt network again instead of stand-alone copies
        super().__setstate__(state)
        self._encodings = [self._network.encoding(i) for i in range(self._num_encodings)]

    def __repr__(self):
        return f'FusedNetwork("{self._cfg}")'

    __str__ = __repr__


class SimulatedNetwork(torch.nn.Module):
    """The same network as plain ``torch.nn.Linear`` layers (identity encoding only).

    It exists to verify :class:`FusedNetwork` (src_py/qmlp/network.py:161-242 of the
    reference); it is never used in place of the fused kernels.
    """

    def __init__(self, cfg: str, weight_dtype=torch.float16):
        super().__init__()
        cfg = json.loads(cfg)
        self._channels_in = cfg["num_inputs"]
        self._channels_out = cfg["num_outputs"]
        self._weight_dtype = weight_dtype
        encodings = cfg["encodings"]
        if len(encodings) == 1:
            e = encodings[0]
            if e["id"] != "Identity" or e["start_in"] != 0 or e["n_in"] != self._channels_in:
                raise ValueError("Only identity encoding supported and it must consume all inputs")
        elif len(encodings) > 1:
            raise ValueError("Only a single encoding supported")
        layers = []
        self._has_bias = []
        n_in, n_out = self._channels_in, None
        for layer in cfg["network"]:
            n_out = layer["n_out"]
            layers.append(torch.nn.Linear(n_in, n_out, bias=layer["bias"], dtype=weight_dtype))
            layers.append(FusedActivation.get_activation(layer["activation"]))
            self._has_bias.append(layer["bias"])
            n_in = n_out
        if n_out != self._channels_out:
            raise ValueError("Last layer does not match the number of outputs")
        self.layers = torch.nn.Sequential(*layers)
        self._num_layers = len(cfg["network"])

    def channels_in(self):
        return self._channels_in

    def channels_out(self):
        return self._channels_out

    def num_layers(self) -> int:
        return self._num_layers

    def has_bias(self, layer: int):
        return self._has_bias[layer]

    def get_weight(self, layer: int, bias: bool, grad: bool) -> torch.Tensor:
        lin = self.layers[2 * layer]
        t = lin.bias if bias else lin.weight
        return torch.clone(t.grad.detach()) if grad else torch.clone(t.detach())

    def set_weight(self, layer: int, bias: bool, grad: bool, value: torch.Tensor):
        lin = self.layers[2 * layer]
        t = lin.bias if bias else lin.weight
        if grad:
            t.grad = torch.clone(value.detach())
        else:
            with torch.no_grad():
                t.copy_(value.detach())

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.layers(x.to(self._weight_dtype)).to(torch.float32)


def copy_torch_to_fused(dst: FusedNetwork, src: SimulatedNetwork, grad: bool = False):
    """Copies the weights (or gradients) of the plain network into the fused one. Widths
    that the fused network padded are filled with zeros."""
    assert dst.num_layers() == src.num_layers()
    for layer in range(src.num_layers()):
        for bias in (False, True):
            if bias and not src.has_bias(layer):
                continue
            w = src.get_weight(layer, bias, grad)
            target = dst.get_weight(layer, bias, grad)
            padded = torch.zeros_like(target)
            padded[tuple(slice(0, s) for s in w.shape)] = w.to(target.dtype).to(target.device)
            dst.set_weight(layer, bias, grad, padded)
