import torch

from .classes import Activation


class FusedActivation(torch.nn.Module):
    """Point-wise activation as a run-time compiled kernel (half precision tensors only).

    ``cfg`` is either the id of a built-in activation ("relu", "celu", "sine",
    "identity") or an inline JSON string with the keys ``id``, ``forward`` and
    ``adjoint`` holding device code snippets, e.g.::

        {"id": "sine", "forward": "z = hsin(x)", "adjoint": "adjx = __hmul(hcos(x), adjz)"}

    Mirrors src_py/qmlp/activation.py:8-79 of the reference.
    """

    @staticmethod
    def get_activation(name: str) -> torch.nn.Module:
        """The plain PyTorch module equivalent to a built-in activation (for verification)."""
        if name == "relu":
            return torch.nn.ReLU()
        if name == "celu":
            return torch.nn.CELU()
        if name == "sine":
            class Sine(torch.nn.Module):
                def forward(self, x):
                    return torch.sin(x)
            return Sine()
        if name == "identity":
            return torch.nn.Identity()
        raise ValueError("Unknown or user-specified activation")

    def __init__(self, cfg: str, scriptable: bool = False):
        """
        :param scriptable: hold the torch custom class ``torch.classes.qmlp_cu.Activation`` instead
            of the ctypes mirror, so that the module can be traced or scripted and saved with
            TorchScript like the reference's module (same kernels and numbers either way)
        """
        super().__init__()
        self._cfg = cfg
        if scriptable:
            from . import load_library
            self._activation = load_library().Activation(cfg)
        else:
            self._activation = Activation(cfg)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        """(batch, channels) half -> (batch, channels) half, with autograd support."""
        return self._activation.forward(input)

    def __repr__(self):
        return f'FusedActivation("{self._cfg}")'

    __str__ = __repr__
