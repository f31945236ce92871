import torch

from .classes import Encoding


class FusedEncoding(torch.nn.Module):
    """One input encoding as a stand-alone, differentiable module.

    ``cfg_or_impl`` is the JSON string of the encoding (keys ``id``, ``start_in``,
    ``n_in`` plus encoding specific ones, e.g. for "HashGrid": ``n_levels``,
    ``n_features_per_level``, ``log2_hashmap_size``, ``min_resolution``,
    ``max_resolution``, ``combination_mode``, ``bounding_box_min``,
    ``bounding_box_size``) or an existing :class:`qmlp.Encoding`, as handed out by
    :meth:`FusedNetwork.encoding`.

    Mirrors src_py/qmlp/encoding.py:9-123 of the reference.
    """

    def __init__(self, cfg_or_impl, scriptable: bool = False):
        """
        :param scriptable: with a JSON string, hold the torch custom class
            ``torch.classes.qmlp_cu.Encoding`` instead of the ctypes mirror, so that the module can
            be traced or scripted and saved with TorchScript like the reference's module
        """
        super().__init__()
        if isinstance(cfg_or_impl, str):
            self._cfg = cfg_or_impl
            if scriptable:
                from . import load_library
                self._encoding = load_library().Encoding(cfg_or_impl)
            else:
                self._encoding = Encoding(cfg_or_impl)
        elif isinstance(cfg_or_impl, Encoding) or isinstance(cfg_or_impl, torch.ScriptObject):
            self._cfg = cfg_or_impl.to_json()
            self._encoding = cfg_or_impl
        else:
            raise TypeError("expected a json string, a qmlp.Encoding or a torch.classes.qmlp_cu.Encoding")
        self._max_input_channel = self._encoding.max_input_channel()
        self._num_output_channels = self._encoding.num_output_channels()
        self._has_parameters = self._encoding.has_parameters()

    def max_input_channel(self) -> int:
        """The highest input channel the encoding reads."""
        return self._max_input_channel

    def num_output_channels(self) -> int:
        return self._num_output_channels

    def has_parameters(self) -> bool:
        """True iff the encoding has trainable parameters (see create_parameter_tensor)."""
        return self._has_parameters

    def create_parameter_tensor(self, device="cuda") -> torch.Tensor:
        """A normally-distributed parameter tensor of the right size and dtype."""
        assert self.has_parameters()
        if isinstance(self._encoding, Encoding):
            t = self._encoding.create_inference_parameters(device)
        else:
            t = self._encoding.create_inference_parameters().to(device)
        tmp = torch.empty(t.shape, dtype=torch.float32, device=t.device)
        torch.nn.init.normal_(tmp)
        t.copy_(tmp)
        return t

    def forward(self, input: torch.Tensor, parameters: torch.Tensor = None) -> torch.Tensor:
        """(batch, channels) float -> (batch, num_output_channels()) float, with autograd."""
        if parameters is None:
            return self._encoding.forward(input)
        return self._encoding.forward_with_parameter(input, parameters)

    def __repr__(self):
        return f'FusedEncoding("""{self._cfg}""")'

    __str__ = __repr__
