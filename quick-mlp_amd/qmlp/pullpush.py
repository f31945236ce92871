import torch

from . import _lib
from ._lib import check, current_stream, desc, lib


def _check_device(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("pullpush works on GPU tensors only")


def pullpush_forward(mask: torch.Tensor, data: torch.Tensor) -> torch.Tensor:
    """The inpainted data without autograd (``utils.pullpush_forward`` of the reference's
    torch bindings, src_cpp/pytorch-bindings/src/bind_utils.cpp:9-20)."""
    _check_device(mask, data)
    output = torch.empty_like(data)
    check(lib.qmlp_utils_pullpush_forward(desc(mask), desc(data), desc(output), current_stream(data.device)))
    return output


def pullpush_backward(mask: torch.Tensor, data: torch.Tensor, adj_output: torch.Tensor):
    """Gradients (adj_mask, adj_data) of the inpainting (``utils.pullpush_backward``,
    src_cpp/pytorch-bindings/src/bind_utils.cpp:22-40)."""
    _check_device(mask, data, adj_output)
    adj_mask = torch.zeros_like(mask)
    adj_data = torch.zeros_like(data)
    check(lib.qmlp_utils_pullpush_adjoint(desc(mask), desc(data), desc(adj_output), desc(adj_mask), desc(adj_data),
                                          current_stream(data.device)))
    return adj_mask, adj_data


def precompile(dtype: torch.dtype = torch.float32) -> None:
    """Compiles the pull-push kernels of one dtype into the kernel cache; needs no GPU."""
    check(lib.qmlp_utils_pullpush_precompile(_lib._PRECISION_OF[dtype]))


class _PullPushFunction(torch.autograd.Function):
    """src_cpp/pytorch-bindings/src/bind_utils.cpp:48-66."""

    @staticmethod
    def forward(ctx, mask, data):
        ctx.save_for_backward(mask, data)
        return pullpush_forward(mask, data)

    @staticmethod
    def backward(ctx, grad_output):
        mask, data = ctx.saved_tensors
        return pullpush_backward(mask, data, grad_output)


def pullpush(mask: torch.Tensor, data: torch.Tensor) -> torch.Tensor:
    """
    Performs differentiable inpainting via the Pull-Push algorithm.

    All tensors must reside on the GPU and are of type float or double.
    The mask is defined as 1: non-empty pixel, 0: empty pixel, and any fraction in between.

    :param mask: the mask of shape (Batch, Height, Width)
    :param data: the data of shape (Batch, Channels, Height, Width), fewer than 16 channels
    :return: the inpainted data of shape (Batch, Channels, Height, Width)

    Mirrors src_py/qmlp/pullpush.py:8-25 of the reference.
    """
    return _PullPushFunction.apply(mask, data)
