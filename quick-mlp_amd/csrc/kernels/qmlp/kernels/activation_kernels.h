// Template of the standalone activation kernels (half in, half out). Everything in
// $$..$$ is replaced by the host before compilation.
// Replaces src_cpp/include/qmlp/kernels/activation_kernels.cuh:28-62 of the reference.

#include <qmlp/kernels/common.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

namespace activations
{
$$DEFINE_ACTIVATIONS$$
}

__global__ void ActivationForwardKernel(
    int rows, int cols,
    const Tensor2Read<half> inputs,
    Tensor2RW<half> outputs)
{
    const long long total = static_cast<long long>(rows) * cols;
    for (long long e = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; e < total;
         e += static_cast<long long>(blockDim.x) * gridDim.x) {
        const int i = static_cast<int>(e / cols), j = static_cast<int>(e - static_cast<long long>(i) * cols);
        const half x = inputs.data_[static_cast<long long>(i) * inputs.strides_[0] + static_cast<long long>(j) * inputs.strides_[1]];
        outputs.data_[static_cast<long long>(i) * outputs.strides_[0] + static_cast<long long>(j) * outputs.strides_[1]]
            = activations::$$ACTIVATION_ID$$::forward(x);
    }
}

__global__ void ActivationAdjointKernel(
    int rows, int cols,
    const Tensor2Read<half> inputs,
    const Tensor2Read<half> adjOutputs,
    Tensor2RW<half> adjInputs)
{
    const long long total = static_cast<long long>(rows) * cols;
    for (long long e = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; e < total;
         e += static_cast<long long>(blockDim.x) * gridDim.x) {
        const int i = static_cast<int>(e / cols), j = static_cast<int>(e - static_cast<long long>(i) * cols);
        const half x = inputs.data_[static_cast<long long>(i) * inputs.strides_[0] + static_cast<long long>(j) * inputs.strides_[1]];
        const half adjz = adjOutputs.data_[static_cast<long long>(i) * adjOutputs.strides_[0] + static_cast<long long>(j) * adjOutputs.strides_[1]];
        adjInputs.data_[static_cast<long long>(i) * adjInputs.strides_[0] + static_cast<long long>(j) * adjInputs.strides_[1]]
            = activations::$$ACTIVATION_ID$$::adjoint(x, adjz);
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
