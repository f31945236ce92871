// Template of the standalone encoding kernels (fp32 in, fp32 out). Everything in
// $$..$$ is replaced by the host before compilation.
// Replaces src_cpp/include/qmlp/kernels/encoding_kernels.cuh:26-62 of the reference.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/arrays.h>

$$INCLUDES$$

QUICKMLP_KERNEL_NAMESPACE_BEGIN

__global__ void EncodingForwardKernel(
    long long numel,
    const Tensor2Read<float> inputs,  //shape (numel, Cin)
    Tensor2RW<float> outputs          //shape (numel, Cout), unit stride along the channels
    $$ENCODING_PARAMETERS$$)
{
    for (long long index = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; index < numel;
         index += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        const StridedArray<const float> encodingInput{inputs.data_ + index * inputs.strides_[0], inputs.strides_[1]};
        WrappedArray<float> encodingOutput{outputs.data_ + index * outputs.strides_[0]};
        $$CALL_ENCODINGS_FORWARD$$
    }
}

// One wavefront takes 64 consecutive points at a time: one lane per point for the input
// gradients, then all lanes together for the parameter gradients of grid encodings (groups
// of lanes add neighbouring table entries in one atomic request).
__global__ void __launch_bounds__(256) EncodingAdjointKernel(
    long long numel,
    const Tensor2Read<float> inputs,      //shape (numel, Cin)
    const Tensor2Read<float> adjOutputs,  //shape (numel, Cout)
    Tensor2RW<float> adjInputs            //shape (numel, Cin), accumulated
    $$ENCODING_PARAMETERS$$)
{
    const int lane = threadIdx.x % WAVE_SIZE;
    const long long wavesPerBlock = blockDim.x / WAVE_SIZE;
    const long long stride = wavesPerBlock * gridDim.x * TILE_POINTS;
    for (long long tileBase = (blockIdx.x * wavesPerBlock + threadIdx.x / WAVE_SIZE) * TILE_POINTS; tileBase < numel;
         tileBase += stride)
    {
        const long long index = tileBase + lane;
        if (index < numel) {
            const StridedArray<const float> encodingInput{inputs.data_ + index * inputs.strides_[0], inputs.strides_[1]};
            const StridedArray<const float> encodingAdjOutput{adjOutputs.data_ + index * adjOutputs.strides_[0], adjOutputs.strides_[1]};
            StridedArray<float> encodingAdjInput{adjInputs.data_ + index * adjInputs.strides_[0], adjInputs.strides_[1]};
            $$CALL_ENCODINGS_ADJOINT$$
        }
        $$CALL_ENCODINGS_SCATTER$$
    }
}

// Test aid: table offsets and interpolation weights of every corner of every level.
__global__ void EncodingCornersKernel(
    long long numel,
    const Tensor2Read<float> inputs,  //shape (numel, Cin)
    unsigned* __restrict__ indices,   //shape (numel, perPoint)
    float* __restrict__ weights,      //shape (numel, perPoint)
    int perPoint
    $$ENCODING_PARAMETERS$$)
{
    for (long long index = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; index < numel;
         index += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        const StridedArray<const float> encodingInput{inputs.data_ + index * inputs.strides_[0], inputs.strides_[1]};
        unsigned* cornerIndices = indices + index * perPoint;
        float* cornerWeights = weights + index * perPoint;
        (void)encodingInput; (void)cornerIndices; (void)cornerWeights;
        $$CALL_ENCODINGS_CORNERS$$
    }
}

// Test aid: the same two arrays, written by the code the fused kernels run. MODE 1: the
// gathers of the forward pass (one lane per point); MODE 2: the gradient scatter of the
// backward pass (one wavefront per 64 points), which records where it would add.
template <int MODE>
__global__ void __launch_bounds__(256) EncodingTraceKernel(
    long long numel,
    const Tensor2Read<float> inputs,  //shape (numel, Cin)
    unsigned* __restrict__ indices,   //shape (numel, perPoint)
    float* __restrict__ weights,      //shape (numel, perPoint)
    int perPoint
    $$ENCODING_PARAMETERS$$)
{
    if constexpr (MODE == 1) {
        for (long long index = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; index < numel;
             index += static_cast<long long>(blockDim.x) * gridDim.x)
        {
            const StridedArray<const float> encodingInput{inputs.data_ + index * inputs.strides_[0], inputs.strides_[1]};
            unsigned* cornerIndices = indices + index * perPoint;
            float* cornerWeights = weights + index * perPoint;
            (void)encodingInput; (void)cornerIndices; (void)cornerWeights;
            $$CALL_ENCODINGS_TRACE_GATHER$$
        }
    } else {
        const int lane = threadIdx.x % WAVE_SIZE;
        const long long wavesPerBlock = blockDim.x / WAVE_SIZE;
        const long long stride = wavesPerBlock * gridDim.x * TILE_POINTS;
        (void)lane;
        for (long long tileBase = (blockIdx.x * wavesPerBlock + threadIdx.x / WAVE_SIZE) * TILE_POINTS; tileBase < numel;
             tileBase += stride)
        {
            $$CALL_ENCODINGS_TRACE_SCATTER$$
        }
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
