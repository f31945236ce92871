#pragma once

#include "common.h"
#include "tensor.h"

QUICKMLP_NAMESPACE_BEGIN

/**
 * Helper operations that are not part of the network path.
 * Mirrors src_cpp/include/qmlp/utils.h:16-85 of the reference.
 */
class Utils
{
public:
    /**
     * Differentiable inpainting by pull-push: down- and upsampling over an image pyramid with
     * fractional masks (1: pixel is known, 0: pixel is empty, anything in between). All
     * tensors live on the GPU and are float or double.
     *
     * \param mask (Batch, Height, Width)
     * \param data (Batch, Channels, Height, Width), at most 15 channels like the reference
     * \param output the inpainted data, (Batch, Channels, Height, Width)
     */
    static void fractionalPullpush(const Tensor& mask, const Tensor& data, Tensor& output, stream_t stream);

    /**
     * Adjoint of fractionalPullpush (runs the forward pass again to get the pyramid).
     * \param adjOutput gradient of the output, (Batch, Channels, Height, Width)
     * \param adjMask gradient of the mask, (Batch, Height, Width); accumulated, zero it first
     * \param adjData gradient of the data, (Batch, Channels, Height, Width); accumulated
     */
    static void adjointFractionalPullpush(const Tensor& mask, const Tensor& data, const Tensor& adjOutput,
                                          Tensor& adjMask, Tensor& adjData, stream_t stream);

    /** Compiles the pull-push kernels of one precision into the kernel cache; needs no GPU. */
    static void precompile(Tensor::Precision precision);
};

QUICKMLP_NAMESPACE_END
