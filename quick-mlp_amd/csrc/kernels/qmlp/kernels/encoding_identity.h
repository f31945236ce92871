#pragma once
// Identity encoding: copies NumChannels input channels starting at StartChannel.
// Replaces src_cpp/include/qmlp/kernels/encoding_identity.cuh:12-39 of the reference.

#include <qmlp/kernels/common.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

template <int StartChannel, int NumChannels>
struct EncodingIdentity
{
    static constexpr int NumOutputs = NumChannels;

    /** input: anything indexable with operator[] returning float; output: indexable, assignable */
    template <typename I, typename O>
    __device__ __forceinline__ static void forward(const I& input, O& output)
    {
        typedef typename O::ValueType O_t;
#pragma unroll
        for (int i = 0; i < NumChannels; ++i) output[i] = fcast<O_t>(input[i + StartChannel]);
    }

    template <int PPL, typename I, typename Os>
    __device__ __forceinline__ static void forwardBatch(const I (&inputs)[PPL], Os& outputs)
    {
#pragma unroll
        for (int q = 0; q < PPL; ++q) {
            auto row = outputs[q];
            forward(inputs[q], row);
        }
    }

    template <bool EvaluateInputGradients, bool EvaluateParameterGradients, typename I, typename O, typename AdjI>
    __device__ __forceinline__ static void adjoint(const I& input, const O& adjOutput, AdjI& adjInput)
    {
        if constexpr (EvaluateInputGradients) {
#pragma unroll
            for (int i = 0; i < NumChannels; ++i) adjInput[i + StartChannel] += fcast<float>(adjOutput[i]);
        }
    }
};

QUICKMLP_KERNEL_NAMESPACE_END
