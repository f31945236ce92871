#pragma once
// Line integration: marches a ray through the bounding box of a child volume encoding
// with a fixed step and sums (or averages) the child's features along the way.
// The input holds the ray start in channels [Start, Start+D) and the ray direction in
// [Start+D, Start+2D); only D = 3 is defined (slab test against the box).
//
// Follows src_cpp/include/qmlp/kernels/encoding_line_integration.cuh:26-166 of the
// reference, including its conventions: the march runs from the entry parameter tmin
// (which is negative if the ray starts inside the box) in steps of `stepsize` while
// t < tmax; "average" divides by floor((tmax-tmin)/stepsize) if that is positive; the
// adjoint treats tmin/tmax as constants.
//
// Difference to the reference, on purpose: its loop `for (t = tmin; t < tmax; t += h)` never
// ends when the interval is unbounded (a zero direction vector gives tmin = -inf) or when h
// is below the spacing of floats at t. Here a ray takes no sample at all unless tmin and
// tmax are finite and the interval holds fewer than 2^20 steps, and the loop also counts
// its iterations (at most steps + 2), so every wavefront leaves the march.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/arrays.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

enum class LineIntegrationBlendingMode
{
    ADDITIVE,
    AVERAGE
};

/** Kernel-argument block; the host writes the child's block first, then 2*D+1 floats. */
template <typename ChildParams, int D>
struct LineIntegrationParams
{
    ChildParams child;
    float boundingBoxMin[D];
    float boundingBoxSize[D];
    float stepsize;
};

template <int StartChannel, int D, LineIntegrationBlendingMode Blending, typename Child>
struct EncodingLineIntegration
{
    static_assert(D == 3, "The ray / bounding box intersection is only defined in 3D");
    typedef LineIntegrationParams<typename Child::param_t, D> param_t;
    static constexpr int NumOutputs = Child::NumOutputs;
    // the child's parameter gradients are added point by point inside the march
    static constexpr bool HasTileScatter = false;
    typedef StaticArray<float, NumOutputs> feature_t;
    typedef StaticArray<float, D> position_t;

    /** Never called (HasTileScatter is false); present because the kernels name it in a
     *  discarded `if constexpr` branch of a non-template function, which is still checked. */
    template <int LDS_LEVELS = 0, typename AdjFn>
    __device__ __forceinline__ static void scatterTile(int, long long, long long, const Tensor2Read<float>&,
                                                       const AdjFn&, const param_t&, float* = nullptr)
    {
    }

    /** Slab test; returns the parameter interval of the ray inside the box. */
    __device__ __forceinline__ static void intersect(const position_t& rayStart, const position_t& rayDir,
                                                     const param_t& params, float& tmin, float& tmax)
    {
#pragma clang fp contract(off)
        float lo[D], hi[D];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const float inv = 1.0f / rayDir[d];
            const float ta = (params.boundingBoxMin[d] - rayStart[d]) * inv;
            const float tb = (params.boundingBoxMin[d] + params.boundingBoxSize[d] - rayStart[d]) * inv;
            lo[d] = fminf(ta, tb);
            hi[d] = fmaxf(ta, tb);
        }
        tmin = fmaxf(fmaxf(lo[0], lo[1]), lo[2]);
        tmax = fminf(fminf(hi[0], hi[1]), hi[2]);
    }

    static constexpr float MaxSteps = 1048576.f;

    /** Number of steps in [tmin, tmax); -2 (so that steps + 2 iterations are none) if the ray
     *  takes no sample, see the file header. */
    __device__ __forceinline__ static int numSteps(float tmin, float tmax, float stepsize)
    {
        const float steps = floorf((tmax - tmin) / stepsize);
        const bool bounded = fabsf(tmin) < __builtin_inff() && fabsf(tmax) < __builtin_inff();
        if (!bounded || !(steps < MaxSteps)) return -2;
        return static_cast<int>(steps);
    }

    template <typename I>
    __device__ __forceinline__ static void readRay(const I& input, position_t& rayStart, position_t& rayDir)
    {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            rayStart[d] = input[d + StartChannel];
            rayDir[d] = input[d + StartChannel + D];
        }
    }

    template <typename I, typename O>
    __device__ static void forward(const I& input, O& output, const param_t& params)
    {
        typedef typename O::ValueType O_t;
        position_t rayStart, rayDir;
        readRay(input, rayStart, rayDir);
        float tmin, tmax;
        intersect(rayStart, rayDir, params, tmin, tmax);
        const int steps = numSteps(tmin, tmax, params.stepsize);

        feature_t accu;
#pragma unroll
        for (int i = 0; i < NumOutputs; ++i) accu[i] = 0.f;
        int iteration = 0;
        for (float t = tmin; t < tmax && iteration < steps + 2; t += params.stepsize, ++iteration) {
            position_t position;
#pragma unroll
            for (int d = 0; d < D; ++d) position[d] = fmaf(t, rayDir[d], rayStart[d]);
            feature_t contribution;
            Child::forward(position, contribution, params.child);
#pragma unroll
            for (int i = 0; i < NumOutputs; ++i) accu[i] += contribution[i];
        }
        if constexpr (Blending == LineIntegrationBlendingMode::AVERAGE) {
            if (steps > 0) {
                const float scale = 1.0f / static_cast<float>(steps);
#pragma unroll
                for (int i = 0; i < NumOutputs; ++i) accu[i] *= scale;
            }
        }
#pragma unroll
        for (int i = 0; i < NumOutputs; ++i) output[i] = fcast<O_t>(accu[i]);
    }

    template <int PPL, typename I, typename Os>
    __device__ __forceinline__ static void forwardBatch(const I (&inputs)[PPL], Os& outputs, const param_t& params)
    {
#pragma unroll 1
        for (int q = 0; q < PPL; ++q) {
            auto row = outputs[q];
            forward(inputs[q], row, params);
        }
    }

    template <bool EvaluateInputGradients, bool EvaluateParameterGradients, typename I, typename O, typename AdjI>
    __device__ static void adjoint(const I& input, const O& adjOutput, AdjI& adjInput, const param_t& params)
    {
        if constexpr (!EvaluateInputGradients && !EvaluateParameterGradients) return;
        position_t rayStart, rayDir;
        readRay(input, rayStart, rayDir);
        float tmin, tmax;
        intersect(rayStart, rayDir, params, tmin, tmax);
        const int steps = numSteps(tmin, tmax, params.stepsize);

        float scale = 1.0f;
        if constexpr (Blending == LineIntegrationBlendingMode::AVERAGE)
            scale = steps > 0 ? 1.0f / static_cast<float>(steps) : 1.0f;
        feature_t adjAccu;
#pragma unroll
        for (int i = 0; i < NumOutputs; ++i) adjAccu[i] = scale * fcast<float>(adjOutput[i]);

        position_t adjRayStart, adjRayDir;
#pragma unroll
        for (int d = 0; d < D; ++d) adjRayStart[d] = adjRayDir[d] = 0.f;
        int iteration = 0;
        for (float t = tmin; t < tmax && iteration < steps + 2; t += params.stepsize, ++iteration) {
            position_t position, adjPosition;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                position[d] = fmaf(t, rayDir[d], rayStart[d]);
                adjPosition[d] = 0.f;
            }
            Child::template adjoint<EvaluateInputGradients, EvaluateParameterGradients>(
                position, adjAccu, adjPosition, params.child);
            if constexpr (EvaluateInputGradients) {
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    adjRayStart[d] += adjPosition[d];
                    adjRayDir[d] += adjPosition[d] * t;
                }
            }
        }
        if constexpr (EvaluateInputGradients) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                adjInput[d + StartChannel] += adjRayStart[d];
                adjInput[d + StartChannel + D] += adjRayDir[d];
            }
        }
    }
};

QUICKMLP_KERNEL_NAMESPACE_END
