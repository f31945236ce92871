#pragma once
// Differentiable pull-push inpainting on an image pyramid (fractional masks): one kernel per
// pyramid level and direction; every kernel is a grid-stride loop with one thread per pixel
// and is bound by HBM bandwidth.
//
//   down:  low-res pixel = mask-weighted mean of its window of high-res pixels, low-res mask =
//          maximum of the window (windows as in adaptive pooling: [floor(i*H/oH), ceil((i+1)*H/oH)),
//          evaluated in fp32 like the reference; they overlap when a size is odd)
//   up:    high-res pixel = m*data + (1-m)*(bilinear mix of the 4 nearest low-res pixels,
//          weights 9/16, 3/16, 3/16, 1/16, renormalised by the low-res masks)
//
// Follows src_cpp/include/qmlp/kernels/pullpush.cuh:22-303 of the reference. Differences on
// purpose: no per-thread channel arrays (the channels are looped and the few mask values
// re-read from cache), and the adjoint of `down` adds with atomics, because the windows of
// neighbouring low-res pixels overlap for odd sizes (the reference adds without).

#include <qmlp/kernels/common.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

template <typename T> using Tensor3Read = TensorAccessor<const T, 3>;
template <typename T> using Tensor4Read = TensorAccessor<const T, 4>;
template <typename T> using Tensor3RW = TensorAccessor<T, 3>;
template <typename T> using Tensor4RW = TensorAccessor<T, 4>;

namespace pullpush
{
// clamped to [0, c]: the fp32 quotient is only exact while the products stay below 2^24
__device__ __forceinline__ int windowStart(int a, int b, int c) { return max(0, static_cast<int>(floorf(static_cast<float>(a * c) / b))); }
__device__ __forceinline__ int windowEnd(int a, int b, int c) { return min(c, static_cast<int>(ceilf(static_cast<float>((a + 1) * c) / b))); }

template <typename A>
__device__ __forceinline__ long long at3(const A& t, int b, int y, int x)
{
    return static_cast<long long>(b) * t.strides_[0] + static_cast<long long>(y) * t.strides_[1]
         + static_cast<long long>(x) * t.strides_[2];
}
template <typename A>
__device__ __forceinline__ long long at4(const A& t, int b, int c, int y, int x)
{
    return static_cast<long long>(b) * t.strides_[0] + static_cast<long long>(c) * t.strides_[1]
         + static_cast<long long>(y) * t.strides_[2] + static_cast<long long>(x) * t.strides_[3];
}

__device__ __forceinline__ void atomicAccumulate(float* p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomicAccumulate(double* p, double v) { unsafeAtomicAdd(p, v); }

/** The 4 low-res neighbours of high-res pixel (i, j) and their bilinear weights. */
struct Neighbours
{
    int ii[4], jj[4];
    float w[4];
    bool inside[4];
};
__device__ __forceinline__ Neighbours neighbours(int i, int j, int oH, int oW)
{
    const int io = (i % 2 == 0) ? -1 : +1;
    const int jo = (j % 2 == 0) ? -1 : +1;
    Neighbours n;
    n.ii[0] = i / 2;      n.jj[0] = j / 2;      n.w[0] = 0.75f * 0.75f;
    n.ii[1] = i / 2 + io; n.jj[1] = j / 2;      n.w[1] = 0.25f * 0.75f;
    n.ii[2] = i / 2;      n.jj[2] = j / 2 + jo; n.w[2] = 0.25f * 0.75f;
    n.ii[3] = i / 2 + io; n.jj[3] = j / 2 + jo; n.w[3] = 0.25f * 0.25f;
#pragma unroll
    for (int k = 0; k < 4; ++k) n.inside[k] = n.ii[k] >= 0 && n.jj[k] >= 0 && n.ii[k] < oH && n.jj[k] < oW;
    return n;
}
} // namespace pullpush

/** One thread per low-res pixel (b, i, j). */
template <typename T>
__global__ void __launch_bounds__(256) PullPushDownKernel(
    long long numel, const Tensor3Read<T> mask, const Tensor4Read<T> data, Tensor3RW<T> maskLow, Tensor4RW<T> dataLow)
{
    using namespace pullpush;
    const int H = mask.sizes_[1], W = mask.sizes_[2], oH = H / 2, oW = W / 2, C = data.sizes_[1];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        const int j = static_cast<int>(idx % oW), i = static_cast<int>((idx / oW) % oH), b = static_cast<int>(idx / (static_cast<long long>(oW) * oH));
        const int i0 = windowStart(i, oH, H), i1 = windowEnd(i, oH, H), j0 = windowStart(j, oW, W), j1 = windowEnd(j, oW, W);
        T n1 = 0, n2 = 0;
        for (int jj = j0; jj < j1; ++jj)
            for (int ii = i0; ii < i1; ++ii) {
                const T m = mask.data_[at3(mask, b, ii, jj)];
                n1 += m;
                n2 = max(n2, m);
            }
        maskLow.data_[at3(maskLow, b, i, j)] = n2;
        for (int c = 0; c < C; ++c) {
            T d = 0;
            for (int jj = j0; jj < j1; ++jj)
                for (int ii = i0; ii < i1; ++ii) d += mask.data_[at3(mask, b, ii, jj)] * data.data_[at4(data, b, c, ii, jj)];
            dataLow.data_[at4(dataLow, b, c, i, j)] = n1 > 0 ? d / n1 : T(0);
        }
    }
}

/** One thread per high-res pixel (b, i, j). */
template <typename T>
__global__ void __launch_bounds__(256) PullPushUpKernel(
    long long numel, const Tensor3Read<T> mask, const Tensor4Read<T> data, const Tensor3Read<T> maskLow,
    const Tensor4Read<T> dataLow, Tensor3RW<T> maskHigh, Tensor4RW<T> dataHigh)
{
    using namespace pullpush;
    const int H = mask.sizes_[1], W = mask.sizes_[2], oH = H / 2, oW = W / 2, C = data.sizes_[1];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        const int j = static_cast<int>(idx % W), i = static_cast<int>((idx / W) % H), b = static_cast<int>(idx / (static_cast<long long>(W) * H));
        const Neighbours nb = neighbours(i, j, oH, oW);
        T weight = 0, n = 0, ml[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ml[k] = nb.inside[k] ? maskLow.data_[at3(maskLow, b, nb.ii[k], nb.jj[k])] : T(0);
            if (nb.inside[k]) {
                weight += nb.w[k];
                n += nb.w[k] * ml[k];
            }
        }
        const T m = mask.data_[at3(mask, b, i, j)];
        maskHigh.data_[at3(maskHigh, b, i, j)] = m + (n > 0 ? (1 - m) * (n / weight) : T(0));
        for (int c = 0; c < C; ++c) {
            T d = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (nb.inside[k]) d += nb.w[k] * ml[k] * dataLow.data_[at4(dataLow, b, c, nb.ii[k], nb.jj[k])];
            dataHigh.data_[at4(dataHigh, b, c, i, j)] = m * data.data_[at4(data, b, c, i, j)] + (1 - m) * (n > 0 ? d / n : T(0));
        }
    }
}

/** Adjoint of PullPushDownKernel; one thread per low-res pixel, gradients accumulated. */
template <typename T>
__global__ void __launch_bounds__(256) PullPushAdjointDownKernel(
    long long numel, const Tensor3Read<T> mask, const Tensor4Read<T> data, const Tensor3Read<T> gradMaskLow,
    const Tensor4Read<T> gradDataLow, Tensor3RW<T> gradMask, Tensor4RW<T> gradData)
{
    using namespace pullpush;
    const int H = mask.sizes_[1], W = mask.sizes_[2], oH = H / 2, oW = W / 2, C = data.sizes_[1];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        const int j = static_cast<int>(idx % oW), i = static_cast<int>((idx / oW) % oH), b = static_cast<int>(idx / (static_cast<long long>(oW) * oH));
        const int i0 = windowStart(i, oH, H), i1 = windowEnd(i, oH, H), j0 = windowStart(j, oW, W), j1 = windowEnd(j, oW, W);
        T n1 = 0, n2 = 0;
        for (int jj = j0; jj < j1; ++jj)
            for (int ii = i0; ii < i1; ++ii) {
                const T m = mask.data_[at3(mask, b, ii, jj)];
                n1 += m;
                n2 = max(n2, m);
            }
        // dataLow_c = d_c / n1: adjoint of n1 collects all channels
        T adjN1 = 0;
        for (int c = 0; c < C; ++c) {
            T d = 0;
            for (int jj = j0; jj < j1; ++jj)
                for (int ii = i0; ii < i1; ++ii) d += mask.data_[at3(mask, b, ii, jj)] * data.data_[at4(data, b, c, ii, jj)];
            if (n1 > 0) adjN1 -= gradDataLow.data_[at4(gradDataLow, b, c, i, j)] * d / (n1 * n1);
        }
        const T adjN2 = gradMaskLow.data_[at3(gradMaskLow, b, i, j)];
        for (int jj = j0; jj < j1; ++jj)
            for (int ii = i0; ii < i1; ++ii) {
                const T m = mask.data_[at3(mask, b, ii, jj)];
                T adjMask = adjN1;
                for (int c = 0; c < C; ++c) {
                    const T adjD = n1 > 0 ? gradDataLow.data_[at4(gradDataLow, b, c, i, j)] / n1 : T(0);
                    atomicAccumulate(gradData.data_ + at4(gradData, b, c, ii, jj), adjD * m);
                    adjMask += adjD * data.data_[at4(data, b, c, ii, jj)];
                }
                if (n2 == m) adjMask += adjN2;   // the maximum passes its gradient to every pixel that attains it
                atomicAccumulate(gradMask.data_ + at3(gradMask, b, ii, jj), adjMask);
            }
    }
}

/** Adjoint of PullPushUpKernel; one thread per high-res pixel. gradMask / gradData are the
 *  gradients of this level's inputs (accumulated), gradMaskLow / gradDataLow those of the
 *  low-res inputs (accumulated with atomics: up to 9 high-res pixels share a low-res one). */
template <typename T>
__global__ void __launch_bounds__(256) PullPushAdjointUpKernel(
    long long numel, const Tensor3Read<T> mask, const Tensor4Read<T> data, const Tensor3Read<T> maskLow,
    const Tensor4Read<T> dataLow, const Tensor3Read<T> gradMaskHigh, const Tensor4Read<T> gradDataHigh,
    Tensor3RW<T> gradMask, Tensor4RW<T> gradData, Tensor3RW<T> gradMaskLow, Tensor4RW<T> gradDataLow)
{
    using namespace pullpush;
    const int H = mask.sizes_[1], W = mask.sizes_[2], oH = H / 2, oW = W / 2, C = data.sizes_[1];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        const int j = static_cast<int>(idx % W), i = static_cast<int>((idx / W) % H), b = static_cast<int>(idx / (static_cast<long long>(W) * H));
        const Neighbours nb = neighbours(i, j, oH, oW);
        T weight = 0, n = 0, ml[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ml[k] = nb.inside[k] ? maskLow.data_[at3(maskLow, b, nb.ii[k], nb.jj[k])] : T(0);
            if (nb.inside[k]) {
                weight += nb.w[k];
                n += nb.w[k] * ml[k];
            }
        }
        const T m = mask.data_[at3(mask, b, i, j)];
        T adjMask = 0, adjN = 0, adjMaskLow[4] = {0, 0, 0, 0};
        for (int c = 0; c < C; ++c) {
            T d = 0, dl[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                dl[k] = nb.inside[k] ? dataLow.data_[at4(dataLow, b, c, nb.ii[k], nb.jj[k])] : T(0);
                if (nb.inside[k]) d += nb.w[k] * ml[k] * dl[k];
            }
            const T g = gradDataHigh.data_[at4(gradDataHigh, b, c, i, j)];
            // dataHigh = m * data + (1 - m) * (n > 0 ? d / n : 0)
            adjMask += g * (data.data_[at4(data, b, c, i, j)] - (n > 0 ? d / n : T(0)));
            gradData.data_[at4(gradData, b, c, i, j)] += g * m;
            const T adjD = n > 0 ? g * (1 - m) / n : T(0);
            if (n > 0) adjN -= g * (1 - m) * d / (n * n);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (nb.inside[k]) {
                    adjMaskLow[k] += adjD * nb.w[k] * dl[k];
                    atomicAccumulate(gradDataLow.data_ + at4(gradDataLow, b, c, nb.ii[k], nb.jj[k]), adjD * nb.w[k] * ml[k]);
                }
        }
        // maskHigh = m + (n > 0 ? (1 - m) * n / weight : 0)
        const T gm = gradMaskHigh.data_[at3(gradMaskHigh, b, i, j)];
        adjMask += gm * (1 - (n / weight));
        adjN += gm * ((1 - m) / weight);
        gradMask.data_[at3(gradMask, b, i, j)] += adjMask;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (nb.inside[k])
                atomicAccumulate(gradMaskLow.data_ + at3(gradMaskLow, b, nb.ii[k], nb.jj[k]), adjMaskLow[k] + adjN * nb.w[k]);
    }
}

namespace pullpush
{
/** Offsets of the idx-th entry (row-major over dst's sizes) in dst and src. */
template <typename D, typename S, int N>
__device__ __forceinline__ void offsetsOf(long long idx, const TensorAccessor<D, N>& dst, const TensorAccessor<S, N>& src,
                                          long long& od, long long& os)
{
    od = 0;
    os = 0;
#pragma unroll
    for (int k = N - 1; k >= 0; --k) {
        const long long c = idx % dst.sizes_[k];
        idx /= dst.sizes_[k];
        od += c * dst.strides_[k];
        os += c * src.strides_[k];
    }
}
} // namespace pullpush

/** dst += src for tensors of 3 or 4 dimensions (the coarsest pyramid level passes its gradients through). */
template <typename T, int N>
__global__ void __launch_bounds__(256) PullPushAddKernel(long long numel, TensorAccessor<T, N> dst, const TensorAccessor<const T, N> src)
{
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        long long od, os;
        pullpush::offsetsOf(idx, dst, src, od, os);
        dst.data_[od] += src.data_[os];
    }
}

/** dst = src for tensors of any strides (an image of one row or column is its own inpainting). */
template <typename T, int N>
__global__ void __launch_bounds__(256) PullPushCopyKernel(long long numel, TensorAccessor<T, N> dst, const TensorAccessor<const T, N> src)
{
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        long long od, os;
        pullpush::offsetsOf(idx, dst, src, od, os);
        dst.data_[od] = src.data_[os];
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
