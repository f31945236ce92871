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
// re-read from cache), the adjoint of `down` adds with atomics when the windows of
// neighbouring low-res pixels overlap (odd sizes; the reference adds without), and the adjoint
// of `up` gathers per low-res pixel in a second pass instead of scattering with atomics.

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

/** Pixel (b, i, j) of the idx-th entry of a (B, h, w) image stack; 32-bit divisions whenever they suffice. */
__device__ __forceinline__ void pixelOf(long long idx, int h, int w, int& b, int& i, int& j)
{
    if (idx <= 0x7fffffffLL) {
        const unsigned u = static_cast<unsigned>(idx), uw = static_cast<unsigned>(w), uh = static_cast<unsigned>(h);
        const unsigned row = u / uw;
        j = static_cast<int>(u - row * uw);
        b = static_cast<int>(row / uh);
        i = static_cast<int>(row - static_cast<unsigned>(b) * uh);
    } else {
        const long long row = idx / w;
        j = static_cast<int>(idx - row * w);
        b = static_cast<int>(row / h);
        i = static_cast<int>(row - static_cast<long long>(b) * h);
    }
}

/** The 4 low-res neighbours of high-res pixel (i, j) and their bilinear weights. A neighbour
 *  outside the image has weight 0 and the coordinates of the pixel's own low-res cell clamped
 *  into the image, so that it can be loaded without a branch. */
struct Neighbours
{
    int ii[4], jj[4];
    float w[4];
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
    for (int k = 0; k < 4; ++k) {
        const bool inside = n.ii[k] >= 0 && n.jj[k] >= 0 && n.ii[k] < oH && n.jj[k] < oW;
        n.w[k] = inside ? n.w[k] : 0.f;
        n.ii[k] = min(max(n.ii[k], 0), oH - 1);
        n.jj[k] = min(max(n.jj[k], 0), oW - 1);
    }
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
        int b, i, j;
        pixelOf(idx, oH, oW, b, i, j);
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
        int b, i, j;
        pixelOf(idx, H, W, b, i, j);
        const Neighbours nb = neighbours(i, j, oH, oW);
        T weight = 0, n = 0, ml[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ml[k] = maskLow.data_[at3(maskLow, b, nb.ii[k], nb.jj[k])];
            weight += nb.w[k];
            n += nb.w[k] * ml[k];
        }
        const T m = mask.data_[at3(mask, b, i, j)];
        maskHigh.data_[at3(maskHigh, b, i, j)] = m + (n > 0 ? (1 - m) * (n / weight) : T(0));
        for (int c = 0; c < C; ++c) {
            T d = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                d += nb.w[k] * ml[k] * dataLow.data_[at4(dataLow, b, c, nb.ii[k], nb.jj[k])];
            dataHigh.data_[at4(dataHigh, b, c, i, j)] = m * data.data_[at4(data, b, c, i, j)] + (1 - m) * (n > 0 ? d / n : T(0));
        }
    }
}

/**
 * Adjoint of PullPushDownKernel; one thread per low-res pixel, gradients accumulated.
 * \tparam OVERLAP the windows of neighbouring low-res pixels share high-res pixels (an odd
 *   height or width): accumulate with atomics. Otherwise every high-res pixel has one owner.
 */
template <typename T, bool OVERLAP>
__global__ void __launch_bounds__(256) PullPushAdjointDownKernel(
    long long numel, const Tensor3Read<T> mask, const Tensor4Read<T> data, const Tensor3Read<T> gradMaskLow,
    const Tensor4Read<T> gradDataLow, Tensor3RW<T> gradMask, Tensor4RW<T> gradData)
{
    using namespace pullpush;
    const int H = mask.sizes_[1], W = mask.sizes_[2], oH = H / 2, oW = W / 2, C = data.sizes_[1];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        int b, i, j;
        pixelOf(idx, oH, oW, b, i, j);
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
                    T* target = gradData.data_ + at4(gradData, b, c, ii, jj);
                    if (OVERLAP) atomicAccumulate(target, adjD * m);
                    else *target += adjD * m;
                    adjMask += adjD * data.data_[at4(data, b, c, ii, jj)];
                }
                if (n2 == m) adjMask += adjN2;   // the maximum passes its gradient to every pixel that attains it
                T* target = gradMask.data_ + at3(gradMask, b, ii, jj);
                if (OVERLAP) atomicAccumulate(target, adjMask);
                else *target += adjMask;
            }
    }
}

/**
 * Adjoint of PullPushUpKernel, first pass; one thread per high-res pixel. Adds the gradients of
 * this level's inputs into gradMask / gradData and stores what the low-res level needs from
 * this pixel: adjFill(b, c, i, j) = gradient of the channel's weighted low-res sum d_c,
 * adjFill(b, C, i, j) = gradient of the low-res mask sum n.
 */
template <typename T>
__global__ void __launch_bounds__(256) PullPushAdjointUpKernel(
    long long numel, const Tensor3Read<T> mask, const Tensor4Read<T> data, const Tensor3Read<T> maskLow,
    const Tensor4Read<T> dataLow, const Tensor3Read<T> gradMaskHigh, const Tensor4Read<T> gradDataHigh,
    Tensor3RW<T> gradMask, Tensor4RW<T> gradData, Tensor4RW<T> adjFill)
{
    using namespace pullpush;
    const int H = mask.sizes_[1], W = mask.sizes_[2], oH = H / 2, oW = W / 2, C = data.sizes_[1];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        int b, i, j;
        pixelOf(idx, H, W, b, i, j);
        const Neighbours nb = neighbours(i, j, oH, oW);
        T weight = 0, n = 0, ml[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ml[k] = maskLow.data_[at3(maskLow, b, nb.ii[k], nb.jj[k])];
            weight += nb.w[k];
            n += nb.w[k] * ml[k];
        }
        const T m = mask.data_[at3(mask, b, i, j)];
        T adjMask = 0, adjN = 0;
        for (int c = 0; c < C; ++c) {
            T d = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                d += nb.w[k] * ml[k] * dataLow.data_[at4(dataLow, b, c, nb.ii[k], nb.jj[k])];
            const T g = gradDataHigh.data_[at4(gradDataHigh, b, c, i, j)];
            // dataHigh = m * data + (1 - m) * (n > 0 ? d / n : 0)
            adjMask += g * (data.data_[at4(data, b, c, i, j)] - (n > 0 ? d / n : T(0)));
            gradData.data_[at4(gradData, b, c, i, j)] += g * m;
            if (n > 0) adjN -= g * (1 - m) * d / (n * n);
            adjFill.data_[at4(adjFill, b, c, i, j)] = n > 0 ? g * (1 - m) / n : T(0);
        }
        // maskHigh = m + (n > 0 ? (1 - m) * n / weight : 0)
        const T gm = gradMaskHigh.data_[at3(gradMaskHigh, b, i, j)];
        adjMask += gm * (1 - (n / weight));
        adjN += gm * ((1 - m) / weight);
        gradMask.data_[at3(gradMask, b, i, j)] += adjMask;
        adjFill.data_[at4(adjFill, b, C, i, j)] = adjN;
    }
}

/**
 * Adjoint of PullPushUpKernel, second pass; one thread per low-res pixel (b, ii, jj). Gathers
 * from the up to 4 x 4 high-res pixels that interpolate from it (rows 2ii-1 .. 2ii+2: the two
 * inner ones with weight 3/4, the outer ones with 1/4; columns alike), so no atomics are
 * needed (the reference scatters with atomicAdd, pullpush.cuh:256-273):
 *   gradDataLow_c += maskLow * sum_p w_p adjFill_c(p)
 *   gradMaskLow   += sum_p w_p (adjFill_C(p) + sum_c adjFill_c(p) dataLow_c)
 */
template <typename T>
__global__ void __launch_bounds__(256) PullPushAdjointUpGatherKernel(
    long long numel, const Tensor3Read<T> maskLow, const Tensor4Read<T> dataLow, const Tensor4Read<T> adjFill,
    Tensor3RW<T> gradMaskLow, Tensor4RW<T> gradDataLow)
{
    using namespace pullpush;
    const int oH = maskLow.sizes_[1], oW = maskLow.sizes_[2], C = dataLow.sizes_[1];
    const int H = adjFill.sizes_[2], W = adjFill.sizes_[3];
    for (long long idx = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; idx < numel;
         idx += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        int b, ii, jj;
        pixelOf(idx, oH, oW, b, ii, jj);
        const T ml = maskLow.data_[at3(maskLow, b, ii, jj)];
        T sumN = 0, adjMaskLow = 0;
#pragma unroll
        for (int di = -1; di <= 2; ++di) {
            const int i = 2 * ii + di;
            if (i < 0 || i >= H) continue;
#pragma unroll
            for (int dj = -1; dj <= 2; ++dj) {
                const int j = 2 * jj + dj;
                if (j < 0 || j >= W) continue;
                const float w = ((di == 0 || di == 1) ? 0.75f : 0.25f) * ((dj == 0 || dj == 1) ? 0.75f : 0.25f);
                sumN += w * adjFill.data_[at4(adjFill, b, C, i, j)];
            }
        }
        for (int c = 0; c < C; ++c) {
            T sumD = 0;
#pragma unroll
            for (int di = -1; di <= 2; ++di) {
                const int i = 2 * ii + di;
                if (i < 0 || i >= H) continue;
#pragma unroll
                for (int dj = -1; dj <= 2; ++dj) {
                    const int j = 2 * jj + dj;
                    if (j < 0 || j >= W) continue;
                    const float w = ((di == 0 || di == 1) ? 0.75f : 0.25f) * ((dj == 0 || dj == 1) ? 0.75f : 0.25f);
                    sumD += w * adjFill.data_[at4(adjFill, b, c, i, j)];
                }
            }
            gradDataLow.data_[at4(gradDataLow, b, c, ii, jj)] += sumD * ml;
            adjMaskLow += sumD * dataLow.data_[at4(dataLow, b, c, ii, jj)];
        }
        gradMaskLow.data_[at3(gradMaskLow, b, ii, jj)] += adjMaskLow + sumN;
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
