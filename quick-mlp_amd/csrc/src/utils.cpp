#include <qmlp/utils.h>

#include <qmlp/errors.h>
#include <qmlp/qmlp.h>

#include "qmlp_hip.h"

#include <algorithm>
#include <map>
#include <mutex>
#include <vector>

QUICKMLP_NAMESPACE_BEGIN

namespace {

const char* scalarName(Tensor::Precision p)
{
    if (p == Tensor::FLOAT) return "float";
    if (p == Tensor::DOUBLE) return "double";
    throw std::runtime_error("fractionalPullpush works on float or double tensors");
}

const char* const KERNEL_NAMES[] = {"PullPushDownKernel<$T>", "PullPushUpKernel<$T>", "PullPushAdjointUpKernel<$T>",
                                    "PullPushAdjointUpGatherKernel<$T>", "PullPushAdjointDownKernel<$T, true>",
                                    "PullPushAdjointDownKernel<$T, false>", "PullPushAddKernel<$T, 3>",
                                    "PullPushAddKernel<$T, 4>", "PullPushCopyKernel<$T, 3>",
                                    "PullPushCopyKernel<$T, 4>"};

std::string pullpushSource() { return KernelLoader::MainFile("qmlp/kernels/pullpush.h"); }

/** The compiled kernels stay loaded for the life of the process, like the reference's static kernels. */
KernelFunction pullpushKernel(const std::string& name)
{
    static std::mutex mutex;
    static std::map<std::string, KernelFunction> kernels;
    std::lock_guard<std::mutex> lock(mutex);
    auto it = kernels.find(name);
    if (it == kernels.end()) {
        auto kl = QuickMLP::Instance().kernelLoader();
        auto fun = kl->getKernel("qmlp::kernel::" + name, pullpushSource(), QuickMLP::Instance().getCompileFlags());
        it = kernels.emplace(name, fun.value()).first;
    }
    return it->second;
}

template <typename T, int N>
kernel::TensorAccessor<T, N> accessorOf(const Tensor& t)
{
    return t.accessor<kernel::TensorAccessor<T, N>>();
}

void launch(KernelFunction& fun, long long numel, stream_t stream, std::vector<void*> args)
{
    if (numel == 0) return;
    const int block = 256;
    const int grid = static_cast<int>(std::min<long long>(divUp<long long>(numel, block), fun.fullGridSize(block, 0)));
    std::vector<void*> all = {&numel};
    all.insert(all.end(), args.begin(), args.end());
    fun.launch(grid, block, 0, stream, all.data());
}

/** One pyramid level: the down-sampled inputs and the inpainted low-res result. */
struct Level
{
    Tensor maskLowPre, dataLowPre, maskLowPost, dataLowPost;
};

template <typename T>
void forwardRecursion(const Tensor& maskInput, const Tensor& dataInput, Tensor& maskOutput, Tensor& dataOutput,
                      std::vector<Level>* saved, stream_t stream)
{
    const int B = dataInput.size(0), C = dataInput.size(1), H = dataInput.size(2), W = dataInput.size(3);
    const auto dtype = dataInput.precision();
    if (H <= 1 || W <= 1) {
        // end of the recursion: nothing coarser to fill from
        const std::string t = scalarName(dtype);
        auto copy3 = pullpushKernel("PullPushCopyKernel<" + t + ", 3>");
        auto copy4 = pullpushKernel("PullPushCopyKernel<" + t + ", 4>");
        auto dstM = accessorOf<T, 3>(maskOutput);
        auto srcM = accessorOf<const T, 3>(maskInput);
        launch(copy3, maskOutput.numel(), stream, {&dstM, &srcM});
        auto dstD = accessorOf<T, 4>(dataOutput);
        auto srcD = accessorOf<const T, 4>(dataInput);
        launch(copy4, dataOutput.numel(), stream, {&dstD, &srcD});
        return;
    }
    const int oH = H / 2, oW = W / 2;
    const std::string t = scalarName(dtype);

    Level level;
    level.maskLowPre = Tensor(dtype, {B, oH, oW});
    level.dataLowPre = Tensor(dtype, {B, C, oH, oW});
    {
        auto fun = pullpushKernel("PullPushDownKernel<" + t + ">");
        auto mask = accessorOf<const T, 3>(maskInput);
        auto data = accessorOf<const T, 4>(dataInput);
        auto maskLow = accessorOf<T, 3>(level.maskLowPre);
        auto dataLow = accessorOf<T, 4>(level.dataLowPre);
        launch(fun, static_cast<long long>(B) * oH * oW, stream, {&mask, &data, &maskLow, &dataLow});
    }
    level.maskLowPost = Tensor(dtype, {B, oH, oW});
    level.dataLowPost = Tensor(dtype, {B, C, oH, oW});
    forwardRecursion<T>(level.maskLowPre, level.dataLowPre, level.maskLowPost, level.dataLowPost, saved, stream);
    {
        auto fun = pullpushKernel("PullPushUpKernel<" + t + ">");
        auto mask = accessorOf<const T, 3>(maskInput);
        auto data = accessorOf<const T, 4>(dataInput);
        auto maskLow = accessorOf<const T, 3>(level.maskLowPost);
        auto dataLow = accessorOf<const T, 4>(level.dataLowPost);
        auto maskHigh = accessorOf<T, 3>(maskOutput);
        auto dataHigh = accessorOf<T, 4>(dataOutput);
        launch(fun, static_cast<long long>(B) * H * W, stream, {&mask, &data, &maskLow, &dataLow, &maskHigh, &dataHigh});
    }
    // The temporaries of this level are freed when 'level' goes out of scope, which may be
    // before the kernels have run: keep them until the caller has synchronised.
    saved->push_back(std::move(level));
}

template <typename T>
void adjointRecursion(const Tensor& maskInput, const Tensor& dataInput, const Tensor& gradMaskOutput,
                      const Tensor& gradDataOutput, Tensor& gradMaskInput, Tensor& gradDataInput,
                      std::vector<Level>& saved, std::vector<Tensor>& keepAlive, stream_t stream)
{
    const int B = dataInput.size(0), C = dataInput.size(1), H = dataInput.size(2), W = dataInput.size(3);
    const auto dtype = dataInput.precision();
    const std::string t = scalarName(dtype);
    if (H <= 1 || W <= 1) {
        auto add3 = pullpushKernel("PullPushAddKernel<" + t + ", 3>");
        auto add4 = pullpushKernel("PullPushAddKernel<" + t + ", 4>");
        auto dstM = accessorOf<T, 3>(gradMaskInput);
        auto srcM = accessorOf<const T, 3>(gradMaskOutput);
        launch(add3, gradMaskInput.numel(), stream, {&dstM, &srcM});
        auto dstD = accessorOf<T, 4>(gradDataInput);
        auto srcD = accessorOf<const T, 4>(gradDataOutput);
        launch(add4, gradDataInput.numel(), stream, {&dstD, &srcD});
        return;
    }
    const int oH = H / 2, oW = W / 2;
    // the levels were saved coarsest first: the finest one is at the back
    Level level = std::move(saved.back());
    saved.pop_back();

    Tensor gradMaskLowPost(dtype, {B, oH, oW}), gradDataLowPost(dtype, {B, C, oH, oW});
    gradMaskLowPost.zeroAsync_(stream);
    gradDataLowPost.zeroAsync_(stream);
    // what every high-res pixel passes down: C channel terms and one mask term
    Tensor adjFill(dtype, {B, C + 1, H, W});
    {
        auto fun = pullpushKernel("PullPushAdjointUpKernel<" + t + ">");
        auto mask = accessorOf<const T, 3>(maskInput);
        auto data = accessorOf<const T, 4>(dataInput);
        auto maskLow = accessorOf<const T, 3>(level.maskLowPost);
        auto dataLow = accessorOf<const T, 4>(level.dataLowPost);
        auto gMaskHigh = accessorOf<const T, 3>(gradMaskOutput);
        auto gDataHigh = accessorOf<const T, 4>(gradDataOutput);
        auto gMask = accessorOf<T, 3>(gradMaskInput);
        auto gData = accessorOf<T, 4>(gradDataInput);
        auto fill = accessorOf<T, 4>(adjFill);
        launch(fun, static_cast<long long>(B) * H * W, stream,
               {&mask, &data, &maskLow, &dataLow, &gMaskHigh, &gDataHigh, &gMask, &gData, &fill});
    }
    {
        auto fun = pullpushKernel("PullPushAdjointUpGatherKernel<" + t + ">");
        auto maskLow = accessorOf<const T, 3>(level.maskLowPost);
        auto dataLow = accessorOf<const T, 4>(level.dataLowPost);
        auto fill = accessorOf<const T, 4>(adjFill);
        auto gMaskLow = accessorOf<T, 3>(gradMaskLowPost);
        auto gDataLow = accessorOf<T, 4>(gradDataLowPost);
        launch(fun, static_cast<long long>(B) * oH * oW, stream, {&maskLow, &dataLow, &fill, &gMaskLow, &gDataLow});
    }
    Tensor gradMaskLowPre(dtype, {B, oH, oW}), gradDataLowPre(dtype, {B, C, oH, oW});
    gradMaskLowPre.zeroAsync_(stream);
    gradDataLowPre.zeroAsync_(stream);
    adjointRecursion<T>(level.maskLowPre, level.dataLowPre, gradMaskLowPost, gradDataLowPost, gradMaskLowPre,
                        gradDataLowPre, saved, keepAlive, stream);
    {
        // windows of neighbouring low-res pixels overlap when a size is odd
        const bool overlap = (H % 2 != 0) || (W % 2 != 0);
        auto fun = pullpushKernel("PullPushAdjointDownKernel<" + t + (overlap ? ", true>" : ", false>"));
        auto mask = accessorOf<const T, 3>(maskInput);
        auto data = accessorOf<const T, 4>(dataInput);
        auto gMaskLow = accessorOf<const T, 3>(gradMaskLowPre);
        auto gDataLow = accessorOf<const T, 4>(gradDataLowPre);
        auto gMask = accessorOf<T, 3>(gradMaskInput);
        auto gData = accessorOf<T, 4>(gradDataInput);
        launch(fun, static_cast<long long>(B) * oH * oW, stream, {&mask, &data, &gMaskLow, &gDataLow, &gMask, &gData});
    }
    for (Tensor* x : {&level.maskLowPre, &level.dataLowPre, &level.maskLowPost, &level.dataLowPost, &gradMaskLowPost,
                      &gradDataLowPost, &gradMaskLowPre, &gradDataLowPre, &adjFill})
        keepAlive.push_back(std::move(*x));
}

void checkShapes(const Tensor& mask, const Tensor& data)
{
    CHECK_DIM(mask, 3);
    CHECK_DIM(data, 4);
    CHECK_SIZE(mask, 0, data.size(0));
    CHECK_SIZE(mask, 1, data.size(2));
    CHECK_SIZE(mask, 2, data.size(3));
    CHECK_DTYPE(mask, data.precision());
    CHECK_ERROR(data.precision() == Tensor::FLOAT || data.precision() == Tensor::DOUBLE,
                "fractionalPullpush works on float or double tensors");
    CHECK_ERROR(data.size(1) < 16, "fractionalPullpush only supports up to 16 channels, but got ", data.size(1));
}

void checkLike(const Tensor& x, const Tensor& like, const char* what)
{
    CHECK_ERROR(x.ndim() == like.ndim(), what, " has the wrong number of dimensions");
    for (int d = 0; d < like.ndim(); ++d) CHECK_ERROR(x.size(d) == like.size(d), what, " has the wrong size at dimension ", d);
    CHECK_DTYPE(x, like.precision());
}

void synchronize(stream_t stream)
{
    QMLP_HIP_CALL(qmlp_hip_stream_synchronize(stream));
}

} // namespace

void Utils::precompile(Tensor::Precision precision)
{
    const std::string t = scalarName(precision);
    auto kl = QuickMLP::Instance().kernelLoader();
    const int flags = QuickMLP::Instance().getCompileFlags() | KernelLoader::CompileOnly;
    for (const char* pattern : KERNEL_NAMES) {
        std::string name = pattern;
        name.replace(name.find("$T"), 2, t);
        kl->getKernel("qmlp::kernel::" + name, pullpushSource(), flags);
    }
}

void Utils::fractionalPullpush(const Tensor& mask, const Tensor& data, Tensor& output, stream_t stream)
{
    checkShapes(mask, data);
    checkLike(output, data, "output");
    if (data.numel() == 0) return;
    std::vector<Level> levels;
    Tensor maskOutput(data.precision(), mask.sizes());
    if (data.precision() == Tensor::FLOAT)
        forwardRecursion<float>(mask, data, maskOutput, output, &levels, stream);
    else
        forwardRecursion<double>(mask, data, maskOutput, output, &levels, stream);
    // the pyramid is temporary device memory of this call: wait before it is released
    synchronize(stream);
}

void Utils::adjointFractionalPullpush(const Tensor& mask, const Tensor& data, const Tensor& adjOutput, Tensor& adjMask,
                                      Tensor& adjData, stream_t stream)
{
    checkShapes(mask, data);
    checkLike(adjOutput, data, "adjOutput");
    checkLike(adjData, data, "adjData");
    checkLike(adjMask, mask, "adjMask");
    if (data.numel() == 0) return;
    const auto dtype = data.precision();
    std::vector<Level> levels;
    std::vector<Tensor> keepAlive;
    Tensor maskOutput(dtype, mask.sizes()), output(dtype, data.sizes()), gradMaskOutput(dtype, mask.sizes());
    gradMaskOutput.zeroAsync_(stream);   // only the data output has a gradient
    if (dtype == Tensor::FLOAT) {
        forwardRecursion<float>(mask, data, maskOutput, output, &levels, stream);
        adjointRecursion<float>(mask, data, gradMaskOutput, adjOutput, adjMask, adjData, levels, keepAlive, stream);
    } else {
        forwardRecursion<double>(mask, data, maskOutput, output, &levels, stream);
        adjointRecursion<double>(mask, data, gradMaskOutput, adjOutput, adjMask, adjData, levels, keepAlive, stream);
    }
    synchronize(stream);
}

QUICKMLP_NAMESPACE_END
