#include <qmlp/tensor.h>

#include "qmlp_hip.h"

QUICKMLP_NAMESPACE_BEGIN

namespace internal {
struct device_delete
{
    void operator()(void* const p) const { qmlp_hip_free(p); }
};
} // namespace internal

const int Tensor::BytesPerEntry[] = {4, 2, 8};
const std::string Tensor::DatatypePerEntry[] = {"float", "half", "double"};
const std::string Tensor::NamePerEntry[] = {"FLOAT", "HALF", "DOUBLE"};

Tensor::Tensor(Precision precision, const std::vector<int32_t>& sizes)
    : hostsData_(true)
    , data_(static_cast<void*>(nullptr))
    , precision_(precision)
    , ndim_(static_cast<int>(sizes.size()))
    , sizes_(sizes)
    , strides_(sizes.size())
{
    if (ndim_ <= 0) throw std::runtime_error("Tensor: at least one dimension required");
    int64_t stride = 1;
    for (int n = ndim_ - 1; n >= 0; --n) {
        strides_[n] = static_cast<int32_t>(stride);
        stride *= sizes[n];
    }
    void* mem = nullptr;
    // keep at least one entry so that rawPtr() of an empty batch is still a valid pointer
    QMLP_HIP_CALL(qmlp_hip_malloc(&mem, static_cast<size_t>(std::max<int64_t>(stride, 1)) * BytesPerEntry[precision]));
    data_ = std::shared_ptr<void>(mem, internal::device_delete());
}

const void* Tensor::rawPtr() const
{
    if (!defined()) throw std::runtime_error("Attempt to obtain pointer to an empty tensor");
    if (std::holds_alternative<void*>(data_)) return std::get<void*>(data_);
    return std::get<std::shared_ptr<void>>(data_).get();
}

void* Tensor::rawPtr()
{
    if (!defined()) throw std::runtime_error("Attempt to obtain pointer to an empty tensor");
    if (std::holds_alternative<void*>(data_)) return std::get<void*>(data_);
    return std::get<std::shared_ptr<void>>(data_).get();
}

void Tensor::zero_()
{
    zeroAsync_(nullptr);
    QMLP_HIP_CALL(qmlp_hip_stream_synchronize(nullptr));
}

void Tensor::zeroAsync_(stream_t stream)
{
    QMLP_HIP_CALL(qmlp_hip_memset_async(rawPtr(), 0, static_cast<size_t>(numBytes()), stream));
}

void Tensor::copyFromHost(const void* src, size_t bytes)
{
    if (bytes > static_cast<size_t>(numBytes())) throw std::runtime_error("copyFromHost: too many bytes");
    QMLP_HIP_CALL(qmlp_hip_memcpy_h2d(rawPtr(), src, bytes, nullptr));
}

void Tensor::copyToHost(void* dst, size_t bytes) const
{
    if (bytes > static_cast<size_t>(numBytes())) throw std::runtime_error("copyToHost: too many bytes");
    QMLP_HIP_CALL(qmlp_hip_memcpy_d2h(dst, rawPtr(), bytes, nullptr));
}

void Tensor::copy_(const Tensor& src)
{
    copyAsync_(src, nullptr);
    QMLP_HIP_CALL(qmlp_hip_stream_synchronize(nullptr));
}

void Tensor::copyAsync_(const Tensor& src, stream_t stream)
{
    CHECK_DIM(src, ndim());
    for (int d = 0; d < ndim(); ++d) {
        CHECK_SIZE(src, d, size(d));
        CHECK_ERROR(src.strides()[d] == strides()[d], "Strides must match!");
    }
    CHECK_DTYPE(src, precision());
    QMLP_HIP_CALL(qmlp_hip_memcpy_d2d(rawPtr(), src.rawPtr(), static_cast<size_t>(numBytes()), stream));
}

QUICKMLP_NAMESPACE_END
