#pragma once

#include "common.h"
#include "errors.h"

#include <array>
#include <cassert>
#include <memory>
#include <random>
#include <string>
#include <type_traits>
#include <variant>
#include <vector>

#include <qmlp/kernels/tensor.h>

QUICKMLP_NAMESPACE_BEGIN

/**
 * Describes an N-dimensional strided tensor in device memory.
 * Datatype can be 'float', 'half' or 'double'.
 * Either wraps external memory (non-owning) or hosts its own allocation.
 */
class Tensor
{
public:
    enum Precision { FLOAT, HALF, DOUBLE, _NUM_PRECISION_ };
    static const int BytesPerEntry[];
    static const std::string DatatypePerEntry[];
    static const std::string NamePerEntry[];

    enum Usage { INFERENCE, GRADIENTS };

private:
    bool hostsData_;
    std::variant<void*, std::shared_ptr<void>> data_;
    Precision precision_;
    int ndim_;
    std::vector<int32_t> sizes_;
    std::vector<int32_t> strides_;

    template <typename T>
    void assertType() const
    {
        typedef std::remove_cv_t<T> U;
        if (std::is_void_v<U>) return;
        if (precision_ == FLOAT && !std::is_same_v<float, U>)
            throw configuration_error("Illegal type, the tensor stores float data!");
        if (precision_ == HALF && !std::is_same_v<half, U>)
            throw configuration_error("Illegal type, the tensor stores half data!");
        if (precision_ == DOUBLE && !std::is_same_v<double, U>)
            throw configuration_error("Illegal type, the tensor stores double data!");
    }

public:
    /** Constructs an undefined tensor (defined() == false) */
    Tensor() : hostsData_(false), data_(static_cast<void*>(nullptr)), precision_(FLOAT), ndim_(0) {}

    /**
     * Wraps external device memory. The caller keeps the memory alive for the
     * lifetime of this instance.
     */
    Tensor(void* data, Precision precision, const std::vector<int32_t>& sizes, const std::vector<int32_t>& strides)
        : hostsData_(false), data_(data), precision_(precision), ndim_(static_cast<int>(sizes.size())),
          sizes_(sizes), strides_(strides)
    {
        if (sizes.empty() || sizes.size() != strides.size())
            throw std::runtime_error("Tensor: sizes and strides must be non-empty and of equal length");
    }

    /** Allocates device memory of the given shape (contiguous, row-major) and owns it. */
    Tensor(Precision precision, const std::vector<int32_t>& sizes);

    [[nodiscard]] bool defined() const { return ndim_ > 0; }
    [[nodiscard]] Precision precision() const { return precision_; }
    [[nodiscard]] int bytesPerEntry() const { return BytesPerEntry[precision_]; }
    [[nodiscard]] int ndim() const { return ndim_; }
    [[nodiscard]] const std::vector<int32_t>& sizes() const { return sizes_; }
    [[nodiscard]] int32_t size(int dim) const { return sizes_[dim]; }
    [[nodiscard]] const std::vector<int32_t>& strides() const { return strides_; }
    [[nodiscard]] int32_t stride(int dim) const { return strides_[dim]; }

    [[nodiscard]] int64_t numel() const
    {
        int64_t n = 1;
        for (int i = 0; i < ndim_; ++i) n *= sizes_[i];
        return n;
    }

    /** Bytes between the first and one past the last addressed entry. */
    [[nodiscard]] int64_t numBytes() const
    {
        int64_t lastIdx = 0;
        for (int i = 0; i < ndim_; ++i) {
            if (sizes_[i] == 0) return 0;
            lastIdx += static_cast<int64_t>(strides_[i]) * (sizes_[i] - 1);
        }
        return (lastIdx + 1) * BytesPerEntry[precision_];
    }

    [[nodiscard]] int64_t idx(std::initializer_list<int32_t> l) const
    {
        assert(static_cast<int>(l.size()) == ndim());
        int64_t idx = 0;
        for (size_t i = 0; i < l.size(); ++i) idx += static_cast<int64_t>(l.begin()[i]) * strides_[i];
        return idx;
    }

    [[nodiscard]] const void* rawPtr() const;
    [[nodiscard]] void* rawPtr();

    template <typename T>
    [[nodiscard]] const T* dataPtr() const
    {
        assertType<T>();
        return static_cast<const T*>(rawPtr());
    }
    template <typename T>
    [[nodiscard]] T* dataPtr()
    {
        assertType<T>();
        return static_cast<T*>(rawPtr());
    }

    /** Fills [first entry, last entry] with zeros (also entries skipped by the strides). */
    void zero_();
    void zeroAsync_(stream_t stream);

    /** Fills this (contiguous) tensor with uniform random numbers in [a,b]. */
    template <typename RNG>
    void rand_(float a, float b, RNG& rng)
    {
        std::uniform_real_distribution<float> distr(a, b);
        const int64_t n = numel();
        if (precision_ == FLOAT) {
            std::vector<float> data(n);
            for (int64_t i = 0; i < n; ++i) data[i] = distr(rng);
            copyFromHost(data.data(), sizeof(float) * n);
        } else if (precision_ == HALF) {
            std::vector<half> data(n);
            for (int64_t i = 0; i < n; ++i) data[i] = static_cast<half>(distr(rng));
            copyFromHost(data.data(), sizeof(half) * n);
        } else {
            std::vector<double> data(n);
            for (int64_t i = 0; i < n; ++i) data[i] = distr(rng);
            copyFromHost(data.data(), sizeof(double) * n);
        }
    }

    /** Synchronous raw copies between host memory and this tensor's memory range. */
    void copyFromHost(const void* src, size_t bytes);
    void copyToHost(void* dst, size_t bytes) const;

    /** Copies 'src' into 'this'. Size, stride, precision must match. */
    void copy_(const Tensor& src);
    void copyAsync_(const Tensor& src, stream_t stream);

    /**
     * Returns the kernel accessor (data pointer + int32 sizes/strides) for this tensor.
     * \tparam Accessor e.g. qmlp::kernel::Tensor2RW<float>
     */
    template <typename Accessor>
    Accessor accessor() const
    {
        typedef typename Accessor::Type T;
        Accessor a;
        a.data_ = const_cast<T*>(static_cast<const T*>(dataPtr<std::remove_cv_t<T>>()));
        constexpr int N = sizeof(a.sizes_) / sizeof(int);
        if (N != ndim_) throw std::runtime_error("accessor(): dimension mismatch");
        for (int i = 0; i < N; ++i) {
            a.sizes_[i] = sizes_[i];
            a.strides_[i] = strides_[i];
        }
        return a;
    }
};

QUICKMLP_NAMESPACE_END
