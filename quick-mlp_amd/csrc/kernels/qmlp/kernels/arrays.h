#pragma once
// Small per-thread views used as inputs / outputs of the encodings.

#include <qmlp/kernels/common.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

/** Fixed-size register array. */
template <typename T, int N>
struct StaticArray
{
    typedef T ValueType;
    T data_[N];
    __device__ __forceinline__ const T& operator[](int i) const { return data_[i]; }
    __device__ __forceinline__ T& operator[](int i) { return data_[i]; }
};

/** Pointer wrapper (LDS row or global row with unit stride). */
template <typename T>
struct WrappedArray
{
    typedef T ValueType;
    T* data_;
    __device__ __forceinline__ const T& operator[](int i) const { return data_[i]; }
    __device__ __forceinline__ T& operator[](int i) { return data_[i]; }
    __device__ __forceinline__ WrappedArray<T> operator+(int i) const { return WrappedArray<T>{data_ + i}; }
};

/** Strided global row. */
template <typename T>
struct StridedArray
{
    typedef T ValueType;
    T* data_;
    int stride_;
    __device__ __forceinline__ T& operator[](int i) const { return data_[static_cast<long long>(i) * stride_]; }
    __device__ __forceinline__ StridedArray<T> operator+(int i) const
    {
        return StridedArray<T>{data_ + static_cast<long long>(i) * stride_, stride_};
    }
};

QUICKMLP_KERNEL_NAMESPACE_END
