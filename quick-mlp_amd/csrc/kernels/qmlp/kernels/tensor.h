#pragma once
// Strided tensor accessors passed by value to the kernels: a data pointer plus
// 32-bit sizes and strides (in elements). The same definition is compiled by the
// host code and, at run time, by the device compiler; it is the kernel ABI of
// every tensor argument.

namespace qmlp { namespace kernel {

template <typename T, int N>
struct TensorAccessor
{
    typedef T Type;
    T* data_;
    int sizes_[N];
    int strides_[N];

#ifdef __HIP_DEVICE_COMPILE__
    __device__ __forceinline__ int size(int i) const { return sizes_[i]; }
    __device__ __forceinline__ int stride(int i) const { return strides_[i]; }
    __device__ __forceinline__ T* data() const { return data_; }
#else
    int size(int i) const { return sizes_[i]; }
    int stride(int i) const { return strides_[i]; }
    T* data() const { return data_; }
#endif
};

template <typename T> using Tensor1Read = TensorAccessor<const T, 1>;
template <typename T> using Tensor2Read = TensorAccessor<const T, 2>;
template <typename T> using Tensor1RW = TensorAccessor<T, 1>;
template <typename T> using Tensor2RW = TensorAccessor<T, 2>;

}} // namespace qmlp::kernel
