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

/**
 * Row of an LDS staging tile of the forward kernel. For row widths of 32, 64 or 128 halves
 * the rows carry no padding; instead the 8-byte chunks of a row are rotated by an amount
 * that depends on the row, such that the 16 rows x 4 chunks a wavefront reads as one
 * matrix-core operand fall onto distinct LDS banks (the padded layout spends 25 % more
 * LDS at 32 channels, which costs a workgroup per compute unit). Other widths keep a
 * padding of 8 halves and no rotation.
 */
template <int C>
struct StageLayout
{
    static constexpr bool Swizzle = (C == 32 || C == 64 || C == 128);
    static constexpr int Stride = Swizzle ? C : C + 8;   // halves
    static constexpr int Chunks = C / 4;                  // 8-byte chunks per row
    static constexpr int RowsPerBankPeriod = Swizzle ? 128 / C : 1;   // rows per 256 bytes
    /** Rotation (in chunks) of row `row` of a 64-row tile. */
    __device__ __forceinline__ static int rotation(int row)
    {
        if constexpr (Swizzle) return (2 * (row / RowsPerBankPeriod) + (row >> 4)) & (Chunks - 1);
        return 0;
    }
    /** Offset in halves of the 4-half chunk `chunk` of row `row` within the tile. */
    __device__ __forceinline__ static int chunkOffset(int row, int chunk)
    {
        if constexpr (Swizzle) return row * Stride + (((chunk + rotation(row)) & (Chunks - 1)) << 2);
        return row * Stride + (chunk << 2);
    }
};

template <typename T, int C>
struct StageRowArray
{
    typedef T ValueType;
    typedef StageLayout<C> Layout;
    T* row_;       // start of the row
    int rotation_;
    int offset_;   // logical channel of element 0
    __device__ __forceinline__ T& operator[](int i) const
    {
        const int j = i + offset_;
        if constexpr (Layout::Swizzle) return row_[((((j >> 2) + rotation_) & (Layout::Chunks - 1)) << 2) | (j & 3)];
        return row_[j];
    }
    __device__ __forceinline__ StageRowArray<T, C> operator+(int i) const
    {
        return StageRowArray<T, C>{row_, rotation_, offset_ + i};
    }
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
