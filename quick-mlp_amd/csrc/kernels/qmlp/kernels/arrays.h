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

/**
 * Encoded rows of PPL points of a lane that wait in registers, two halves per 32-bit register,
 * one register vector per point. The point index has to be a compile-time constant once the
 * loops over the points are unrolled; the register of a point may be selected by a value that
 * is uniform over the wavefront (a level counter): that is one indexed register move.
 */
template <typename T, int PPL, int C>
struct PackedRegisterRows
{
    static_assert(sizeof(T) == 2, "two values per register");
    typedef unsigned int Vector __attribute__((ext_vector_type(C / 2)));
    Vector data_[PPL];
};

/** The rows of PackedRegisterRows from channel OFFSET on: rows[q][i] = value. */
template <typename T, int PPL, int C, int OFFSET>
struct PackedRegisterRowsView
{
    typedef T ValueType;
    typedef PackedRegisterRows<T, PPL, C> Rows;
    struct Element
    {
        typename Rows::Vector& vector_;
        int channel_;
        __device__ __forceinline__ void operator=(T v) const
        {
            const unsigned int bits = __builtin_bit_cast(unsigned short, v);
            const unsigned int old = vector_[channel_ >> 1];
            vector_[channel_ >> 1] = (channel_ & 1) ? ((old & 0xffffu) | (bits << 16)) : ((old & 0xffff0000u) | bits);
        }
    };
    struct Row
    {
        typedef T ValueType;
        Rows& rows_;
        int q_;
        __device__ __forceinline__ Element operator[](int i) const { return Element{rows_.data_[q_], i + OFFSET}; }
    };
    Rows& rows_;
    __device__ __forceinline__ Row operator[](int q) const { return Row{rows_, q}; }
};

/** rows[q][i] = a, rows[q][i + 1] = b for an even channel i. */
template <typename Rows, typename T>
__device__ __forceinline__ void storePair(Rows& rows, int q, int i, T a, T b)
{
    rows[q][i] = a;
    rows[q][i + 1] = b;
}
template <typename T, int PPL, int C, int OFFSET>
__device__ __forceinline__ void storePair(PackedRegisterRowsView<T, PPL, C, OFFSET>& rows, int q, int i, T a, T b)
{
    static_assert(OFFSET % 2 == 0, "pairs start at even channels");
    const unsigned int lo = __builtin_bit_cast(unsigned short, a), hi = __builtin_bit_cast(unsigned short, b);
    rows.rows_.data_[q][(i + OFFSET) >> 1] = lo | (hi << 16);
}

/** Element type of a set of output rows: a C array of row views, or PackedRegisterRowsView. */
template <typename Rows>
struct RowsValueType
{
    typedef typename Rows::ValueType Type;
};
template <typename Row, int N>
struct RowsValueType<Row[N]>
{
    typedef typename Row::ValueType Type;
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
