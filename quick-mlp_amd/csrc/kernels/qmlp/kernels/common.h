#pragma once
// Device-side basics shared by every runtime-compiled QuickMLP kernel (gfx950, wave64).

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <qmlp/kernels/tensor.h>

#define QUICKMLP_KERNEL_NAMESPACE ::qmlp::kernel
#define QUICKMLP_KERNEL_NAMESPACE_BEGIN namespace qmlp { namespace kernel {
#define QUICKMLP_KERNEL_NAMESPACE_END }}

QUICKMLP_KERNEL_NAMESPACE_BEGIN

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// One wavefront works on a tile of 64 points: NT column tiles of 16 points each.
// Lane l = 16*g + r. In an MFMA accumulator tile the lane holds output rows
// 4g..4g+3 (channels) of column r; column r of column-tile nt is point 4*r + nt
// of the 64-point tile, so that one lane owns 4 consecutive points per channel.
constexpr int WAVE_SIZE = 64;
constexpr int TILE_POINTS = 64;
constexpr int NT = 4;

__device__ __forceinline__ half hZERO() { return __half_raw{static_cast<f16>(0)}; }
__device__ __forceinline__ half2 h2ZERO() { return __half2{hZERO(), hZERO()}; }

__device__ __forceinline__ half toHalf(f16 v) { return __half_raw{v}; }
__device__ __forceinline__ f16 fromHalf(half v) { return static_cast<__half_raw>(v).data; }

/**
 * Transcendental functions of the half-precision intrinsics vocabulary that activation
 * snippets use (hsin, hcos, hexp), evaluated with the hardware's fp32 units on the
 * fp16 argument: convert, one multiply, one quarter-rate instruction, convert back.
 * The library versions of the HIP headers run a software argument reduction of some
 * forty instructions per value, which made sine networks ALU-bound at a small fraction
 * of the matrix-core rate. The results differ from the correctly rounded ones by at
 * most one fp16 ulp.
 *
 * They are function objects on purpose: a snippet inside this namespace that calls
 * hsin(x) finds the object by ordinary lookup, and because that is not a function, the
 * argument-dependent lookup that would also bring in ::hsin(__half) does not take place.
 */
namespace fastmath
{
/** x * c in fp32 from the fp16 x. Written as a fused multiply-add with a zero addend (the same value, bit for
 *  bit): the compiler then takes v_fma_mix_f32, which reads either half of a register as its fp16 operand, instead
 *  of a conversion (and a shift for the upper half) followed by a multiply. */
__device__ __forceinline__ float scaled(half x, float c)
{
    return __builtin_fmaf(__half2float(x), c, 0.0f);
}
struct Sin
{
    __device__ __forceinline__ half operator()(half x) const
    {
        // v_sin_f32 takes revolutions and is defined on [-256, 256]
        return __float2half(__builtin_amdgcn_sinf(__builtin_amdgcn_fractf(scaled(x, 0.15915494309189535f))));
    }
};
struct Cos
{
    __device__ __forceinline__ half operator()(half x) const
    {
        return __float2half(__builtin_amdgcn_cosf(__builtin_amdgcn_fractf(scaled(x, 0.15915494309189535f))));
    }
};
struct Exp
{
    __device__ __forceinline__ half operator()(half x) const
    {
        return __float2half(__builtin_amdgcn_exp2f(scaled(x, 1.4426950408889634f)));
    }
};
}
static constexpr fastmath::Sin hsin{};
static constexpr fastmath::Cos hcos{};
static constexpr fastmath::Exp hexp{};

/** Templated casting between float and half datatypes */
template <typename Dst, typename Src> __device__ __forceinline__ Dst fcast(const Src& src);
template <> __device__ __forceinline__ float fcast<float, half>(const half& src) { return __half2float(src); }
template <> __device__ __forceinline__ float fcast<float, float>(const float& src) { return src; }
template <> __device__ __forceinline__ half fcast<half, half>(const half& src) { return src; }
template <> __device__ __forceinline__ half fcast<half, float>(const float& src) { return __float2half(src); }
template <> __device__ __forceinline__ float fcast<float, f16>(const f16& src) { return static_cast<float>(src); }
template <> __device__ __forceinline__ f16 fcast<f16, float>(const float& src) { return static_cast<f16>(src); }
template <> __device__ __forceinline__ f16 fcast<f16, f16>(const f16& src) { return src; }

/**
 * Orders LDS traffic between the lanes of one wavefront: everything written before
 * is visible to every lane's reads after. Waves run their tile loops independently,
 * so a workgroup barrier must not be used inside them.
 */
__device__ __forceinline__ void waveLdsSync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

/**
 * Makes the compiler materialise the activations of a tile at this point of the program.
 * Used in front of workgroup barriers inside the layer sequence: otherwise the matrix
 * instructions that produce them are sunk behind the barrier (they touch no memory), while
 * the LDS reads feeding them have to stay in front of it, and the operands of whole layers
 * end up spilled to scratch memory in between.
 */
template <int A, int B>
__device__ __forceinline__ void materialize(f16x4 (&x)[A][B])
{
#pragma unroll
    for (int a = 0; a < A; ++a)
#pragma unroll
        for (int b = 0; b < B; ++b) asm volatile("" : "+v"(x[a][b]));
}

/** Row of the per-wave staging area that holds point p (0..63) of the tile. Points
 *  4r+nt (fixed nt) of the 16 lanes r land in 16 consecutive rows, which together with
 *  an odd multiple of 16 bytes as row stride makes the tile reads bank-conflict free. */
__device__ __forceinline__ int stageRow(int p) { return ((p & 3) << 4) | (p >> 2); }

__device__ __forceinline__ f16x8 concat(f16x4 a, f16x4 b)
{
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ f16x4 toF16(f32x4 v)
{
    // as one vector conversion: two packed round-to-nearest conversions instead of four
    // scalar ones and two packs
    return __builtin_convertvector(v, f16x4);
}

/** Detects the optional packed form `static f16x4 forward4(f16x4)` of an activation. */
template <typename Act, typename = void>
struct HasPackedForward
{
    static constexpr bool value = false;
};
template <typename Act>
struct HasPackedForward<Act, decltype(void(Act::forward4(f16x4{})))>
{
    static constexpr bool value = true;
};

/** Detects composites with one activation per channel (forwardAt / adjointAt with a channel). */
template <typename Act, typename = void>
struct IsPerChannel
{
    static constexpr bool value = false;
};
template <typename Act>
struct IsPerChannel<Act, decltype(void(Act::PerChannel))>
{
    static constexpr bool value = true;
};

/** Activation of 4 values that belong to the consecutive channels channel0 .. channel0+3. */
template <typename Act>
__device__ __forceinline__ f16x4 activationForwardChannels(f16x4 v, int channel0);

/** Activation of values that all belong to the same channel. */
template <typename Act>
__device__ __forceinline__ f16x8 activationForwardChannel(f16x8 v, int channel);

template <typename Act>
__device__ __forceinline__ half activationAdjointChannel(half x, half adjz, int channel)
{
    if constexpr (IsPerChannel<Act>::value) return Act::adjointAt(x, adjz, channel);
    else return Act::adjoint(x, adjz);
}

template <typename Act>
__device__ __forceinline__ f16x4 activationForward(f16x4 v)
{
    if constexpr (HasPackedForward<Act>::value) {
        return Act::forward4(v);
    } else {
        f16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = fromHalf(Act::forward(toHalf(v[i])));
        return o;
    }
}

template <typename Act>
__device__ __forceinline__ f16x8 activationForward(f16x8 v)
{
    const f16x4 lo = activationForward<Act>(f16x4{v[0], v[1], v[2], v[3]});
    const f16x4 hi = activationForward<Act>(f16x4{v[4], v[5], v[6], v[7]});
    return concat(lo, hi);
}

template <typename Act>
__device__ __forceinline__ f16x4 activationForwardChannels(f16x4 v, int channel0)
{
    if constexpr (IsPerChannel<Act>::value) {
        f16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = fromHalf(Act::forwardAt(toHalf(v[i]), channel0 + i));
        return o;
    } else {
        return activationForward<Act>(v);
    }
}

template <typename Act>
__device__ __forceinline__ f16x8 activationForwardChannel(f16x8 v, int channel)
{
    if constexpr (IsPerChannel<Act>::value) {
        f16x8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = fromHalf(Act::forwardAt(toHalf(v[i]), channel));
        return o;
    } else {
        return activationForward<Act>(v);
    }
}

/** One row of a strided 2-D tensor. */
template <typename T>
struct RowAccessor
{
    T* p;
    int stride;
    __device__ __forceinline__ T& operator[](int i) const { return p[static_cast<long long>(i) * stride]; }
};

QUICKMLP_KERNEL_NAMESPACE_END
