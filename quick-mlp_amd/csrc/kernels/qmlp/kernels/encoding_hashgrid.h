#pragma once
// Multi-resolution dense + hashed latent grid, 1-D to 6-D, evaluated per point.
//
// The level table (resolution, dense or hashed, offset into the flat parameter
// tensor) is a pure function of the JSON specification, so the host bakes it into
// a generated configuration struct `Cfg`; every level is unrolled with its
// resolution, offset and hash-table size as literals. Only the table pointers and
// the bounding box travel as a kernel argument (HashGridParams), which replaces
// the per-call upload into __constant__ memory of the reference.
//
// Index arithmetic (must stay bit-exact with the reference,
// src_cpp/include/qmlp/kernels/encoding_hashgrid.cuh:17-60,72-85,279-287):
//   pos = (x - bbmin) * bbinv;  p = pos * (R-1);  iL = clamp(int(p), 0, R-1);
//   iH = clamp(int(p)+1, 0, R-1);  f = p - iL
//   dense:  idx = ((i0*R + i1)*R + ...) + i_{D-1}          (last coordinate fastest)
//   hashed: idx = (i0*1 ^ i1*43857811 ^ i2*83857661 ^ i3*73856093 ^ i4*19349663 ^ i5*834927) % size
//   element = memoryOffset + idx*F + feature
// Corner weights are products of (1-f_d | f_d), multiplied from dimension D-1 down
// to 0 (encoding_hashgrid.cuh:177-206).
//
// Differences to the reference, on purpose: the table may be stored as fp16
// (Cfg::table_t), features of the levels are summed in fp32 in "add" mode, and the
// input gradient carries the (R-1) chain-rule factor when Cfg::ResolutionFactor.

#include <qmlp/kernels/common.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

template <typename T, int D>
struct HashGridParams
{
    const T* __restrict__ parametersForward;
    float* parametersBackward;
    float boundingBoxMin[D];
    float boundingBoxInvSize[D];
};

namespace detail {

template <int D> struct HashPrime;
template <> struct HashPrime<0> { static constexpr unsigned value = 1u; };
template <> struct HashPrime<1> { static constexpr unsigned value = 43857811u; };
template <> struct HashPrime<2> { static constexpr unsigned value = 83857661u; };
template <> struct HashPrime<3> { static constexpr unsigned value = 73856093u; };
template <> struct HashPrime<4> { static constexpr unsigned value = 19349663u; };
template <> struct HashPrime<5> { static constexpr unsigned value = 834927u; };

__device__ __forceinline__ constexpr unsigned hashPrime(int d)
{
    return d == 0 ? 1u : d == 1 ? 43857811u : d == 2 ? 83857661u : d == 3 ? 73856093u
         : d == 4 ? 19349663u : 834927u;
}

__device__ __forceinline__ constexpr unsigned upow(unsigned x, int p)
{
    unsigned r = 1u;
    for (int i = 0; i < p; ++i) r *= x;
    return r;
}

/** Loads F consecutive table entries as floats with the widest aligned vector loads. */
template <int F, typename T>
__device__ __forceinline__ void loadFeatures(const T* __restrict__ p, float (&v)[F])
{
    constexpr int MAXV = 16 / static_cast<int>(sizeof(T));
    constexpr int V = (F % 8 == 0 && MAXV >= 8) ? 8 : (F % 4 == 0 && MAXV >= 4) ? 4 : (F % 2 == 0) ? 2 : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
#pragma unroll
    for (int i = 0; i < F; i += V) {
        if constexpr (V == 1) {
            v[i] = static_cast<float>(p[i]);
        } else {
            const vec_t t = *reinterpret_cast<const vec_t*>(p + i);
#pragma unroll
            for (int j = 0; j < V; ++j) v[i + j] = static_cast<float>(t[j]);
        }
    }
}

} // namespace detail

/**
 * \tparam Cfg generated struct with
 *   static constexpr int Start, Dim, Levels, Features; static constexpr bool Concat, ResolutionFactor;
 *   typedef table_t (float or f16);
 *   static constexpr int resolution[Levels], memoryOffset[Levels];
 *   static constexpr unsigned hashGridSize[Levels]; static constexpr bool hashed[Levels];
 */
template <typename Cfg>
struct EncodingHashGrid
{
    static constexpr int D = Cfg::Dim;
    static constexpr int F = Cfg::Features;
    static constexpr int L = Cfg::Levels;
    static constexpr int NC = 1 << D;
    typedef typename Cfg::table_t table_t;
    typedef HashGridParams<table_t, D> param_t;
    static constexpr int NumOutputs = Cfg::Concat ? L * F : F;

    /** Cell corners, fractional position and the per-dimension index terms of one level. */
    struct LevelSetup
    {
        float f[D];
        unsigned termL[D], termH[D];
    };

    template <typename I>
    __device__ __forceinline__ static void unitPosition(const I& input, const param_t& params, float (&pos)[D])
    {
#pragma clang fp contract(off)
#pragma unroll
        for (int d = 0; d < D; ++d)
            pos[d] = (input[d + Cfg::Start] - params.boundingBoxMin[d]) * params.boundingBoxInvSize[d];
    }

    __device__ __forceinline__ static LevelSetup setupLevel(int l, const float (&pos)[D])
    {
#pragma clang fp contract(off)
        LevelSetup s;
        const int R = Cfg::resolution[l];
        const int rm1 = R - 1;
        const bool hashed = Cfg::hashed[l];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const float p = pos[d] * static_cast<float>(rm1);
            const int ip = static_cast<int>(p);
            const unsigned iL = static_cast<unsigned>(max(0, min(rm1, ip)));
            const unsigned iH = static_cast<unsigned>(max(0, min(rm1, ip + 1)));
            s.f[d] = p - static_cast<float>(iL);
            // uint32 ring arithmetic: the dense index ((i0*R+i1)*R+..) equals sum_d i_d*R^(D-1-d)
            const unsigned mult = hashed ? detail::hashPrime(d)
                                         : detail::upow(static_cast<unsigned>(R), D - 1 - d);
            s.termL[d] = iL * mult;
            s.termH[d] = iH * mult;
        }
        return s;
    }

    /** Offset (in table entries) of feature 0 of corner c (bit d set = upper corner in dim d). */
    __device__ __forceinline__ static unsigned cornerOffset(int l, const LevelSetup& s, int c)
    {
        unsigned idx;
        if (Cfg::hashed[l]) {
            idx = 0u;
#pragma unroll
            for (int d = 0; d < D; ++d) idx ^= ((c >> d) & 1) ? s.termH[d] : s.termL[d];
            idx %= Cfg::hashGridSize[l];
        } else {
            idx = 0u;
#pragma unroll
            for (int d = 0; d < D; ++d) idx += ((c >> d) & 1) ? s.termH[d] : s.termL[d];
        }
        return static_cast<unsigned>(Cfg::memoryOffset[l]) + idx * static_cast<unsigned>(F);
    }

    __device__ __forceinline__ static float cornerWeight(const LevelSetup& s, int c)
    {
        float a = 1.f;
#pragma unroll
        for (int d = D - 1; d >= 0; --d) a = a * (((c >> d) & 1) ? s.f[d] : (1.f - s.f[d]));
        return a;
    }

    /**
     * \param input indexable raw input row (float)
     * \param output indexable output row; ValueType float or half/f16
     */
    template <typename I, typename O>
    __device__ __forceinline__ static void forward(const I& input, O& output, const param_t& params)
    {
        typedef typename O::ValueType O_t;
        float pos[D];
        unitPosition(input, params, pos);
        float sum[F];
#pragma unroll
        for (int i = 0; i < F; ++i) sum[i] = 0.f;
#pragma unroll
        for (int l = 0; l < L; ++l) {
            const LevelSetup s = setupLevel(l, pos);
            float feat[F];
#pragma unroll
            for (int i = 0; i < F; ++i) feat[i] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float w = cornerWeight(s, c);
                float v[F];
                detail::loadFeatures<F>(params.parametersForward + cornerOffset(l, s, c), v);
#pragma unroll
                for (int i = 0; i < F; ++i) feat[i] += w * v[i];
            }
            if constexpr (Cfg::Concat) {
#pragma unroll
                for (int i = 0; i < F; ++i) output[l * F + i] = fcast<O_t>(feat[i]);
            } else {
#pragma unroll
                for (int i = 0; i < F; ++i) sum[i] += feat[i];
            }
        }
        if constexpr (!Cfg::Concat) {
#pragma unroll
            for (int i = 0; i < F; ++i) output[i] = fcast<O_t>(sum[i]);
        }
    }

    /**
     * Adjoint: scatters w * adjFeature into the gradient table with hardware fp32
     * atomics and accumulates the analytic multilinear derivative into adjInput.
     */
    template <bool EvaluateInputGradients, bool EvaluateParameterGradients, typename I, typename O, typename AdjI>
    __device__ __forceinline__ static void adjoint(const I& input, const O& adjOutput, AdjI& adjInput,
                                                   const param_t& params)
    {
        if constexpr (!EvaluateInputGradients && !EvaluateParameterGradients) return;
        float pos[D];
        unitPosition(input, params, pos);
        float adjPos[D];
#pragma unroll
        for (int d = 0; d < D; ++d) adjPos[d] = 0.f;
#pragma unroll
        for (int l = 0; l < L; ++l) {
            const LevelSetup s = setupLevel(l, pos);
            float adjFeat[F];
#pragma unroll
            for (int i = 0; i < F; ++i)
                adjFeat[i] = fcast<float>(adjOutput[(Cfg::Concat ? l * F : 0) + i]);
            float lvl[D];
#pragma unroll
            for (int d = 0; d < D; ++d) lvl[d] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const unsigned off = cornerOffset(l, s, c);
                if constexpr (EvaluateParameterGradients) {
                    const float w = cornerWeight(s, c);
#pragma unroll
                    for (int i = 0; i < F; ++i)
                        unsafeAtomicAdd(params.parametersBackward + (off + i), w * adjFeat[i]);
                }
                if constexpr (EvaluateInputGradients) {
                    float v[F];
                    detail::loadFeatures<F>(params.parametersForward + off, v);
                    float dot = 0.f;
#pragma unroll
                    for (int i = 0; i < F; ++i) dot += adjFeat[i] * v[i];
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        float prod = 1.f;
#pragma unroll
                        for (int e = D - 1; e >= 0; --e)
                            if (e != d) prod *= ((c >> e) & 1) ? s.f[e] : (1.f - s.f[e]);
                        lvl[d] += (((c >> d) & 1) ? prod : -prod) * dot;
                    }
                }
            }
            if constexpr (EvaluateInputGradients) {
                const float scale = Cfg::ResolutionFactor ? static_cast<float>(Cfg::resolution[l] - 1) : 1.f;
#pragma unroll
                for (int d = 0; d < D; ++d) adjPos[d] += scale * lvl[d];
            }
        }
        if constexpr (EvaluateInputGradients) {
#pragma unroll
            for (int d = 0; d < D; ++d)
                adjInput[d + Cfg::Start] += adjPos[d] * params.boundingBoxInvSize[d];
        }
    }

    /** Writes the element offset and weight of every corner (index checks in tests). */
    template <typename I>
    __device__ __forceinline__ static void corners(const I& input, const param_t& params,
                                                   unsigned* __restrict__ idx, float* __restrict__ w)
    {
        float pos[D];
        unitPosition(input, params, pos);
#pragma unroll
        for (int l = 0; l < L; ++l) {
            const LevelSetup s = setupLevel(l, pos);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                idx[l * NC + c] = cornerOffset(l, s, c);
                w[l * NC + c] = cornerWeight(s, c);
            }
        }
    }
};

QUICKMLP_KERNEL_NAMESPACE_END
