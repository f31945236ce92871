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
#include <qmlp/kernels/arrays.h>

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

/** The F values of a table entry as they are loaded (the widest aligned vectors), converted to float only when
 *  asked for: nothing touches the loaded registers in between, so the loads may stay in flight. */
template <int F, typename T>
struct HeldFeatures
{
    static constexpr int MAXV = 16 / static_cast<int>(sizeof(T));
    static constexpr int V = (F % 8 == 0 && MAXV >= 8) ? 8 : (F % 4 == 0 && MAXV >= 4) ? 4 : (F % 2 == 0) ? 2 : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    vec_t part[F / V];
    __device__ __forceinline__ void load(const T* __restrict__ p)
    {
#pragma unroll
        for (int i = 0; i < F / V; ++i) part[i] = *reinterpret_cast<const vec_t*>(p + i * V);
    }
    __device__ __forceinline__ void toFloat(float (&v)[F]) const
    {
#pragma unroll
        for (int i = 0; i < F / V; ++i)
#pragma unroll
            for (int j = 0; j < V; ++j) v[i * V + j] = static_cast<float>(part[i][j]);
    }
};

/** Loads two consecutive table entries (2*F values) with one wide load; the address is
 *  only guaranteed to be aligned to one entry. */
template <int F, typename T>
__device__ __forceinline__ void loadPair(const T* __restrict__ p, float (&a)[F], float (&b)[F])
{
    constexpr int ENTRY_BYTES = F * static_cast<int>(sizeof(T));
    // the largest power of two that divides the size of an entry (12-byte entries: 4, 6-byte entries: 2)
    constexpr int ALIGN = (ENTRY_BYTES & -ENTRY_BYTES) >= 16 ? 16 : (ENTRY_BYTES & -ENTRY_BYTES);
    typedef T pair_t __attribute__((ext_vector_type(2 * F), aligned(ALIGN)));
    const pair_t t = *reinterpret_cast<const pair_t*>(p);
#pragma unroll
    for (int i = 0; i < F; ++i) {
        a[i] = static_cast<float>(t[i]);
        b[i] = static_cast<float>(t[F + i]);
    }
}

__device__ __forceinline__ constexpr bool isPow2(unsigned v) { return v != 0u && (v & (v - 1u)) == 0u; }

} // namespace detail

/** gatherLevel / scatterTile without a record of what they touch (every kernel of the product). */
struct NoCornerTrace
{
    static constexpr bool Enabled = false;
};

/**
 * Test aid: gatherLevel and scatterTile write, for every table entry whose value they use (or add
 * to), its element offset (of feature 0) and the weight it is used with, instead of leaving no
 * trace. The arrays hold Levels * 2^Dim slots per point; slot = level * 2^Dim + corner in the
 * order the code visits them.
 */
struct CornerTrace
{
    static constexpr bool Enabled = true;
    unsigned* __restrict__ elements;   // slots of the point (gather) or of the whole batch (scatter)
    float* __restrict__ weights;
    __device__ __forceinline__ void record(long long slot, unsigned element, float weight) const
    {
        elements[slot] = element;
        weights[slot] = weight;
    }
};

/**
 * Where a training pass keeps, per point and level, the derivatives of the interpolated features with respect to
 * the position within the level (in cells: without the factor resolution - 1): d feature_i / d p_d at value
 * i * Dim + d, in the precision of the table (half values are clamped to the finite range), padded with zeros to whole
 * chunks of 16 bytes. Per tile of 64 points the chunks lie level by level, chunk by chunk, 64 points side by side:
 * chunk k of level l of point j of tile t is chunk ((t * Levels + l) * CHUNKS + k) * 64 + j of the region. A lane
 * writes and reads whole chunks, neighbouring lanes neighbouring chunks.
 * With these the input gradients of the adjoint pass need no second gather of the table (2^Dim entries per point
 * and level): they are sum_i adjoint_i * derivative_(i, d), read in one or a few coalesced loads.
 */
template <typename Cfg>
struct PositionDerivativeLayout
{
    typedef typename Cfg::table_t value_t;
    static constexpr int VALUES = Cfg::Dim * Cfg::Features;
    static constexpr int PER_CHUNK = 16 / static_cast<int>(sizeof(value_t));
    static constexpr int CHUNKS = (VALUES + PER_CHUNK - 1) / PER_CHUNK;
    static constexpr int BYTES_PER_POINT = Cfg::Levels * CHUNKS * 16;
    typedef value_t chunk_t __attribute__((ext_vector_type(PER_CHUNK)));

    __device__ __forceinline__ static long long chunkIndex(long long tile, int level, int chunk, int lane)
    {
        return ((tile * Cfg::Levels + level) * CHUNKS + chunk) * TILE_POINTS + lane;
    }

    __device__ __forceinline__ static value_t narrow(float v)
    {
        if constexpr (sizeof(value_t) == 2) return static_cast<value_t>(fminf(fmaxf(v, -65504.f), 65504.f));
        else return v;
    }

    /** The chunks of one level of one point from its VALUES derivatives. */
    __device__ __forceinline__ static void store(chunk_t* __restrict__ level0, int level, const float (&values)[VALUES])
    {
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            chunk_t c;
#pragma unroll
            for (int j = 0; j < PER_CHUNK; ++j)
                c[j] = k * PER_CHUNK + j < VALUES ? narrow(values[k * PER_CHUNK + j < VALUES ? k * PER_CHUNK + j : 0]) : static_cast<value_t>(0);
            level0[(level * CHUNKS + k) * TILE_POINTS] = c;
        }
    }

    __device__ __forceinline__ static void load(const chunk_t* __restrict__ level0, int level, float (&values)[VALUES])
    {
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            const chunk_t c = level0[(level * CHUNKS + k) * TILE_POINTS];
#pragma unroll
            for (int j = 0; j < PER_CHUNK; ++j)
                if (k * PER_CHUNK + j < VALUES) values[k * PER_CHUNK + j] = static_cast<float>(c[j]);
        }
    }
};

/** forwardBatch without derivatives with respect to the position (inference; training passes that need none). */
struct NoPositionDerivatives
{
    static constexpr bool Enabled = false;
};

/** forwardBatch stores the derivatives with respect to the position (PositionDerivativeLayout). */
template <typename Cfg>
struct StorePositionDerivatives
{
    static constexpr bool Enabled = true;
    typedef PositionDerivativeLayout<Cfg> Layout;
    typename Layout::chunk_t* __restrict__ first;   // chunk 0 of level 0 of this lane's point of the lane's first tile
    int tiles;                                      // the lane's tiles q = 0 .. tiles-1 lie inside the batch
    __device__ __forceinline__ void store(int q, int level, const float (&values)[Layout::VALUES]) const
    {
        if (q < tiles) Layout::store(first + static_cast<long long>(q) * (Cfg::Levels * Layout::CHUNKS * TILE_POINTS), level, values);
    }
};

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
     * Interpolated features of one level at one point. The 2^D corners are fetched as
     * 2^(D-1) pairs: per lane-load the memory pipeline handles one address regardless of the
     * width, so one wider load per pair of neighbouring entries halves the number of loads.
     *  - dense level: neighbours along the last (fastest) coordinate are adjacent entries;
     *  - hashed level with a power-of-two table: the multiplier of coordinate 0 is 1, so its
     *    two corners are entries idx and idx^1 of one aligned pair whenever the lower
     *    coordinate is even (or clamped); only otherwise a second, lane-masked load is needed.
     * Values and weights are the same as in the corner-by-corner evaluation, only the order
     * of the fp32 additions differs.
     */
    template <typename Trace = NoCornerTrace>
    __device__ __forceinline__ static void gatherLevel(int l, const float (&pos)[D],
                                                       const table_t* __restrict__ table, float (&feat)[F],
                                                       const Trace& trace = Trace{})
    {
        float none[F * D];
        gatherLevelImpl<false>(l, pos, table, feat, none, trace);
    }

    /**
     * \tparam DERIVATIVES also computes dfeat[i * D + d] = d feat[i] / d p_d, p the position in cells of the level:
     *    sum over the corners of +-(product of the weights of the other dimensions) * value, from the values that
     *    the interpolation has loaded anyway
     */
    template <bool DERIVATIVES, typename Trace = NoCornerTrace>
    __device__ __forceinline__ static void gatherLevelImpl(int l, const float (&pos)[D],
                                                           const table_t* __restrict__ table, float (&feat)[F],
                                                           float (&dfeat)[F * D], const Trace& trace = Trace{})
    {
        // no contraction into fused multiply-adds: the kernels of different shapes (tiles per
        // wave) would contract differently, and the same point has to give the same bits
        // whatever the batch size
#pragma clang fp contract(off)
        const LevelSetup s = setupLevel(l, pos);
        const int R = Cfg::resolution[l];
        const bool hashed = Cfg::hashed[l];
        const unsigned base = static_cast<unsigned>(Cfg::memoryOffset[l]);
#pragma unroll
        for (int i = 0; i < F; ++i) feat[i] = 0.f;
        if constexpr (DERIVATIVES) {
#pragma unroll
            for (int i = 0; i < F * D; ++i) dfeat[i] = 0.f;
        }

        if (!hashed && R >= 2) {
            // pairs along dimension D-1: entries (zb, zb+1) with zb = min(iL, R-2)
            constexpr int PD = D - 1;
            const unsigned zL = s.termL[PD], zH = s.termH[PD];   // multiplier of the last dim is 1
            const unsigned zb = min(zL, static_cast<unsigned>(R - 2));
            const bool lSecond = zL != zb, hSecond = zH != zb;
            const float wzL = 1.f - s.f[PD], wzH = s.f[PD];
#pragma unroll
            for (int c = 0; c < NC / 2; ++c) {
                unsigned idx = zb;
                float w = 1.f;
#pragma unroll
                for (int d = PD - 1; d >= 0; --d) {
                    const bool hi = (c >> d) & 1;
                    idx += hi ? s.termH[d] : s.termL[d];
                    w = w * (hi ? s.f[d] : (1.f - s.f[d]));
                }
                float e0[F], e1[F];
                const unsigned pairElement = base + idx * static_cast<unsigned>(F);   // e0 = this entry, e1 = the next
                detail::loadPair<F>(table + pairElement, e0, e1);
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    const float vL = lSecond ? e1[i] : e0[i];
                    const float vH = hSecond ? e1[i] : e0[i];
                    const float along = wzL * vL + wzH * vH;
                    feat[i] += w * along;
                    if constexpr (DERIVATIVES) {
                        dfeat[i * D + PD] += w * (vH - vL);
#pragma unroll
                        for (int d = 0; d < PD; ++d) {
                            float others = 1.f;
#pragma unroll
                            for (int e = PD - 1; e >= 0; --e)
                                if (e != d) others = others * (((c >> e) & 1) ? s.f[e] : (1.f - s.f[e]));
                            dfeat[i * D + d] += (((c >> d) & 1) ? others : -others) * along;
                        }
                    }
                }
                if constexpr (Trace::Enabled) {
                    trace.record(l * NC + 2 * c, pairElement + (lSecond ? F : 0), w * wzL);
                    trace.record(l * NC + 2 * c + 1, pairElement + (hSecond ? F : 0), w * wzH);
                }
            }
        } else if (hashed && detail::isPow2(Cfg::hashGridSize[l]) && Cfg::hashGridSize[l] >= 2u) {
            const unsigned mask = Cfg::hashGridSize[l] - 1u;
            const float wxL = 1.f - s.f[0], wxH = s.f[0];
#pragma unroll
            for (int c = 0; c < NC / 2; ++c) {
                unsigned rest = 0u;
                float w = 1.f;
#pragma unroll
                for (int d = D - 1; d >= 1; --d) {
                    const bool hi = (c >> (d - 1)) & 1;
                    rest ^= hi ? s.termH[d] : s.termL[d];
                    w = w * (hi ? s.f[d] : (1.f - s.f[d]));
                }
                const unsigned idxL = (s.termL[0] ^ rest) & mask;
                const unsigned idxH = (s.termH[0] ^ rest) & mask;
                float e0[F], e1[F];
                const unsigned pairElement = base + (idxL & ~1u) * static_cast<unsigned>(F);   // e0 = this entry, e1 = the next
                detail::loadPair<F>(table + pairElement, e0, e1);
                float vH[F];
                const bool samePair = ((idxL ^ idxH) & ~1u) == 0u;
                const unsigned upperElement = base + idxH * static_cast<unsigned>(F);
                if constexpr (Trace::Enabled) {
                    trace.record(l * NC + 2 * c, pairElement + ((idxL & 1u) ? F : 0), w * wxL);
                    trace.record(l * NC + 2 * c + 1, samePair ? pairElement + ((idxH & 1u) ? F : 0) : upperElement, w * wxH);
                }
                if (!samePair) {
                    detail::loadFeatures<F>(table + upperElement, vH);
                } else {
#pragma unroll
                    for (int i = 0; i < F; ++i) vH[i] = (idxH & 1u) ? e1[i] : e0[i];
                }
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    const float vL = (idxL & 1u) ? e1[i] : e0[i];
                    const float along = wxL * vL + wxH * vH[i];
                    feat[i] += w * along;
                    if constexpr (DERIVATIVES) {
                        dfeat[i * D] += w * (vH[i] - vL);
#pragma unroll
                        for (int d = 1; d < D; ++d) {
                            float others = 1.f;
#pragma unroll
                            for (int e = D - 1; e >= 1; --e)
                                if (e != d) others = others * (((c >> (e - 1)) & 1) ? s.f[e] : (1.f - s.f[e]));
                            dfeat[i * D + d] += (((c >> (d - 1)) & 1) ? others : -others) * along;
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float w = cornerWeight(s, c);
                float v[F];
                const unsigned element = cornerOffset(l, s, c);
                detail::loadFeatures<F>(table + element, v);
#pragma unroll
                for (int i = 0; i < F; ++i) feat[i] += w * v[i];
                if constexpr (Trace::Enabled) trace.record(l * NC + c, element, w);
                if constexpr (DERIVATIVES) {
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        float others = 1.f;
#pragma unroll
                        for (int e = D - 1; e >= 0; --e)
                            if (e != d) others = others * (((c >> e) & 1) ? s.f[e] : (1.f - s.f[e]));
#pragma unroll
                        for (int i = 0; i < F; ++i) dfeat[i * D + d] += (((c >> d) & 1) ? others : -others) * v[i];
                    }
                }
            }
        }
    }

    /**
     * Level-major evaluation of PPL points of one lane: all points finish level l before
     * any starts level l+1, so that the workgroups of the device sweep through the level
     * tables together and a level's table stays in L2 while it is in use.
     */
    template <int PPL, typename I, typename Os, typename Derivatives = NoPositionDerivatives>
    __device__ __forceinline__ static void forwardBatch(const I (&inputs)[PPL], Os& outputs, const param_t& params,
                                                        const Derivatives& derivatives = Derivatives{})
    {
        typedef typename RowsValueType<Os>::Type O_t;
        float pos[PPL][D];
#pragma unroll
        for (int q = 0; q < PPL; ++q) unitPosition(inputs[q], params, pos[q]);
        float sum[PPL][F];
#pragma unroll
        for (int q = 0; q < PPL; ++q)
#pragma unroll
            for (int i = 0; i < F; ++i) sum[q][i] = 0.f;
#pragma unroll
        for (int l = 0; l < L; ++l) {
            float feat[PPL][F];
#pragma unroll
            for (int q = 0; q < PPL; ++q) {
                if constexpr (Derivatives::Enabled) {
                    float dfeat[F * D];
                    gatherLevelImpl<true>(l, pos[q], params.parametersForward, feat[q], dfeat);
                    derivatives.store(q, l, dfeat);
                } else {
                    gatherLevel(l, pos[q], params.parametersForward, feat[q]);
                }
            }
#pragma unroll
            for (int q = 0; q < PPL; ++q) {
                if constexpr (Cfg::Concat && F % 2 == 0) {
#pragma unroll
                    for (int i = 0; i < F; i += 2)
                        storePair(outputs, q, l * F + i, fcast<O_t>(feat[q][i]), fcast<O_t>(feat[q][i + 1]));
                } else if constexpr (Cfg::Concat) {
#pragma unroll
                    for (int i = 0; i < F; ++i) outputs[q][l * F + i] = fcast<O_t>(feat[q][i]);
                } else {
#pragma unroll
                    for (int i = 0; i < F; ++i) sum[q][i] += feat[q][i];
                }
            }
        }
        if constexpr (!Cfg::Concat) {
#pragma unroll
            for (int q = 0; q < PPL; ++q)
#pragma unroll
                for (int i = 0; i < F; ++i) outputs[q][i] = fcast<O_t>(sum[q][i]);
        }
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
            float feat[F];
            gatherLevel(l, pos, params.parametersForward, feat);
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

    /** Table elements of the first LEVELS levels. */
    template <int LEVELS>
    static constexpr int leadingElements()
    {
        if constexpr (LEVELS <= 0) return 0;
        else if constexpr (LEVELS < L) return Cfg::memoryOffset[LEVELS] - Cfg::memoryOffset[0];
        else return Cfg::ParameterCount - Cfg::memoryOffset[0];
    }

    /** Float addition in LDS (a native LDS instruction; p must point into LDS). */
    __device__ __forceinline__ static void ldsAdd(float* p, float v)
    {
        typedef __attribute__((address_space(3))) float lds_float;
        __hip_atomic_fetch_add((lds_float*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }

    /** Adds the gradients a workgroup has summed in LDS to the gradient tensor (after a barrier). */
    template <int LEVELS>
    __device__ __forceinline__ static void flushLdsGradients(const float* ldsGradients, const param_t& params,
                                                             int thread, int numThreads)
    {
        float* __restrict__ grad = params.parametersBackward + Cfg::memoryOffset[0];
        for (int e = thread; e < leadingElements<LEVELS>(); e += numThreads) {
            const float v = ldsGradients[e];
            if (v != 0.f) unsafeAtomicAdd(grad + e, v);
        }
    }

    /** True if the gradient scatter of a whole tile (scatterTile) is available. */
    static constexpr bool HasTileScatter = detail::isPow2(static_cast<unsigned>(F)) && 2 * F <= WAVE_SIZE;

    /**
     * Parameter gradients of the 64 points of one wavefront tile. The atomic units handle
     * one request per aligned 64-byte block that neighbouring lanes of an instruction
     * address, and their rate is bound by requests (about 21e9 per second on the whole
     * device, wherever the data lives), not by lanes. Therefore 2*F neighbouring lanes share
     * one point and add the F features of two corners that are neighbours in memory; the
     * wavefront covers its 64 points in 2*F rounds of 64/(2F) points. Every lane recomputes the level setup of its point; the
     * arithmetic is free next to the atomics.
     *
     * \tparam LDS_LEVELS the gradients of this many leading levels are first summed in LDS
     *    (ldsGradients, leadingElements<LDS_LEVELS>() floats, zeroed by the workgroup) and reach
     *    global memory once per workgroup through flushLdsGradients: a coarse level receives
     *    many points per cell, so this saves its share of the atomic requests
     * \param index0 index of the first point of the tile
     * \param adjOutput callable (point of the tile 0..63, output channel of this encoding) ->
     *    adjoint of that output as float
     */
    template <int LDS_LEVELS = 0, typename AdjFn, typename Trace = NoCornerTrace>
    __device__ __forceinline__ static void scatterTile(int lane, long long index0, long long numel,
                                                       const Tensor2Read<float>& inputs, const AdjFn& adjOutput,
                                                       const param_t& params, float* ldsGradients = nullptr,
                                                       const Trace& trace = Trace{})
    {
        constexpr int G = 2 * F;            // lanes per point
        constexpr int PPR = WAVE_SIZE / G;  // points per round
        const int sub = lane % G;
        const int k = sub / F;              // position within the pair of entries
        const int i = sub % F;              // feature
        float* __restrict__ grad = params.parametersBackward;
#pragma unroll 1
        for (int round = 0; round < G; ++round) {
            const int pt = round * PPR + lane / G;
            const long long index = index0 + pt;
            if (index >= numel) continue;
            float in[D];
#pragma unroll
            for (int d = 0; d < D; ++d)
                in[d] = inputs.data_[index * inputs.strides_[0]
                                     + static_cast<long long>(d + Cfg::Start) * inputs.strides_[1]];
            float pos[D];
            {
#pragma clang fp contract(off)
#pragma unroll
                for (int d = 0; d < D; ++d) pos[d] = (in[d] - params.boundingBoxMin[d]) * params.boundingBoxInvSize[d];
            }
#pragma unroll
            for (int l = 0; l < L; ++l) {
                const LevelSetup s = setupLevel(l, pos);
                const bool hashed = Cfg::hashed[l];
                const unsigned base = static_cast<unsigned>(Cfg::memoryOffset[l]);
                const float adj = adjOutput(pt, (Cfg::Concat ? l * F : 0) + i);
                // The lanes k = 0 | 1 of a group take the lower | upper corner along the dimension whose
                // neighbours are close in memory: the last one in a dense level (adjacent entries), the
                // first one in a hashed level (multiplier 1: the same 64-byte block 7 times out of 8).
                const int PD = hashed ? 0 : D - 1;
                const float wk = k ? s.f[PD] : 1.f - s.f[PD];
                const unsigned tk = k ? s.termH[PD] : s.termL[PD];
#pragma unroll
                for (int c = 0; c < NC / 2; ++c) {
                    unsigned idx = tk;
                    float w = 1.f;
                    int bit = 0;
#pragma unroll
                    for (int d = D - 1; d >= 0; --d) {
                        if (d == PD) continue;
                        const bool hi = (c >> bit) & 1;
                        ++bit;
                        const unsigned t = hi ? s.termH[d] : s.termL[d];
                        idx = hashed ? (idx ^ t) : (idx + t);
                        w = w * (hi ? s.f[d] : (1.f - s.f[d]));
                    }
                    if (hashed) idx %= Cfg::hashGridSize[l];
                    const unsigned element = idx * static_cast<unsigned>(F) + static_cast<unsigned>(i);
                    if constexpr (Trace::Enabled) {
                        // where this lane would add, instead of adding: one slot per corner, from its feature-0 lane
                        if (i == 0) trace.record((index * L + l) * NC + 2 * c + k, base + element, w * wk);
                    } else
                    if (l < LDS_LEVELS)
                        ldsAdd(ldsGradients + (base - static_cast<unsigned>(Cfg::memoryOffset[0]) + element), (w * wk) * adj);
                    else
                        unsafeAtomicAdd(grad + (base + element), (w * wk) * adj);
                }
            }
        }
    }

    /** Test aid: what the gathers of the fused forward kernels (gatherLevel) read for this point:
     *  element offset and weight per corner, slots as in CornerTrace. */
    template <typename I>
    __device__ __forceinline__ static void traceGather(const I& input, const param_t& params,
                                                       unsigned* __restrict__ idx, float* __restrict__ w)
    {
        float pos[D];
        unitPosition(input, params, pos);
        const CornerTrace trace{idx, w};
#pragma unroll
        for (int l = 0; l < L; ++l) {
            float feat[F];
            gatherLevel(l, pos, params.parametersForward, feat, trace);
            // the values are part of the trace kernel's result so that the loads stay in the program
            if (feat[0] == 12345.678f) w[l * NC] = 0.f;
        }
    }

    /** Test aid: where the gradient scatter of the fused backward kernel (scatterTile) adds for the
     *  64 points from index0 on (called by a whole wavefront); slots of the whole batch. */
    __device__ __forceinline__ static void traceScatter(int lane, long long index0, long long numel,
                                                        const Tensor2Read<float>& inputs, const param_t& params,
                                                        unsigned* __restrict__ idx, float* __restrict__ w)
    {
        scatterTile<0>(lane, index0, numel, inputs, [](int, int) { return 1.f; }, params, nullptr, CornerTrace{idx, w});
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
