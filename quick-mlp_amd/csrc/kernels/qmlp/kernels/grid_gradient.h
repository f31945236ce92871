// Parameter gradients of a grid encoding without a global atomic per contribution: the
// contributions are first written as records into buckets, one bucket per slice of the gradient
// table, and a workgroup per slice then sums its bucket in LDS and adds the slice to the gradient
// tensor once.
//
// Float atomics on device memory complete at about 21e9 requests per second on the whole
// device wherever the data lives, and a hashed level offers nothing to combine (a batch of
// random points touches every entry about once). So the scatter of the fused backward kernel
// (EncodingHashGrid::scatterTile, 4.5 requests per point and level) bounds a train step. Here
// the backward kernel only stores the adjoint of the encoded rows. Then
//   GridGradientRecordsKernel  walks over the points, one per lane, level by level: for every
//       pair of corners that are neighbours in memory it forms a record (the offsets of the two
//       entries within their slice, their weights, the adjoint of the level's features), sorts the
//       records of the workgroup by the slice of the gradient table they belong to (a slice is a
//       run of 8192 or 16 384 floats, whose 64-bit sums take 64 or 128 KiB of LDS) in LDS, reserves
//       room in the buckets of these slices with one atomic per slice and workgroup, and copies the
//       sorted records there in runs: all stores of the records are coalesced. An upper entry that
//       lies in another slice than the lower one is added to the gradient tensor right away. With
//       INPUT_GRADIENTS the kernel also gathers the entries of all corners and adds the grid's
//       share of the gradient with respect to the input (what EncodingHashGrid::adjoint computes,
//       operation by operation): two entries that lie side by side with one load, issued after the
//       bucket atomics of the level and used at its end, while the barriers in between (ldsBarrier)
//       wait for LDS only, so the gathers stay in flight over the staging and the copy of the records
//       (16 levels of a 3-D hash grid, 2^18 points: 203 -> 188 us; without the gathers 117 us). Where the forward
//       pass kept the derivatives of the features with respect to the position (PositionDerivativeLayout,
//       INPUT_GRADIENTS == 2), the share is adjoint x derivative from one or two coalesced loads per level
//       instead (same grid: 126 us);
//   GridGradientSlicesKernel   runs one workgroup per work item (level, slice, part of the
//       bucket): it streams through its records and adds weight * adjoint to the slice in LDS,
//       then adds the slice to the gradient tensor (with atomics only for a coarse level, whose
//       few slices receive all records of the level and are shared out over several work items).
// The sums in LDS are 64-bit fixed point, added with integer atomics: ds_add_f32 completes one
// lane every three cycles on this hardware (0.32 lanes per clock and CU measured, whatever the
// addresses), ds_add_u64 3.5 lanes per clock. The scale is a power of two chosen per launch from the
// largest adjoint of the batch (which the records kernel finds on its way) and the number of
// records, such that no sum can overflow: at least 37 bits remain below the largest possible
// contribution at 2^24 records, and the sums do not depend on the order of the additions. Batches whose
// adjoints are not finite take the float additions, so that NaN and infinity reach the gradients. Weights
// are at most one for points inside the box; the records of points outside of it (extrapolated with weights
// beyond one, or NaN for a NaN coordinate) are added to the gradient tensor by the records kernel itself.
// Two forms that were measured and dropped: a workgroup per slice that tests every point of
// the batch against its slice and recomputes the hits (the work of a hit falls to one lane of
// 64, 890 us for 2^18 points and 16 levels), and the same with the hits queued in LDS first (the
// queued hits gather their point's coordinates and adjoints at random: bound by line requests).
// A bucket has room for 1.25 times its share of the records of a uniform batch; a record that
// finds its bucket full is added to the gradient tensor with atomics by the lane that holds it.
//
// Replaces, for batches that are large enough, the atomicAdd of
// src_cpp/include/qmlp/kernels/encoding_hashgrid.cuh:117-166,345-369 of the reference.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/encoding_hashgrid.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

/** One work item of GridGradientSlicesKernel: the `floats` elements of the gradient table from
 *  element `first` on (slice `slice` of level `level`), part `part` of `parts` of its bucket. */
struct GridGradientSlice
{
    int level;
    unsigned first;
    int floats;
    int slice;
    int part;
    int parts;       // > 1: other work items hold sums for the same slice, all add it with atomics
    int reserved0;
    int reserved1;
};

template <typename Cfg, int SLICE_FLOATS>
struct GridGradientLayout
{
    typedef EncodingHashGrid<Cfg> Grid;
    static constexpr int D = Grid::D;
    static constexpr int F = Grid::F;
    static constexpr int L = Grid::L;
    static constexpr int PAIRS = Grid::NC / 2 > 0 ? Grid::NC / 2 : 1;
    /** A record in 32-bit words: the offsets of the lower and of the upper entry within the slice (16 bits
     *  each), their two weights, F halves of adjoint; one word of padding where that makes it a multiple of
     *  16 bytes (records of 16 or 32 bytes move as whole vector loads and stores). */
    static constexpr int RECORD_WORDS_USED = 3 + (F + 1) / 2;
    static constexpr int RECORD_WORDS = RECORD_WORDS_USED % 4 == 3 ? RECORD_WORDS_USED + 1 : RECORD_WORDS_USED;
    static_assert(SLICE_FLOATS <= 65536, "offsets within a slice are stored in 16 bits");

    /** Records start at multiples of their size from a 16-byte aligned base (LDS or global memory). */
    template <typename Pointer>
    __device__ __forceinline__ static void loadRecord(Pointer src, unsigned (&r)[RECORD_WORDS])
    {
        if constexpr (RECORD_WORDS % 4 == 0) {
#pragma unroll
            for (int v = 0; v < RECORD_WORDS / 4; ++v) {
                const uint4 q = reinterpret_cast<const uint4*>(src)[v];
                r[4 * v] = q.x, r[4 * v + 1] = q.y, r[4 * v + 2] = q.z, r[4 * v + 3] = q.w;
            }
        } else {
#pragma unroll
            for (int v = 0; v < RECORD_WORDS; ++v) r[v] = src[v];
        }
    }
    __device__ __forceinline__ static void storeRecord(unsigned* dst, const unsigned (&r)[RECORD_WORDS])
    {
        if constexpr (RECORD_WORDS % 4 == 0) {
#pragma unroll
            for (int v = 0; v < RECORD_WORDS / 4; ++v)
                reinterpret_cast<uint4*>(dst)[v] = make_uint4(r[4 * v], r[4 * v + 1], r[4 * v + 2], r[4 * v + 3]);
        } else {
#pragma unroll
            for (int v = 0; v < RECORD_WORDS; ++v) dst[v] = r[v];
        }
    }

    __device__ __host__ static constexpr int levelFloats(int l)
    {
        return (l + 1 < L ? Cfg::memoryOffset[l + 1] : Cfg::ParameterCount) - Cfg::memoryOffset[l];
    }
    __device__ __host__ static constexpr int numSlices(int l) { return (levelFloats(l) + SLICE_FLOATS - 1) / SLICE_FLOATS; }
    /** Records a bucket of level l holds for a batch of numel points. */
    __device__ __host__ static constexpr long long capacity(int l, long long numel)
    {
        return ((5 * numel * PAIRS / 4) / numSlices(l) + 2048) & ~3ll;
    }
    /** Index of the first bucket of level l. */
    __device__ __host__ static constexpr int firstBucket(int l)
    {
        int n = 0;
        for (int k = 0; k < l; ++k) n += numSlices(k);
        return n;
    }
    /** Offset in records of the first bucket of level l. */
    __device__ __host__ static constexpr long long levelOffset(int l, long long numel)
    {
        long long n = 0;
        for (int k = 0; k < l; ++k) n += numSlices(k) * capacity(k, numel);
        return n;
    }
};

/**
 * A workgroup barrier that orders the LDS accesses of the workgroup and nothing else. __syncthreads() also waits for
 * every load from and store to global memory that the wavefront has in flight; the records kernel keeps the gathers
 * of a level's table entries in flight across the barriers of that level's sort, and nothing it writes to global
 * memory is read again before the kernel ends.
 */
__device__ __forceinline__ void ldsBarrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <typename Cfg, int ROW_CHANNELS, int CHANNEL_OFFSET, int SLICE_FLOATS, int POINTS>
struct GridGradientRecords
{
    typedef GridGradientLayout<Cfg, SLICE_FLOATS> Layout;
    typedef EncodingHashGrid<Cfg> Grid;
    typedef typename Grid::param_t param_t;
    static constexpr int D = Grid::D;
    static constexpr int F = Grid::F;
    static constexpr int PAIRS = Layout::PAIRS;
    static constexpr int RW = Layout::RECORD_WORDS;
    static constexpr int MAX_SLICES = 512;
    typedef PositionDerivativeLayout<Cfg> DerivativeLayout;
    typedef typename DerivativeLayout::chunk_t DerivativeChunk;

    /** The two table entries of pair c of a point (bit b of c: upper corner in the b-th dimension
     *  other than the pair's own) and the weight of the pair without its own dimension. */
    template <int LEVEL>
    __device__ __forceinline__ static void pairEntries(const typename Grid::LevelSetup& s, int c, unsigned& idxL,
                                                       unsigned& idxH, float& w)
    {
        constexpr bool hashed = Cfg::hashed[LEVEL];
        constexpr int PD = hashed ? 0 : D - 1;   // the dimension whose two corners are neighbours in memory
        unsigned rest = 0u;
        w = 1.f;
        int bit = 0;
#pragma unroll
        for (int d = D - 1; d >= 0; --d) {
            if (d == PD) continue;
            const bool hi = (c >> bit) & 1;
            ++bit;
            const unsigned t = hi ? s.termH[d] : s.termL[d];
            rest = hashed ? (rest ^ t) : (rest + t);
            w = w * (hi ? s.f[d] : (1.f - s.f[d]));
        }
        if (hashed) {
            idxL = (rest ^ s.termL[PD]) % Cfg::hashGridSize[LEVEL];
            idxH = (rest ^ s.termH[PD]) % Cfg::hashGridSize[LEVEL];
        } else {
            idxL = rest + s.termL[PD];
            idxH = rest + s.termH[PD];
        }
    }

    /** Two entries fit one load of 16 bytes: the entries of a pair that lie side by side in the table (all pairs of a
     *  dense level away from its border; in a hashed level those whose lower corner has an even first coordinate)
     *  come with one request instead of two. */
    static constexpr bool PAIR_LOADS = 2 * F * static_cast<int>(sizeof(typename Cfg::table_t)) <= 16;

    /** The corner (bit d: upper in dimension d) of pair c's lower or upper entry. */
    template <int LEVEL>
    __device__ __forceinline__ static constexpr int cornerOfPair(int c, bool upper)
    {
        constexpr int PD = Cfg::hashed[LEVEL] ? 0 : D - 1;
        int corner = upper ? (1 << PD) : 0, bit = 0;
        for (int d = D - 1; d >= 0; --d) {
            if (d == PD) continue;
            corner |= ((c >> bit) & 1) << d;
            ++bit;
        }
        return corner;
    }

    /** The F values from position 'first' on of a wider vector that one load brought in. */
    template <typename Wide>
    __device__ __forceinline__ static void takeHeld(detail::HeldFeatures<F, typename Cfg::table_t>& h, const Wide& w, int first)
    {
        constexpr int V = detail::HeldFeatures<F, typename Cfg::table_t>::V;
#pragma unroll
        for (int i = 0; i < F / V; ++i)
#pragma unroll
            for (int j = 0; j < V; ++j) h.part[i][j] = w[first + i * V + j];
    }

    template <int LEVEL>
    __device__ __forceinline__ static void loadHeld(const typename Grid::LevelSetup& s, const param_t& params,
                                                    detail::HeldFeatures<F, typename Cfg::table_t> (&held)[Grid::NC])
    {
        if constexpr (PAIR_LOADS) {
            loadHeldPairs<LEVEL>(s, params, held);
        } else {
#pragma unroll
            for (int c = 0; c < Grid::NC; ++c) held[c].load(params.parametersForward + Grid::cornerOffset(LEVEL, s, c));
        }
    }

    template <int LEVEL>
    __device__ __forceinline__ static void loadHeldPairs(const typename Grid::LevelSetup& s, const param_t& params,
                                                         detail::HeldFeatures<F, typename Cfg::table_t> (&held)[Grid::NC])
    {
        const typename Cfg::table_t* __restrict__ table = params.parametersForward + Cfg::memoryOffset[LEVEL];
#pragma unroll
        for (int c = 0; c < PAIRS; ++c) {
            unsigned idxL, idxH;
            float w;
            pairEntries<LEVEL>(s, c, idxL, idxH, w);
            loadHeldPair<LEVEL>(c, idxL, idxH, table, held);
        }
    }

    template <int LEVEL>
    __device__ __forceinline__ static void loadHeldPair(int c, unsigned idxL, unsigned idxH, const typename Cfg::table_t* __restrict__ table,
                                                              detail::HeldFeatures<F, typename Cfg::table_t> (&held)[Grid::NC])
    {
        typedef typename Cfg::table_t table_t;
        constexpr int ENTRY_BYTES = F * static_cast<int>(sizeof(table_t));
        // entries lie at multiples of their size: aligned to the largest power of two that divides it
        constexpr int ALIGN = (ENTRY_BYTES & -ENTRY_BYTES) >= 8 ? 8 : (ENTRY_BYTES & -ENTRY_BYTES);
        typedef table_t pair_t __attribute__((ext_vector_type(2 * F), aligned(ALIGN)));
        const int lower = cornerOfPair<LEVEL>(c, false), upper = cornerOfPair<LEVEL>(c, true);   // constants once the loop over c is unrolled
        if (idxH == idxL + 1u) {
            const pair_t both = *reinterpret_cast<const pair_t*>(table + idxL * F);
            takeHeld(held[lower], both, 0);
            takeHeld(held[upper], both, F);
        } else {
            held[lower].load(table + idxL * F);
            held[upper].load(table + idxH * F);
        }
    }

    /** What happens to an upper entry that lies in another slice than its record: the product adds it to the
     *  gradient tensor right away. */
    struct AddToTensor
    {
        float* __restrict__ gradients;
        __device__ __forceinline__ void operator()(unsigned element, float weight, const unsigned (&adjWords)[(F + 1) / 2]) const
        {
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const unsigned short bits = static_cast<unsigned short>(adjWords[i / 2] >> (16 * (i % 2)));
                unsafeAtomicAdd(gradients + element + i, weight * static_cast<float>(__builtin_bit_cast(f16, bits)));
            }
        }
    };

    /**
     * The record of pair c of a point in one level: the offsets of its two entries within the slice of the lower
     * one, their weights and the adjoint words. Returns the slice (= bucket within the level) that files it.
     * \param otherSlice called with (element of feature 0 in the table, weight, adjWords) for an upper entry that
     *    lies in another slice (an entry next to a slice boundary; in a hashed level one pair in thousands): the
     *    record then keeps the lower entry only
     */
    template <int LEVEL, typename OtherSlice>
    __device__ __forceinline__ static int buildRecord(const typename Grid::LevelSetup& s, int c,
                                                      const unsigned (&adjWords)[(F + 1) / 2], unsigned (&rec)[RW],
                                                      const OtherSlice& otherSlice)
    {
        constexpr int PD = Cfg::hashed[LEVEL] ? 0 : D - 1;
        constexpr unsigned base = static_cast<unsigned>(Cfg::memoryOffset[LEVEL]);
        unsigned idxL, idxH;
        float w;
        pairEntries<LEVEL>(s, c, idxL, idxH, w);
        const int bucket = static_cast<int>(idxL * F / SLICE_FLOATS);   // the slice of the lower entry files the record
        const unsigned sliceStart = static_cast<unsigned>(bucket) * SLICE_FLOATS;
        const unsigned eL = idxL * F - sliceStart;
        unsigned eH = idxH * F - sliceStart;                     // wraps if the upper entry lies below the slice
        float wH = w * s.f[PD];
        const float wL = w * (1.f - s.f[PD]);
        if (eH >= static_cast<unsigned>(SLICE_FLOATS)) {
            otherSlice(base + idxH * F, wH, adjWords);
            eH = eL;
            wH = 0.f;
        }
        rec[0] = eL | (eH << 16);
        rec[1] = __builtin_bit_cast(unsigned, wL);
        rec[2] = __builtin_bit_cast(unsigned, wH);
#pragma unroll
        for (int i = 0; i < (F + 1) / 2; ++i) rec[3 + i] = adjWords[i];
#pragma unroll
        for (int v = Layout::RECORD_WORDS_USED; v < RW; ++v) rec[v] = 0u;
        return bucket;
    }

    /** Adds a record to the gradient tensor itself (its bucket was full); grad: element 0 of the record's slice. */
    __device__ __forceinline__ static void addToTensor(const unsigned (&rec)[RW], float* __restrict__ grad)
    {
        const float wL = __builtin_bit_cast(float, rec[1]), wH = __builtin_bit_cast(float, rec[2]);
        const unsigned eL = rec[0] & 0xffffu, eH = rec[0] >> 16;
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const unsigned short bits = static_cast<unsigned short>(rec[3 + i / 2] >> (16 * (i % 2)));
            const float adj = static_cast<float>(__builtin_bit_cast(f16, bits));
            unsafeAtomicAdd(grad + eL + i, wL * adj);
            if (wH != 0.f) unsafeAtomicAdd(grad + eH + i, wH * adj);
        }
    }

    template <int LEVEL, int INPUT_GRADIENTS>
    __device__ __forceinline__ static void runLevel(int p, bool valid, long long numel, const float (&pos)[D],
                                                    const f16* __restrict__ adjEncoded, const param_t& params,
                                                    unsigned* __restrict__ records, int* __restrict__ cursors,
                                                    unsigned* sStage, unsigned short* sBucketOf, int* sHist,
                                                    int* sLocalBase, long long* sGlobalBase, unsigned& maxAdjBits,
                                                    float (&adjPos)[D], const DerivativeChunk* __restrict__ derivatives)
    {
        constexpr bool hashed = Cfg::hashed[LEVEL];
        constexpr int PD = hashed ? 0 : D - 1;
        constexpr unsigned base = static_cast<unsigned>(Cfg::memoryOffset[LEVEL]);
        constexpr int NS = Layout::numSlices(LEVEL);
        static_assert(NS <= MAX_SLICES, "the slice of a record is kept in the histogram arrays");
        const int tid = threadIdx.x;
        for (int b = tid; b < NS; b += POINTS) sHist[b] = 0;
        ldsBarrier();   // also: the staging area of the previous level has been copied out

        // my records of this level, in registers, and their places among the workgroup's records of the same slice
        unsigned rec[PAIRS][RW];
        int bucket[PAIRS], rank[PAIRS];
        const typename Grid::LevelSetup s = Grid::setupLevel(LEVEL, pos);
        detail::HeldFeatures<F, typename Cfg::table_t> held[Grid::NC];
        (void)held;
        if (valid) {
            const f16* adjRow = adjEncoded + static_cast<long long>(p / TILE_POINTS) * (ROW_CHANNELS * TILE_POINTS)
                + (CHANNEL_OFFSET + (Cfg::Concat ? LEVEL * F : 0)) * TILE_POINTS + (p % TILE_POINTS);
            unsigned adjWords[(F + 1) / 2];
#pragma unroll
            for (int i = 0; i < (F + 1) / 2; ++i) adjWords[i] = 0u;
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const unsigned bits = __builtin_bit_cast(unsigned short, adjRow[i * TILE_POINTS]);
                adjWords[i / 2] |= bits << (16 * (i % 2));
                // largest magnitude seen (as fp16 bits without the sign: ordered like the values, NaN above infinity)
                maxAdjBits = max(maxAdjBits, bits & 0x7fffu);
            }
            if constexpr (INPUT_GRADIENTS == 1 && !DEFER_ENTRIES) {
                // the entries of all corners, for this grid's share of dL/dinput (a dense 4-D grid with 8 features
                // holds 64 registers: used at once; held until the end of the level 302 against 275 us)
                loadHeld<LEVEL>(s, params, held);
                positionGradient<LEVEL>(p, s, held, adjEncoded, adjPos);
            }
#pragma unroll
            for (int c = 0; c < PAIRS; ++c) {
                bucket[c] = buildRecord<LEVEL>(s, c, adjWords, rec[c], AddToTensor{params.parametersBackward});
                // (a level of one slice needs no sorting: every lane has fixed places)
                rank[c] = NS == 1 ? tid * PAIRS + c : atomicAdd(sHist + bucket[c], 1);
            }
            // The sums of the slice kernel are fixed point with a scale that counts on weights of at most one, which
            // holds while every fractional position lies in [0, 1]: for every point inside the box. A point outside of
            // it is extrapolated (the fractional position is not clamped) with weights that grow with its distance, a
            // NaN coordinate gives NaN weights: the records of such a point are added to the gradient tensor right
            // here, as records are whose bucket is full, and go to the buckets with weights of zero.
            bool inside = true;
#pragma unroll
            for (int d = 0; d < D; ++d) inside = inside && s.f[d] >= 0.f && s.f[d] <= 1.f;
            if (!inside) {
                // (rare: a loop that recomputes the pairs and reads the adjoints again, so that it costs the points
                // inside the box neither registers nor code)
                float* __restrict__ grad = params.parametersBackward + base;
#pragma unroll 1
                for (int c = 0; c < PAIRS; ++c) {
                    unsigned idxL, idxH;
                    float w;
                    pairEntries<LEVEL>(s, c, idxL, idxH, w);
                    const float wL = w * (1.f - s.f[PD]), wH = w * s.f[PD];
                    // (an upper entry in another slice than the lower one has been added by buildRecord already)
                    const unsigned sliceStart = idxL * F / SLICE_FLOATS * SLICE_FLOATS;
                    const bool upperAdded = idxH * F - sliceStart >= static_cast<unsigned>(SLICE_FLOATS);
#pragma unroll 1
                    for (int i = 0; i < F; ++i) {
                        const float adj = static_cast<float>(adjRow[i * TILE_POINTS]);
                        unsafeAtomicAdd(grad + idxL * F + i, wL * adj);
                        if (!upperAdded) unsafeAtomicAdd(grad + idxH * F + i, wH * adj);
                    }
                }
#pragma unroll
                for (int c = 0; c < PAIRS; ++c) {
                    rec[c][1] = 0u;
                    rec[c][2] = 0u;
                }
            }
        } else {
            // lanes beyond the batch: in a level of one slice they fill their fixed places with records that add nothing
#pragma unroll
            for (int c = 0; c < PAIRS; ++c) {
#pragma unroll
                for (int v = 0; v < RW; ++v) rec[c][v] = 0u;
                bucket[c] = 0;
                rank[c] = tid * PAIRS + c;
            }
        }
        if (NS == 1 && tid == 0) sHist[0] = POINTS * PAIRS;
        ldsBarrier();

        // places of the slices in the staging area, and room in their buckets (one atomic per slice)
        if (tid < 64) {
            int running = 0;
            for (int b0 = 0; b0 < NS; b0 += 64) {
                const int b = b0 + tid;
                const int n = b < NS ? sHist[b] : 0;
                int inclusive = n;
#pragma unroll
                for (int d = 1; d < 64; d *= 2) {
                    const int other = __shfl_up(inclusive, d, 64);
                    if (tid >= d) inclusive += other;
                }
                if (b < NS) {
                    sLocalBase[b] = running + inclusive - n;
                    sGlobalBase[b] = n > 0 ? static_cast<long long>(atomicAdd(cursors + Layout::firstBucket(LEVEL) + b, n)) : 0;
                }
                running += __shfl(inclusive, 63, 64);
            }
            if (tid == 0) sLocalBase[NS] = running;
        }
        ldsBarrier();

        if constexpr (INPUT_GRADIENTS == 1 && DEFER_ENTRIES) {
            // The entries of all corners, for this grid's share of dL/dinput, where they take few registers: loaded
            // here and used at the end of the level, so that the two steps in between hide their latency (the
            // barriers order LDS only). Not earlier: the first wavefront waits for its bucket atomics above, and
            // loads return in the order of their issue.
            if (valid) loadHeld<LEVEL>(s, params, held);
        }
        if (valid || NS == 1) {
#pragma unroll
            for (int c = 0; c < PAIRS; ++c) {
                const int at = sLocalBase[bucket[c]] + rank[c];
                Layout::storeRecord(sStage + at * RW, rec[c]);
                sBucketOf[at] = static_cast<unsigned short>(bucket[c]);
            }
        }
        ldsBarrier();

        // sorted by slice: consecutive lanes copy consecutive records of a bucket
        const int total = sLocalBase[NS];
        const long long capacity = Layout::capacity(LEVEL, numel);
        unsigned* levelRecords = records + Layout::levelOffset(LEVEL, numel) * RW;
        for (int j = tid; j < total; j += POINTS) {
            const int b = sBucketOf[j];
            const long long at = sGlobalBase[b] + (j - sLocalBase[b]);
            unsigned r[RW];
            Layout::loadRecord(sStage + j * RW, r);
            if (at < capacity) {
                Layout::storeRecord(levelRecords + (static_cast<long long>(b) * capacity + at) * RW, r);
            } else {
                addToTensor(r, params.parametersBackward + base + static_cast<unsigned>(b) * SLICE_FLOATS);
            }
        }

        if constexpr (INPUT_GRADIENTS == 1 && DEFER_ENTRIES) {
            if (valid) positionGradient<LEVEL>(p, s, held, adjEncoded, adjPos);
        }
        if constexpr (INPUT_GRADIENTS == 2) {
            if (valid) positionGradientFromDerivatives<LEVEL>(p, derivatives, adjEncoded, adjPos);
        }
    }

    /**
     * This level's share of the gradient with respect to the position from the derivatives of the level's features
     * that the forward pass stored (PositionDerivativeLayout): sum_i adjoint_i * d feature_i / d p_d, read with one
     * or a few coalesced loads instead of a gather of all corners of the cell.
     */
    template <int LEVEL>
    __device__ __forceinline__ static void positionGradientFromDerivatives(int p, const DerivativeChunk* __restrict__ derivatives,
                                                                           const f16* __restrict__ adjEncoded, float (&adjPos)[D])
    {
        const f16* adjRow = adjEncoded + static_cast<long long>(p / TILE_POINTS) * (ROW_CHANNELS * TILE_POINTS)
            + (CHANNEL_OFFSET + (Cfg::Concat ? LEVEL * F : 0)) * TILE_POINTS + (p % TILE_POINTS);
        float values[DerivativeLayout::VALUES];
        DerivativeLayout::load(derivatives + DerivativeLayout::chunkIndex(p / TILE_POINTS, 0, 0, p % TILE_POINTS), LEVEL, values);
        float lvl[D];
#pragma unroll
        for (int d = 0; d < D; ++d) lvl[d] = 0.f;
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const float adj = static_cast<float>(adjRow[i * TILE_POINTS]);
#pragma unroll
            for (int d = 0; d < D; ++d) lvl[d] += adj * values[i * D + d];
        }
        const float scale = Cfg::ResolutionFactor ? static_cast<float>(Cfg::resolution[LEVEL] - 1) : 1.f;
#pragma unroll
        for (int d = 0; d < D; ++d) adjPos[d] += scale * lvl[d];
    }

    /** Registers worth holding across the sort of a level's records: 64 bytes of table entries per lane. */
    static constexpr bool DEFER_ENTRIES = Grid::NC * F * static_cast<int>(sizeof(typename Cfg::table_t)) <= 64;

    /**
     * This level's share of the gradient with respect to the position, operation by operation as
     * EncodingHashGrid::adjoint computes it (same corner order, same products), so both give the same bits.
     */
    template <int LEVEL>
    __device__ __forceinline__ static void positionGradient(int p, const typename Grid::LevelSetup& s,
                                                            const detail::HeldFeatures<F, typename Cfg::table_t> (&held)[Grid::NC],
                                                            const f16* __restrict__ adjEncoded, float (&adjPos)[D])
    {
        const f16* adjRow = adjEncoded + static_cast<long long>(p / TILE_POINTS) * (ROW_CHANNELS * TILE_POINTS)
            + (CHANNEL_OFFSET + (Cfg::Concat ? LEVEL * F : 0)) * TILE_POINTS + (p % TILE_POINTS);
        float adjFeat[F];
#pragma unroll
        for (int i = 0; i < F; ++i) adjFeat[i] = static_cast<float>(adjRow[i * TILE_POINTS]);
        positionGradient<LEVEL>(s, held, adjFeat, adjPos);
    }

    /** The same from the adjoint of the level's features as floats. */
    template <int LEVEL>
    __device__ __forceinline__ static void positionGradient(const typename Grid::LevelSetup& s,
                                                            const detail::HeldFeatures<F, typename Cfg::table_t> (&held)[Grid::NC],
                                                            const float (&adjFeat)[F], float (&adjPos)[D])
    {
        float lvl[D];
#pragma unroll
        for (int d = 0; d < D; ++d) lvl[d] = 0.f;
#pragma unroll
        for (int c = 0; c < Grid::NC; ++c) {
            float v[F];
            held[c].toFloat(v);
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
        const float scale = Cfg::ResolutionFactor ? static_cast<float>(Cfg::resolution[LEVEL] - 1) : 1.f;
#pragma unroll
        for (int d = 0; d < D; ++d) adjPos[d] += scale * lvl[d];
    }

    template <int LEVEL, int INPUT_GRADIENTS>
    __device__ __forceinline__ static void runLevels(int p, bool valid, long long numel, const float (&pos)[D],
                                                     const f16* __restrict__ adjEncoded, const param_t& params,
                                                     unsigned* __restrict__ records, int* __restrict__ cursors,
                                                     unsigned* sStage, unsigned short* sBucketOf, int* sHist,
                                                     int* sLocalBase, long long* sGlobalBase, unsigned& maxAdjBits,
                                                     float (&adjPos)[D], const DerivativeChunk* __restrict__ derivatives)
    {
        if constexpr (LEVEL < Cfg::Levels) {
            runLevel<LEVEL, INPUT_GRADIENTS>(p, valid, numel, pos, adjEncoded, params, records, cursors, sStage, sBucketOf, sHist,
                                             sLocalBase, sGlobalBase, maxAdjBits, adjPos, derivatives);
            runLevels<LEVEL + 1, INPUT_GRADIENTS>(p, valid, numel, pos, adjEncoded, params, records, cursors, sStage, sBucketOf,
                                                  sHist, sLocalBase, sGlobalBase, maxAdjBits, adjPos, derivatives);
        }
    }
};

/**
 * \tparam POINTS points (= lanes) of a workgroup; its records of one level are staged in LDS
 * records: room for levelOffset(Levels, layoutNumel) records; cursors: one int per bucket, then one word that
 * receives the largest magnitude among the adjoints (fp16 bits without the sign); all zeroed by the caller.
 */
template <typename Cfg, int ROW_CHANNELS, int CHANNEL_OFFSET, int SLICE_FLOATS, int POINTS, int INPUT_GRADIENTS>
__global__ void __launch_bounds__(POINTS) GridGradientRecordsKernel(
    int numel,
    int layoutNumel,                          //points the buckets are laid out for (numel rounded up to whole tiles)
    const Tensor2Read<float> inputs,          //shape (numel, Cin)
    const half* __restrict__ adjEncodedH,     //adjoint of the encoded rows: (tiles, ROW_CHANNELS, 64)
    const HashGridParams<typename Cfg::table_t, Cfg::Dim> params,
    unsigned* __restrict__ records, int* __restrict__ cursors,
    Tensor2RW<float> adjInputs,               //INPUT_GRADIENTS: shape (numel, Cin), this grid's share of dL/dinput is added
    const void* __restrict__ derivativesV)    //INPUT_GRADIENTS == 2: the position derivatives of this grid that the forward pass stored
{
    typedef GridGradientRecords<Cfg, ROW_CHANNELS, CHANNEL_OFFSET, SLICE_FLOATS, POINTS> Impl;
    constexpr int D = Cfg::Dim;
    extern __shared__ __align__(16) unsigned char sMemory[];
    unsigned* sStage = reinterpret_cast<unsigned*>(sMemory);                               // POINTS * PAIRS records
    long long* sGlobalBase = reinterpret_cast<long long*>(sStage + POINTS * Impl::PAIRS * Impl::RW);
    int* sHist = reinterpret_cast<int*>(sGlobalBase + Impl::MAX_SLICES);
    int* sLocalBase = sHist + Impl::MAX_SLICES;
    unsigned short* sBucketOf = reinterpret_cast<unsigned short*>(sLocalBase + Impl::MAX_SLICES + 1);
    unsigned maxAdjBits = 0u;
    for (int chunk = blockIdx.x * POINTS; chunk < numel; chunk += gridDim.x * POINTS) {
        const int p = chunk + threadIdx.x;
        const bool valid = p < numel;
        float pos[D];
        {
#pragma clang fp contract(off)
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const float in = valid ? inputs.data_[static_cast<long long>(p) * inputs.strides_[0]
                                                      + static_cast<long long>(d + Cfg::Start) * inputs.strides_[1]] : 0.f;
                pos[d] = (in - params.boundingBoxMin[d]) * params.boundingBoxInvSize[d];
            }
        }
        float adjPos[D];
#pragma unroll
        for (int d = 0; d < D; ++d) adjPos[d] = 0.f;
        Impl::template runLevels<0, INPUT_GRADIENTS>(p, valid, layoutNumel, pos, reinterpret_cast<const f16*>(adjEncodedH), params,
                                                     records, cursors, sStage, sBucketOf, sHist, sLocalBase, sGlobalBase, maxAdjBits,
                                                     adjPos, static_cast<const typename Impl::DerivativeChunk*>(derivativesV));
        if constexpr (INPUT_GRADIENTS != 0) {
            // every point belongs to one lane of one workgroup: a plain read-modify-write
            if (valid) {
#pragma unroll
                for (int d = 0; d < D; ++d)
                    adjInputs.data_[static_cast<long long>(p) * adjInputs.strides_[0]
                                    + static_cast<long long>(d + Cfg::Start) * adjInputs.strides_[1]] += adjPos[d] * params.boundingBoxInvSize[d];
            }
        }
        ldsBarrier();
    }
    // the largest adjoint of the workgroup: one LDS word, then one atomic per workgroup
    if (threadIdx.x == 0) sHist[0] = 0;
    __syncthreads();
    if (maxAdjBits != 0u) atomicMax(sHist, static_cast<int>(maxAdjBits));
    __syncthreads();
    if (threadIdx.x == 0 && sHist[0] != 0)
        atomicMax(cursors + GridGradientLayout<Cfg, SLICE_FLOATS>::firstBucket(Cfg::Levels), sHist[0]);
}

template <typename Cfg, int SLICE_FLOATS, int LEVEL>
struct GridGradientTraceLevels
{
    template <typename Words>
    __device__ __forceinline__ static void run(const float (&pos)[Cfg::Dim], const Words& adjWords, unsigned* idx, float* w)
    {
        if constexpr (LEVEL < Cfg::Levels) {
            typedef GridGradientRecords<Cfg, 16, 0, SLICE_FLOATS, 256> Impl;
            typedef EncodingHashGrid<Cfg> Grid;
            constexpr int NC = Grid::NC;
            const typename Grid::LevelSetup s = Grid::setupLevel(LEVEL, pos);
#pragma unroll
            for (int c = 0; c < Impl::PAIRS; ++c) {
                unsigned rec[Impl::RW];
                unsigned otherElement = 0u;
                float otherWeight = 0.f;
                bool other = false;
                const int bucket = Impl::template buildRecord<LEVEL>(s, c, adjWords, rec,
                    [&](unsigned element, float weight, const Words&) { other = true; otherElement = element; otherWeight = weight; });
                // (the records of a point outside the box are added by the records kernel itself, entry by entry as decoded here)
                const unsigned sliceStart = static_cast<unsigned>(Cfg::memoryOffset[LEVEL]) + static_cast<unsigned>(bucket) * SLICE_FLOATS;
                idx[LEVEL * NC + 2 * c] = sliceStart + (rec[0] & 0xffffu);
                w[LEVEL * NC + 2 * c] = __builtin_bit_cast(float, rec[1]);
                if (NC > 1) {
                    idx[LEVEL * NC + 2 * c + 1] = other ? otherElement : sliceStart + (rec[0] >> 16);
                    w[LEVEL * NC + 2 * c + 1] = other ? otherWeight : __builtin_bit_cast(float, rec[2]);
                }
            }
            GridGradientTraceLevels<Cfg, SLICE_FLOATS, LEVEL + 1>::run(pos, adjWords, idx, w);
        }
    }
};

/**
 * Test aid: for every point (one per lane) and level, the table elements and weights that the records of
 * GridGradientRecords::buildRecord stand for, decoded as the slice kernel decodes them (slice of the bucket +
 * 16-bit offset), and the entries the records kernel adds itself because they lie in another slice.
 * Slots as in CornerTrace: level * 2^Dim + 2 * pair (+ 1 for the upper entry).
 */
template <typename Cfg, int SLICE_FLOATS>
__global__ void __launch_bounds__(256) GridGradientTraceKernel(
    long long numel, const Tensor2Read<float> inputs, unsigned* __restrict__ indices, float* __restrict__ weights,
    const HashGridParams<typename Cfg::table_t, Cfg::Dim> params)
{
    typedef GridGradientRecords<Cfg, 16, 0, SLICE_FLOATS, 256> Impl;
    typedef EncodingHashGrid<Cfg> Grid;
    constexpr int D = Cfg::Dim, F = Cfg::Features, NC = Grid::NC;
    for (long long index = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; index < numel;
         index += static_cast<long long>(blockDim.x) * gridDim.x)
    {
        float pos[D];
        {
#pragma clang fp contract(off)
#pragma unroll
            for (int d = 0; d < D; ++d)
                pos[d] = (inputs.data_[index * inputs.strides_[0] + static_cast<long long>(d + Cfg::Start) * inputs.strides_[1]]
                          - params.boundingBoxMin[d]) * params.boundingBoxInvSize[d];
        }
        unsigned* idx = indices + index * (Cfg::Levels * NC);
        float* w = weights + index * (Cfg::Levels * NC);
        unsigned adjWords[(F + 1) / 2];
#pragma unroll
        for (int i = 0; i < (F + 1) / 2; ++i) adjWords[i] = 0x3c003c00u;   // 1.0 | 1.0
        GridGradientTraceLevels<Cfg, SLICE_FLOATS, 0>::run(pos, adjWords, idx, w);
    }
}

template <typename Cfg, int SLICE_FLOATS>
struct GridGradientSlices
{
    typedef GridGradientLayout<Cfg, SLICE_FLOATS> Layout;
    typedef EncodingHashGrid<Cfg> Grid;
    static constexpr int F = Grid::F;
    static constexpr int RW = Layout::RECORD_WORDS;
    static constexpr int BLOCK = 1024;

    /** v * 2^scaleExponent as a 64-bit integer, rounded towards minus infinity in the low word (|v * 2^scaleExponent| < 2^62). */
    __device__ __forceinline__ static long long toFixed(float v, int scaleExponent)
    {
        const float x = ldexpf(v, scaleExponent - 32);             // in units of 2^32
        const float hi = floorf(x);
        // the low bits of a 24-bit mantissa: exact, in [0, 2^32) (a tiny negative x gives hi = -1 and x - hi = 1 after rounding)
        const float lo = fminf(ldexpf(x - hi, 32), 4294967040.f);
        return (static_cast<long long>(static_cast<int>(hi)) << 32) + static_cast<long long>(static_cast<unsigned>(lo));
    }

    __device__ __forceinline__ static void ldsAddFixed(long long* p, long long v)
    {
        typedef __attribute__((address_space(3))) unsigned long long lds_u64;
        __hip_atomic_fetch_add((lds_u64*)p, static_cast<unsigned long long>(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }

    /** FIXED: 64-bit fixed-point sums (the slice is SLICE_FLOATS long long); else float sums. */
    template <int LEVEL, bool FIXED>
    __device__ __forceinline__ static void sumRecords(long long numel, const unsigned* __restrict__ records,
                                                      const int* __restrict__ cursors, float* __restrict__ gradients,
                                                      const GridGradientSlice item, long long* sFixed, float* sFloat,
                                                      int scaleExponent)
    {
        const int tid = threadIdx.x;
        const long long capacity = Layout::capacity(LEVEL, numel);
        const long long filled = min(static_cast<long long>(cursors[Layout::firstBucket(LEVEL) + item.slice]), capacity);
        const long long begin = filled * item.part / item.parts, end = filled * (item.part + 1) / item.parts;
        const unsigned* bucket = records + (Layout::levelOffset(LEVEL, numel) + static_cast<long long>(item.slice) * capacity) * RW;
        constexpr int UNROLL = 4;
        for (long long j0 = begin + tid; j0 < end; j0 += UNROLL * BLOCK) {
            unsigned rec[UNROLL][RW];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const long long j = j0 + u * BLOCK;
                if (j < end) {
                    Layout::loadRecord(bucket + j * RW, rec[u]);
                } else {
#pragma unroll
                    for (int v = 0; v < RW; ++v) rec[u][v] = 0u;
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (j0 + u * BLOCK >= end) continue;
                const unsigned eL = rec[u][0] & 0xffffu, eH = rec[u][0] >> 16;   // both inside this slice
                const float wL = __builtin_bit_cast(float, rec[u][1]), wH = __builtin_bit_cast(float, rec[u][2]);
#pragma unroll
                for (int step = 0; step < F; ++step) {
                    // Neighbouring lanes take the features in rotated order: an entry starts at a multiple of
                    // 8 * F bytes, so lanes that all add feature `step` meet on a few LDS banks (measured on a
                    // dense grid with 8 features: conflicts 90 % of the LDS cycles of this kernel).
                    const int i = (F & (F - 1)) == 0 ? ((step + tid) & (F - 1)) : ((step + tid % F) % F);
                    unsigned word = rec[u][3];
#pragma unroll
                    for (int w = 1; w < (F + 1) / 2; ++w) word = (i >> 1) == w ? rec[u][3 + w] : word;
                    const unsigned short bits = static_cast<unsigned short>(word >> (16 * (i & 1)));
                    const float adj = static_cast<float>(__builtin_bit_cast(f16, bits));
                    if constexpr (FIXED) {
                        ldsAddFixed(sFixed + eL + i, toFixed(wL * adj, scaleExponent));
                        ldsAddFixed(sFixed + eH + i, toFixed(wH * adj, scaleExponent));
                    } else {
                        Grid::ldsAdd(sFloat + eL + i, wL * adj);
                        Grid::ldsAdd(sFloat + eH + i, wH * adj);
                    }
                }
            }
        }
    }

    template <int LEVEL>
    __device__ __forceinline__ static void runLevel(long long numel, const unsigned* __restrict__ records,
                                                    const int* __restrict__ cursors, float* __restrict__ gradients,
                                                    const GridGradientSlice item, long long* sSlice)
    {
        const int tid = threadIdx.x;
        for (int i = tid; i < item.floats; i += BLOCK) sSlice[i] = 0;
        __syncthreads();
        // |adjoint| < 2^maxExponent; a sum has at most 2 * PAIRS * numel terms, each at most that large (weights <= 1)
        const unsigned maxBits = static_cast<unsigned>(cursors[Layout::firstBucket(Cfg::Levels)]);
        if (maxBits == 0u) return;   // all adjoints are zero: nothing to add
        const bool finite = maxBits < 0x7c00u;
        const int maxExponent = static_cast<int>(maxBits >> 10) - 14;          // fp16: value < 2^(biased exponent - 14), subnormals included
        const int termsLog2 = 64 - __builtin_clzll(static_cast<unsigned long long>(2 * Layout::PAIRS) * static_cast<unsigned long long>(numel));
        const int scaleExponent = 61 - maxExponent - termsLog2;
        float* sFloat = reinterpret_cast<float*>(sSlice);
        if (finite) sumRecords<LEVEL, true>(numel, records, cursors, gradients, item, sSlice, sFloat, scaleExponent);
        else sumRecords<LEVEL, false>(numel, records, cursors, gradients, item, sSlice, sFloat, 0);
        __syncthreads();
        // Added to the gradient tensor: with atomics (16 neighbouring floats per request) where other work
        // items hold sums for the same slice (parts > 1), else this workgroup is the only writer of its
        // slice in this launch (contributions to entries of other slices were added by the records kernel).
        float* __restrict__ grad = gradients + item.first;
        for (int i = tid; i < item.floats; i += BLOCK) {
            float v;
            if (finite) {
                const long long fixed = sSlice[i];
                v = static_cast<float>(ldexp(static_cast<double>(fixed), -scaleExponent));
            } else {
                v = sFloat[i];
            }
            if (v != 0.f) {
                if (item.parts > 1) unsafeAtomicAdd(grad + i, v);
                else grad[i] += v;
            }
        }
    }

    template <int LEVEL>
    __device__ __forceinline__ static void dispatch(long long numel, const unsigned* __restrict__ records,
                                                    const int* __restrict__ cursors, float* __restrict__ gradients,
                                                    const GridGradientSlice item, long long* sSlice)
    {
        if constexpr (LEVEL < Cfg::Levels) {
            if (item.level == LEVEL) runLevel<LEVEL>(numel, records, cursors, gradients, item, sSlice);
            else dispatch<LEVEL + 1>(numel, records, cursors, gradients, item, sSlice);
        }
    }
};

/** One workgroup of 1024 lanes per work item; `items` is indexed by the workgroup; SLICE_FLOATS * 8 bytes of dynamic LDS. */
template <typename Cfg, int SLICE_FLOATS>
__global__ void __launch_bounds__(1024) GridGradientSlicesKernel(
    int numel, const unsigned* __restrict__ records, const int* __restrict__ cursors, float* __restrict__ gradients,
    const GridGradientSlice* __restrict__ items)
{
    extern __shared__ __align__(16) unsigned char sMemory[];
    GridGradientSlices<Cfg, SLICE_FLOATS>::template dispatch<0>(numel, records, cursors, gradients, items[blockIdx.x],
                                                                reinterpret_cast<long long*>(sMemory));
}

QUICKMLP_KERNEL_NAMESPACE_END
