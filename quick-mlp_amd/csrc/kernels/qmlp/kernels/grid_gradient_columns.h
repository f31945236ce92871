// Parameter gradients of a dense single-level grid for a batch that is sorted by grid slab (point_order.h):
// no records at all. The nodes of the grid are shared out by the two sorted coordinates: owner (o0, o1) holds
// the nodes whose first two indices lie in [o0 * CPS, (o0 + 1) * CPS) x [o1 * CPS, (o1 + 1) * CPS) (CPS: cells
// per slab and coordinate) and every index of the other coordinates -- a "column" of the table whose sums fit
// the LDS (a 4-D grid of 32 nodes per coordinate with 8 features, CPS = 1: 32 x 32 x 8 sums of 8 bytes = 64 KiB).
// A point of slab (a0, a1) touches nodes of the owners (a0 | a0 + 1, a1 | a1 + 1) only, so the workgroup of
// an owner walks the points of the up to four slabs (o0 - 1 | o0, o1 - 1 | o1) -- two runs of the sorted batch --
// and adds, of every point, the corners that it owns: 64-bit fixed-point sums in LDS as in the slice kernel
// (grid_gradient.h), added to the gradient tensor once at the end (atomics of 16 neighbouring floats per request,
// 0.5 M requests for the grid above). Every point is read by four workgroups (32 bytes from the L2 each time); in
// return the 2^(D-1) records of 16 + 2 F bytes per point are neither written nor read, nor sorted into buckets.
//   GridGradientColumnsPlan    one workgroup: slab totals of the sort -> slab starts; per owner the number of
//                              points it visits and from it the work items (an owner whose slabs hold more than
//                              PART_POINTS points is split over several workgroups, which then add their sums
//                              with atomics: a batch that crowds into few slabs still uses the whole device);
//   GridGradientColumnsKernel  one workgroup per work item, as above. The workgroup whose owner indices equal
//                              the slab of a point (its home) also adds the grid's share of the gradient with
//                              respect to the input, from a gather of all corners as in the records kernel, and
//                              adds all corners of points that do not fit the scheme with atomics on the
//                              gradient tensor: points outside the box (extrapolated with weights beyond one,
//                              NaN coordinates; the fixed-point scale counts on weights of at most one), points
//                              whose adjoint is not finite, and points whose cell lies in another slab than
//                              the sort's slab arithmetic put them (a coordinate within rounding of a slab
//                              boundary, or on the upper border).
// Measured on the dense 4-D grid above, 2^21 points: 165 + 7 us where the records and slice kernels take 281 + 154 us.
// Of the 165 us about 100 are the 268 M additions in LDS (ds_add_u64 retires 4 to 6 lanes per clock and compute
// unit, whatever feeds it), 37 the input gradients, 30 the rest (largest adjoint, zeroing and writing back the sums).
// A term is the product of two integers (the adjoint in units chosen from the largest adjoint of the work item, the
// weight of the corner in units of 2^-22): one v_mad_i64_i32 instead of the nine instructions that split a float
// product into two words (190 -> 165 us).
//
// Replaces, for such batches, the atomicAdd of src_cpp/include/qmlp/kernels/encoding_hashgrid.cuh:117-166,345-369
// of the reference.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/encoding_hashgrid.h>
#include <qmlp/kernels/grid_gradient.h>
#include <qmlp/kernels/point_order_key.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

/** One workgroup of GridGradientColumnsKernel: part `part` of `parts` of the points that owner (owner0, owner1) visits. */
struct GridGradientColumnItem
{
    int owner0;
    int owner1;
    int part;
    int parts;
};

constexpr int GRID_GRADIENT_COLUMNS_MAX_SLABS = 1024;   // as POINT_ORDER_MAX_SLABS
/** Points per work item from which an owner is split (four average slabs of 2^21 points in 31 x 31 slabs: 8.7 K). */
constexpr int GRID_GRADIENT_COLUMNS_PART_POINTS = 24 * 1024;

template <typename Cfg, int CPS>
struct GridGradientColumns
{
    typedef EncodingHashGrid<Cfg> Grid;
    typedef typename Grid::param_t param_t;
    static constexpr int D = Grid::D;
    static constexpr int F = Grid::F;
    static constexpr int NC = Grid::NC;
    static_assert(Cfg::Levels == 1 && !Cfg::hashed[0] && D >= 2, "one dense level of two or more dimensions");
    static constexpr int R = Cfg::resolution[0];                       // nodes per coordinate
    static constexpr int REST = static_cast<int>(detail::upow(static_cast<unsigned>(R), D - 2));   // nodes of the coordinates from 2 on
    static constexpr int OWNERS = (R + CPS - 1) / CPS;                 // per sorted coordinate
    static constexpr int COLUMN_FLOATS = REST * F;                     // all nodes that share their first two indices
    static constexpr int LOCAL_FLOATS = CPS * CPS * COLUMN_FLOATS;     // sums of one owner

    /** Where an owner keeps feature 0 of node (n0, n1, rest), rest = sum over d >= 2 of n_d R^(D-1-d). */
    __device__ __forceinline__ static int localElement(int n0, int n1, unsigned rest, int owner0, int owner1)
    {
        return (((n0 - owner0 * CPS) * CPS + (n1 - owner1 * CPS)) * REST + static_cast<int>(rest)) * F;
    }

    /** The element of the gradient table that local sum `local` of an owner stands for; valid: the node exists. */
    __device__ __forceinline__ static unsigned globalElement(int local, int owner0, int owner1, bool& valid)
    {
        const int column = local / COLUMN_FLOATS, within = local % COLUMN_FLOATS;
        const int n0 = owner0 * CPS + column / CPS, n1 = owner1 * CPS + column % CPS;
        valid = n0 < R && n1 < R;
        return static_cast<unsigned>(Cfg::memoryOffset[0])
            + (static_cast<unsigned>(n0) * static_cast<unsigned>(R) + static_cast<unsigned>(n1)) * static_cast<unsigned>(COLUMN_FLOATS)
            + static_cast<unsigned>(within);
    }

    /** Entries of the table around one slab: the nodes (a * CPS .. (a + 1) * CPS) in both sorted coordinates, all others. */
    static constexpr int REGION_NODES = CPS + 1;
    static constexpr int REGION_ENTRIES = REGION_NODES * REGION_NODES * REST;
    static constexpr int REGION_BYTES = REGION_ENTRIES * F * static_cast<int>(sizeof(typename Cfg::table_t));
    static constexpr int LDS_BYTES = ((LOCAL_FLOATS * 8 > REGION_BYTES ? LOCAL_FLOATS * 8 : REGION_BYTES) + 15) / 16 * 16;

    /** Place of node (n0, n1, rest) in the staged region of slab (a0, a1), in entries; valid: the node lies inside it. */
    __device__ __forceinline__ static int regionEntry(int n0, int n1, unsigned rest, int a0, int a1, bool& valid)
    {
        const int l0 = n0 - a0 * CPS, l1 = n1 - a1 * CPS;
        valid = l0 >= 0 && l0 < REGION_NODES && l1 >= 0 && l1 < REGION_NODES;
        return (l0 * REGION_NODES + l1) * REST + static_cast<int>(rest);
    }

    /** The position of point p in the unit box, as every kernel of the grid computes it. */
    __device__ __forceinline__ static void loadPosition(const Tensor2Read<float>& inputs, int p, const param_t& params,
                                                        bool rowsOfFloat4, float (&pos)[D])
    {
#pragma clang fp contract(off)
        float in[D];
        if (D == 4 && rowsOfFloat4) {
            const float4 v = *reinterpret_cast<const float4*>(inputs.data_ + static_cast<long long>(p) * inputs.strides_[0] + Cfg::Start);
            in[0] = v.x, in[1 % D] = v.y, in[2 % D] = v.z, in[3 % D] = v.w;
        } else {
#pragma unroll
            for (int d = 0; d < D; ++d)
                in[d] = inputs.data_[static_cast<long long>(p) * inputs.strides_[0] + static_cast<long long>(d + Cfg::Start) * inputs.strides_[1]];
        }
#pragma unroll
        for (int d = 0; d < D; ++d) pos[d] = (in[d] - params.boundingBoxMin[d]) * params.boundingBoxInvSize[d];
    }

    /** Node indices of corner c (bit d: upper in dimension d) in the two sorted coordinates, and the rest of its index. */
    __device__ __forceinline__ static void cornerNode(const typename Grid::LevelSetup& s, int c, int& n0, int& n1, unsigned& rest)
    {
        constexpr unsigned M0 = detail::upow(static_cast<unsigned>(R), D - 1), M1 = detail::upow(static_cast<unsigned>(R), D - 2);
        n0 = static_cast<int>(((c & 1) ? s.termH[0] : s.termL[0]) / M0);
        n1 = static_cast<int>(((c & 2) ? s.termH[1] : s.termL[1]) / M1);
        rest = 0u;
#pragma unroll
        for (int d = 2; d < D; ++d) rest += ((c >> d) & 1) ? s.termH[d] : s.termL[d];
    }

    /** The cell of the point in the two sorted coordinates, as the grid computes it. */
    __device__ __forceinline__ static void cell(const typename Grid::LevelSetup& s, int& c0, int& c1)
    {
        constexpr unsigned M0 = detail::upow(static_cast<unsigned>(R), D - 1), M1 = detail::upow(static_cast<unsigned>(R), D - 2);
        c0 = static_cast<int>(s.termL[0] / M0);
        c1 = static_cast<int>(s.termL[1] / M1);
    }

    __device__ __forceinline__ static bool insideBox(const typename Grid::LevelSetup& s)
    {
        bool inside = true;
#pragma unroll
        for (int d = 0; d < D; ++d) inside = inside && s.f[d] >= 0.f && s.f[d] <= 1.f;
        return inside;
    }

    /** The runs of the sorted batch that owner (o0, o1) visits: run r covers the slabs (a0, o1 - 1 | o1), a0 = o0 - 1 + r. */
    struct Runs
    {
        int begin[2], middle[2], end[2];   // points [begin, middle) lie in slab (a0, o1 - 1), [middle, end) in (a0, o1)
        __device__ __forceinline__ int points() const { return (end[0] - begin[0]) + (end[1] - begin[1]); }
    };
    __device__ __forceinline__ static Runs runsOf(int owner0, int owner1, const int* __restrict__ starts, int slabs0, int slabs1)
    {
        Runs runs;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int a0 = owner0 - 1 + r;
            runs.begin[r] = runs.middle[r] = runs.end[r] = 0;
            if (a0 < 0 || a0 >= slabs0) continue;
            const int lo = owner1 - 1, hi = owner1;   // slabs of the second coordinate
            const int first = a0 * slabs1 + max(lo, 0), last = a0 * slabs1 + min(hi, slabs1 - 1);
            if (first > last) continue;
            runs.begin[r] = starts[first];
            runs.end[r] = starts[last + 1];
            // the boundary between slab lo and slab hi (all points belong to one of them if the other does not exist)
            runs.middle[r] = lo < 0 ? runs.begin[r] : hi > slabs1 - 1 ? runs.end[r] : starts[a0 * slabs1 + hi];
        }
        return runs;
    }
};

/**
 * totals: points per slab (slabs0 * slabs1 <= 1024 values, as PointOrderScan leaves them). Writes starts
 * (slabs + 1 values), the work items and their number. One workgroup of 1024 threads.
 */
template <typename Cfg, int CPS>
__global__ void __launch_bounds__(1024) GridGradientColumnsPlan(
    int numel, const int* __restrict__ totals, int slabs0, int slabs1, int* __restrict__ starts,
    GridGradientColumnItem* __restrict__ items, int* __restrict__ itemCount, int maxItems)
{
    typedef GridGradientColumns<Cfg, CPS> Impl;
    __shared__ int sScan[GRID_GRADIENT_COLUMNS_MAX_SLABS + 1];
    __shared__ int sItems;
    const int tid = threadIdx.x;
    const int slabs = slabs0 * slabs1;
    // exclusive scan of the totals
    const int mine = tid < slabs ? totals[tid] : 0;
    int inclusive = mine;
#pragma unroll
    for (int d = 1; d < 64; d *= 2) {
        const int other = __shfl_up(inclusive, d, 64);
        if ((tid & 63) >= d) inclusive += other;
    }
    if ((tid & 63) == 63) sScan[tid / 64] = inclusive;   // wave totals
    if (tid == 0) sItems = 0;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < tid / 64; ++w) before += sScan[w];
    __syncthreads();
    sScan[tid] = before + inclusive - mine;
    if (tid == 1023) sScan[1024] = before + inclusive;
    __syncthreads();
    if (tid < slabs) starts[tid] = sScan[tid];
    if (tid == 0) starts[slabs] = numel;
    // work items
    for (int o = tid; o < Impl::OWNERS * Impl::OWNERS; o += 1024) {
        const int o0 = o / Impl::OWNERS, o1 = o % Impl::OWNERS;
        // (the starts are read from LDS: the global copy is not visible to the whole workgroup yet; the totals
        // beyond the last slab are zero, so sScan[slabs] is the number of all points)
        const typename Impl::Runs runs = Impl::runsOf(o0, o1, sScan, slabs0, slabs1);
        const int points = runs.points();
        if (points == 0) continue;
        const int parts = (points + GRID_GRADIENT_COLUMNS_PART_POINTS - 1) / GRID_GRADIENT_COLUMNS_PART_POINTS;
        const int at = atomicAdd(&sItems, parts);
        for (int part = 0; part < parts; ++part)
            if (at + part < maxItems) items[at + part] = GridGradientColumnItem{o0, o1, part, parts};
    }
    __syncthreads();
    if (tid == 0) *itemCount = min(sItems, maxItems);
}

/**
 * \tparam CPS cells per slab and sorted coordinate
 * \tparam ROW_CHANNELS, CHANNEL_OFFSET the tile layout of the adjoint of the encoded rows, as for the records kernel
 * \tparam INPUT_GRADIENTS 0: none; 1: from a gather of all corners; 2: from the position derivatives of the forward pass
 * inputs: the rows of the batch in sorted order; starts, items, itemCount: as GridGradientColumnsPlan wrote them.
 * Launched with as many workgroups as there can be work items; those beyond itemCount leave at once.
 * Dynamic LDS: GridGradientColumns::LDS_BYTES (the sums of an owner, then the entries of the table around its slab).
 */
template <typename Cfg, int CPS, int ROW_CHANNELS, int CHANNEL_OFFSET, int INPUT_GRADIENTS, int BLOCK>
__global__ void __launch_bounds__(BLOCK) GridGradientColumnsKernel(
    int numel, const Tensor2Read<float> inputs, const half* __restrict__ adjEncodedH,
    const HashGridParams<typename Cfg::table_t, Cfg::Dim> params, const int* __restrict__ starts, int slabs0, int slabs1,
    const GridGradientColumnItem* __restrict__ items, const int* __restrict__ itemCount, Tensor2RW<float> adjInputs,
    const void* __restrict__ derivativesV)
{
    typedef GridGradientColumns<Cfg, CPS> Impl;
    typedef EncodingHashGrid<Cfg> Grid;
    typedef GridGradientRecords<Cfg, ROW_CHANNELS, CHANNEL_OFFSET, 8192, 256> Records;   // its gathers for the input gradients
    typedef GridGradientSlices<Cfg, 8192> Fixed;                                         // its fixed-point arithmetic
    constexpr int D = Cfg::Dim, F = Cfg::Features, NC = Grid::NC;
    extern __shared__ __align__(16) unsigned char sMemory[];
    long long* sSums = reinterpret_cast<long long*>(sMemory);
    __shared__ int sMaxBits;
    if (static_cast<int>(blockIdx.x) >= *itemCount) return;
    const GridGradientColumnItem item = items[blockIdx.x];
    const int tid = threadIdx.x;
    const f16* __restrict__ adjEncoded = reinterpret_cast<const f16*>(adjEncodedH);
    const typename Impl::Runs runs = Impl::runsOf(item.owner0, item.owner1, starts, slabs0, slabs1);

    for (int i = tid; i < Impl::LOCAL_FLOATS; i += BLOCK) sSums[i] = 0;
    if (tid == 0) sMaxBits = 0;
    __syncthreads();

    // this part's share of both runs
    int begin[2], end[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const long long length = runs.end[r] - runs.begin[r];
        begin[r] = runs.begin[r] + static_cast<int>(length * item.part / item.parts);
        end[r] = runs.begin[r] + static_cast<int>(length * (item.part + 1) / item.parts);
        // (slab starts are sums of counts of this batch: never outside of it)
        begin[r] = max(0, min(begin[r], numel));
        end[r] = max(begin[r], min(end[r], numel));
    }

    // the largest adjoint among the points of this work item: the scale of the fixed-point sums
    {
        unsigned maxBits = 0u;
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll 4
            for (int p = begin[r] + tid; p < end[r]; p += BLOCK) {
                const f16* adjRow = adjEncoded + static_cast<long long>(p / TILE_POINTS) * (ROW_CHANNELS * TILE_POINTS)
                    + CHANNEL_OFFSET * TILE_POINTS + (p % TILE_POINTS);
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    // (a point with an adjoint that is not finite takes the atomics, see below)
                    const unsigned bits = static_cast<unsigned>(__builtin_bit_cast(unsigned short, adjRow[i * TILE_POINTS])) & 0x7fffu;
                    if (bits < 0x7c00u) maxBits = max(maxBits, bits);
                }
            }
        if (maxBits != 0u) atomicMax(&sMaxBits, static_cast<int>(maxBits));
    }
    __syncthreads();
    const unsigned maxBits = static_cast<unsigned>(sMaxBits);
    const int maxExponent = static_cast<int>(maxBits >> 10) - 14;   // |adjoint| < 2^maxExponent
    const long long terms = static_cast<long long>(NC) * max(1, (end[0] - begin[0]) + (end[1] - begin[1]));
    const int termsLog2 = 64 - __builtin_clzll(static_cast<unsigned long long>(terms));
    // A term is the product of two integers: the adjoint in units of 2^-adjointShift (below 2^adjointBits in
    // magnitude) and the weight of the corner in units of 2^-WEIGHT_BITS (at most one): one multiply-add instruction
    // per term instead of the nine of a float product split into two words. The sum of all terms that can meet in
    // one element stays below 2^62.
    constexpr int WEIGHT_BITS = 22;
    const int adjointBits = min(30, 62 - WEIGHT_BITS - termsLog2);
    const int adjointShift = adjointBits - maxExponent;
    const int scaleExponent = adjointShift + WEIGHT_BITS;
    float* __restrict__ gradients = params.parametersBackward;
    // rows of four floats that lie side by side: one load
    const bool rowsOfFloat4 = D == 4 && Cfg::Start % 4 == 0 && inputs.strides_[1] == 1 && inputs.strides_[0] % 4 == 0
        && reinterpret_cast<unsigned long long>(inputs.data_) % 16 == 0;

#pragma unroll 1
    for (int r = 0; r < 2; ++r) {
        const int a0 = item.owner0 - 1 + r;
        // (the position and the adjoints of a lane's next point are loaded before it works on this one: with four
        // wavefronts per SIMD nothing else hides the latency of the loads)
        float nextPos[D];
        f16 nextAdj[F];
        auto loadPoint = [&](int q) {
            Impl::loadPosition(inputs, q, params, rowsOfFloat4, nextPos);
            const f16* row = adjEncoded + static_cast<long long>(q / TILE_POINTS) * (ROW_CHANNELS * TILE_POINTS)
                + CHANNEL_OFFSET * TILE_POINTS + (q % TILE_POINTS);
#pragma unroll
            for (int i = 0; i < F; ++i) nextAdj[i] = row[i * TILE_POINTS];
        };
        if (begin[r] + tid < end[r]) loadPoint(begin[r] + tid);
#pragma unroll 1
        for (int p = begin[r] + tid; p < end[r]; p += BLOCK) {
            const int a1 = p < runs.middle[r] ? item.owner1 - 1 : item.owner1;
            const bool home = a0 == item.owner0 && a1 == item.owner1;
            float pos[D];
            f16 adjHalf[F];
#pragma unroll
            for (int d = 0; d < D; ++d) pos[d] = nextPos[d];
#pragma unroll
            for (int i = 0; i < F; ++i) adjHalf[i] = nextAdj[i];
            if (p + BLOCK < end[r]) loadPoint(p + BLOCK);
            const typename Grid::LevelSetup s = Grid::setupLevel(0, pos);
            int c0, c1;
            Impl::cell(s, c0, c1);
            // Points that do not fit the scheme -- the same verdict in every workgroup that visits the point: outside
            // the box, in a cell of another slab than the sort's, or with an adjoint that is not finite (NaN and
            // infinity have no fixed-point form and reach the gradients through the atomics of the point's home).
            float adj[F];
            bool finite = true;
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const f16 h = adjHalf[i];
                finite = finite && (static_cast<unsigned>(__builtin_bit_cast(unsigned short, h)) & 0x7c00u) != 0x7c00u;
                adj[i] = static_cast<float>(h);
            }
            const bool regular = finite && Impl::insideBox(s) && c0 / CPS == a0 && c1 / CPS == a1;
            if (!regular && !home) continue;
            if (regular) {
                if (maxBits != 0u) {
                    // neighbouring lanes take the features in rotated order (an entry starts at a multiple of
                    // 8 F bytes: lanes that all add the same feature would meet on a few LDS banks)
                    int rotated[F];
#pragma unroll
                    for (int step = 0; step < F; ++step) {
                        const int i = (F & (F - 1)) == 0 ? ((step + tid) & (F - 1)) : ((step + tid % F) % F);
                        float a = adj[0];
#pragma unroll
                        for (int k = 1; k < F; ++k) a = i == k ? adj[k] : a;
                        rotated[step] = static_cast<int>(rintf(ldexpf(a, adjointShift)));
                    }
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        int n0, n1;
                        unsigned rest;
                        Impl::cornerNode(s, c, n0, n1, rest);
                        if (n0 / CPS != item.owner0 || n1 / CPS != item.owner1) continue;
                        const int w = static_cast<int>(rintf(ldexpf(Grid::cornerWeight(s, c), WEIGHT_BITS)));
                        long long* sums = sSums + Impl::localElement(n0, n1, rest, item.owner0, item.owner1);
#pragma unroll
                        for (int step = 0; step < F; ++step) {
                            const int i = (F & (F - 1)) == 0 ? ((step + tid) & (F - 1)) : ((step + tid % F) % F);
                            Fixed::ldsAddFixed(sums + i, static_cast<long long>(w) * static_cast<long long>(rotated[step]));
                        }
                    }
                }
            } else {
                // home of a point that does not fit the scheme: all of its corners, with atomics
#pragma unroll 1
                for (int c = 0; c < NC; ++c) {
                    const float w = Grid::cornerWeight(s, c);
                    const unsigned element = Grid::cornerOffset(0, s, c);
#pragma unroll 1
                    for (int i = 0; i < F; ++i) unsafeAtomicAdd(gradients + element + i, w * adj[i]);
                }
            }
        }
    }
    __syncthreads();

    // The sums of this owner, added with atomics (16 neighbouring floats per request): other workgroups may be adding
    // the corners of points that do not fit the scheme to the same elements at this moment, and the parts of a
    // split owner hold sums for the same elements.
    if (maxBits != 0u) {
        for (int i = tid; i < Impl::LOCAL_FLOATS; i += BLOCK) {
            const long long fixed = sSums[i];
            if (fixed == 0) continue;
            bool valid;
            const unsigned element = Impl::globalElement(i, item.owner0, item.owner1, valid);
            if (!valid) continue;
            const float v = static_cast<float>(ldexp(static_cast<double>(fixed), -scaleExponent));
            unsafeAtomicAdd(gradients + element, v);
        }
    }

    if constexpr (INPUT_GRADIENTS != 0) {
        // The grid's share of the gradient with respect to the input, for the points whose slab has the indices of
        // this owner (every point has one such home: a plain read-modify-write of its row). From the position
        // derivatives of the forward pass where it kept them; else from the entries of all corners, as the records
        // kernel gathers them -- but out of the LDS, which the sums have left: the entries around one slab are as
        // many bytes as an owner's sums (half tables) and are copied in with coalesced loads once, instead of
        // 2^D gathers of one entry per point (dense 4-D grid with 8 features, 2^21 points: 96 -> 37 us).
        const int a0 = item.owner0, a1 = item.owner1;
        if (a0 >= slabs0 || a1 >= slabs1) return;   // an owner of border nodes only: no slab of its own
        const int homeBegin = max(begin[1], min(runs.middle[1], end[1])), homeEnd = end[1];
        if (homeBegin >= homeEnd) return;           // (the same for the whole workgroup)
        typedef typename Cfg::table_t table_t;
        table_t* sRegion = reinterpret_cast<table_t*>(sMemory);
        if constexpr (INPUT_GRADIENTS == 1) {
            __syncthreads();   // the sums have been read
            // 16 bytes per load: the entries of one (n0, n1) are REST * F values side by side in the table and in the region
            constexpr int COLUMN_VALUES = Impl::REST * F;
            constexpr int WIDEST = 16 / static_cast<int>(sizeof(table_t));
            constexpr int PER_LOAD = COLUMN_VALUES % WIDEST == 0 ? WIDEST : COLUMN_VALUES % (WIDEST / 2) == 0 ? WIDEST / 2
                : COLUMN_VALUES % (WIDEST / 4) == 0 ? WIDEST / 4 : 1;
            typedef table_t load_t __attribute__((ext_vector_type(PER_LOAD)));
            for (int i = tid; i < Impl::REGION_NODES * Impl::REGION_NODES * (COLUMN_VALUES / PER_LOAD); i += BLOCK) {
                const int column = i / (COLUMN_VALUES / PER_LOAD), within = i % (COLUMN_VALUES / PER_LOAD);
                const int n0 = a0 * CPS + column / Impl::REGION_NODES, n1 = a1 * CPS + column % Impl::REGION_NODES;
                if (n0 < Impl::R && n1 < Impl::R) {
                    const table_t* src = params.parametersForward + Cfg::memoryOffset[0]
                        + (static_cast<long long>(n0) * Impl::R + n1) * COLUMN_VALUES + within * PER_LOAD;
                    *reinterpret_cast<load_t*>(sRegion + column * COLUMN_VALUES + within * PER_LOAD) = *reinterpret_cast<const load_t*>(src);
                }
            }
            __syncthreads();
        }
#pragma unroll 1
        for (int p = homeBegin + tid; p < homeEnd; p += BLOCK) {
            float pos[D];
            Impl::loadPosition(inputs, p, params, rowsOfFloat4, pos);
            float adjPos[D];
#pragma unroll
            for (int d = 0; d < D; ++d) adjPos[d] = 0.f;
            if constexpr (INPUT_GRADIENTS == 2) {
                Records::template positionGradientFromDerivatives<0>(
                    p, static_cast<const typename Records::DerivativeChunk*>(derivativesV), adjEncoded, adjPos);
            } else {
                const typename Grid::LevelSetup s = Grid::setupLevel(0, pos);
                detail::HeldFeatures<F, table_t> held[NC];
                // (a point in a cell of another slab than the sort's -- within rounding of a slab boundary, on the upper
                // border -- may have corners outside the region: it gathers from the table)
                bool staged = true;
                int entry[NC];
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    int n0, n1;
                    unsigned rest;
                    Impl::cornerNode(s, c, n0, n1, rest);
                    bool valid;
                    entry[c] = Impl::regionEntry(n0, n1, rest, a0, a1, valid);
                    staged = staged && valid;
                }
                if (staged) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) held[c].load(sRegion + entry[c] * F);
                } else {
                    Records::template loadHeld<0>(s, params, held);
                }
                Records::template positionGradient<0>(p, s, held, adjEncoded, adjPos);
            }
#pragma unroll
            for (int d = 0; d < D; ++d)
                adjInputs.data_[static_cast<long long>(p) * adjInputs.strides_[0]
                                + static_cast<long long>(d + Cfg::Start) * adjInputs.strides_[1]] += adjPos[d] * params.boundingBoxInvSize[d];
        }
    }
}

/**
 * Test aid: for every point (one per lane) and corner, the element of the gradient table that the sum stands for
 * to which GridGradientColumnsKernel adds the corner -- through the place in the LDS of the owner of the corner's
 * node and back, as the kernel goes -- and its weight. Slots: corner (bit d: upper in dimension d).
 */
template <typename Cfg, int CPS>
__global__ void __launch_bounds__(256) GridGradientColumnsTraceKernel(
    long long numel, const Tensor2Read<float> inputs, unsigned* __restrict__ indices, float* __restrict__ weights,
    const HashGridParams<typename Cfg::table_t, Cfg::Dim> params)
{
    typedef GridGradientColumns<Cfg, CPS> Impl;
    typedef EncodingHashGrid<Cfg> Grid;
    constexpr int D = Cfg::Dim, NC = Grid::NC;
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
        const typename Grid::LevelSetup s = Grid::setupLevel(0, pos);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            int n0, n1;
            unsigned rest;
            Impl::cornerNode(s, c, n0, n1, rest);
            const int o0 = n0 / CPS, o1 = n1 / CPS;
            bool valid;
            const unsigned element = Impl::globalElement(Impl::localElement(n0, n1, rest, o0, o1), o0, o1, valid);
            indices[index * NC + c] = valid ? element : 0xffffffffu;
            weights[index * NC + c] = Grid::cornerWeight(s, c);
        }
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
