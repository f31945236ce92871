// Orders the points of a batch by the slab of a grid they fall into, so that the
// wavefronts that run side by side gather from the same few megabytes of the table and
// find them in L1 / L2, and the lanes of one gather instruction fall onto fewer cache lines. A counting sort over at most 1024 slabs in three launches, without
// atomics on device memory (a first version reserved the ranges with one returning atomic per
// slab and workgroup: 256 workgroups on the same 64 cache lines took 120 us):
//   PointOrderCount   one histogram per workgroup (summed in LDS) over its chunk of the batch,
//   PointOrderScan    per slab, the running sum over the workgroups (in place) and the total,
//   PointOrderScatter scans the totals into slab offsets, sorts its chunk in LDS and writes
//                     it to slab offset + running sum + rank in the chunk: a copy of the
//                     input rows in sorted order and, per sorted position, the index of the
//                     point in the caller's batch (and, for training passes, per point its sorted position).
// The order of the points of one chunk inside a slab depends on the timing of the wavefronts;
// the fused kernel evaluates every point on its own, so its results do not.
// No counterpart in the reference, which evaluates the points in the order given.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/point_order_key.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

constexpr int POINT_ORDER_MAX_SLABS = 1024;
constexpr int POINT_ORDER_BLOCK = 1024;
constexpr int POINT_ORDER_POINTS_PER_THREAD = 4;    // a workgroup's chunk: 4096 points (offsets in it take 12 bits)
constexpr int POINT_ORDER_SCAN_SLABS = 16;          // slabs per workgroup of PointOrderScan

/** Slab of one coordinate value, clamped to the box (the comparisons are false for NaN, which then lands in slab 0). */
__device__ __forceinline__ int pointOrderSlab1(float value, float lo, float scale, int slabs)
{
    const float p = (value - lo) * scale;
    return p > 0.f ? static_cast<int>(fminf(p, static_cast<float>(slabs - 1))) : 0;
}

/** Slab of a point: up to three grid coordinates, clamped to the box. channel(c): the value of input channel c. */
template <typename Channel>
__device__ __forceinline__ int pointOrderSlabOf(const Channel& channel, const PointOrderKey& key)
{
    int s = pointOrderSlab1(channel(key.channel0), key.min0, key.scale0, key.slabs0);
    if (key.slabs1 > 1) {
        const int s1 = pointOrderSlab1(channel(key.channel1), key.min1, key.scale1, key.slabs1);
        if (key.slabs2 > 1) {
            const int s2 = pointOrderSlab1(channel(key.channel2), key.min2, key.scale2, key.slabs2);
            if (key.interleave12) {
                // bit b of s1 to position 2b + 1, of s2 to 2b (at most 5 bits each)
                int z = 0;
#pragma unroll
                for (int b = 0; b < 5; ++b) z |= ((s1 >> b) & 1) << (2 * b + 1) | ((s2 >> b) & 1) << (2 * b);
                s = s * (key.slabs1 * key.slabs2) + z;
            } else {
                s = (s * key.slabs1 + s1) * key.slabs2 + s2;
            }
        } else {
            s = s * key.slabs1 + s1;
        }
    }
    return s;
}

/** Slab of the point in row `index` of the inputs. */
__device__ __forceinline__ int pointOrderSlab(const Tensor2Read<float>& inputs, long long index, const PointOrderKey& key)
{
    const float* row = inputs.data_ + index * inputs.strides_[0];
    const long long channelStride = inputs.strides_[1];
    return pointOrderSlabOf([&](int c) { return row[static_cast<long long>(c) * channelStride]; }, key);
}

/** histogram: (workgroups, POINT_ORDER_MAX_SLABS), every entry is written. */
__global__ void __launch_bounds__(POINT_ORDER_BLOCK) PointOrderCount(
    int numel, const Tensor2Read<float> inputs, const PointOrderKey key, int* __restrict__ histogram)
{
    __shared__ int sCount[POINT_ORDER_MAX_SLABS];
    sCount[threadIdx.x] = 0;
    __syncthreads();
    const long long chunk = static_cast<long long>(blockIdx.x) * (POINT_ORDER_BLOCK * POINT_ORDER_POINTS_PER_THREAD);
#pragma unroll
    for (int k = 0; k < POINT_ORDER_POINTS_PER_THREAD; ++k) {
        const long long index = chunk + k * POINT_ORDER_BLOCK + threadIdx.x;
        if (index < numel) atomicAdd(&sCount[pointOrderSlab(inputs, index, key)], 1);
    }
    __syncthreads();
    histogram[blockIdx.x * POINT_ORDER_MAX_SLABS + threadIdx.x] = sCount[threadIdx.x];
}

/**
 * histogram[w][slab] becomes the number of points of the slab in the chunks before w,
 * totals[slab] their number in all chunks. A workgroup takes POINT_ORDER_SCAN_SLABS slabs; 64 groups of
 * its threads take a 64th of the chunks each: sum, exchange through LDS, running sum. (64 workgroups: with
 * 16 workgroups of 64 slabs the pass took 8 us for 256 chunks and 13 us for 512.)
 */
__global__ void __launch_bounds__(POINT_ORDER_BLOCK) PointOrderScan(int chunks, int* __restrict__ histogram, int* __restrict__ totals)
{
    constexpr int GROUPS = POINT_ORDER_BLOCK / POINT_ORDER_SCAN_SLABS;
    constexpr int BATCH = 8;   // loads in flight
    __shared__ int sPartial[GROUPS][POINT_ORDER_SCAN_SLABS];
    const int local = threadIdx.x % POINT_ORDER_SCAN_SLABS, group = threadIdx.x / POINT_ORDER_SCAN_SLABS;
    const int slab = blockIdx.x * POINT_ORDER_SCAN_SLABS + local;
    const int perGroup = (chunks + GROUPS - 1) / GROUPS;
    const int begin = min(group * perGroup, chunks), end = min(begin + perGroup, chunks);
    int sum = 0;
    for (int w0 = begin; w0 < end; w0 += BATCH) {
#pragma unroll
        for (int j = 0; j < BATCH; ++j)
            if (w0 + j < end) sum += histogram[(w0 + j) * POINT_ORDER_MAX_SLABS + slab];
    }
    sPartial[group][local] = sum;
    __syncthreads();
    int running = 0;
    for (int q = 0; q < group; ++q) running += sPartial[q][local];
    if (group == GROUPS - 1) totals[slab] = running + sum;
    for (int w0 = begin; w0 < end; w0 += BATCH) {
        int v[BATCH];
#pragma unroll
        for (int j = 0; j < BATCH; ++j) v[j] = w0 + j < end ? histogram[(w0 + j) * POINT_ORDER_MAX_SLABS + slab] : 0;
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            if (w0 + j < end) histogram[(w0 + j) * POINT_ORDER_MAX_SLABS + slab] = running;
            running += v[j];
        }
    }
}

/** Exclusive scan over the POINT_ORDER_MAX_SLABS values held one per thread of the workgroup. */
__device__ __forceinline__ int pointOrderBlockScan(int value, int* sWaveSum)
{
    const int lane = threadIdx.x % WAVE_SIZE, wave = threadIdx.x / WAVE_SIZE;
    int inclusive = value;
#pragma unroll
    for (int d = 1; d < WAVE_SIZE; d *= 2) {
        const int other = __shfl_up(inclusive, d, WAVE_SIZE);
        if (lane >= d) inclusive += other;
    }
    __syncthreads();   // sWaveSum may still be read from a previous scan
    if (lane == WAVE_SIZE - 1) sWaveSum[wave] = inclusive;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w) before += sWaveSum[w];
    return before + inclusive - value;
}

/** The channels of one input row; one load of 8, 12 or 16 bytes where the layout allows it (vectorChannels > 0:
 *  rows of that many channels with unit stride between them, aligned to the vector). */
template <int MAX_CHANNELS>
__device__ __forceinline__ void pointOrderLoadRow(const Tensor2Read<float>& inputs, long long index, int vectorChannels, float (&row)[MAX_CHANNELS])
{
    const float* src = inputs.data_ + index * inputs.strides_[0];
    typedef float f32x3a __attribute__((ext_vector_type(3), aligned(4)));
    if (MAX_CHANNELS >= 4 && vectorChannels == 4) {
        const float4 v = *reinterpret_cast<const float4*>(src);
        row[0] = v.x; row[1] = v.y; row[2 % MAX_CHANNELS] = v.z; row[3 % MAX_CHANNELS] = v.w;
    } else if (MAX_CHANNELS >= 3 && vectorChannels == 3) {
        const f32x3a v = *reinterpret_cast<const f32x3a*>(src);
        row[0] = v[0]; row[1] = v[1]; row[2 % MAX_CHANNELS] = v[2];
    } else if (MAX_CHANNELS >= 2 && vectorChannels == 2) {
        const float2 v = *reinterpret_cast<const float2*>(src);
        row[0] = v.x; row[1] = v.y;
    } else {
#pragma unroll
        for (int c = 0; c < MAX_CHANNELS; ++c)
            row[c] = c < inputs.sizes_[1] ? src[static_cast<long long>(c) * inputs.strides_[1]] : 0.f;
    }
}

/** How the rows of inputs can be loaded as one vector each (pointOrderLoadRow), 0 if they cannot. */
__device__ __forceinline__ int pointOrderVectorChannels(const Tensor2Read<float>& inputs)
{
    const int channels = inputs.sizes_[1];
    if (inputs.strides_[1] != 1) return 0;
    const unsigned long long base = reinterpret_cast<unsigned long long>(inputs.data_);
    if (channels == 4 && inputs.strides_[0] % 4 == 0 && base % 16 == 0) return 4;
    if (channels == 3) return 3;   // three words from an address that is a multiple of four
    if (channels == 2 && inputs.strides_[0] % 2 == 0 && base % 8 == 0) return 2;
    return 0;
}

/** Writes the channels of one row of the sorted copy; one store of 8, 12 or 16 bytes where the rows came as vectors. */
template <int MAX_CHANNELS>
__device__ __forceinline__ void pointOrderStoreRow(float* __restrict__ sortedInputs, long long position, int channels, int vectorChannels,
                                                   const float (&row)[MAX_CHANNELS])
{
    typedef float f32x3a __attribute__((ext_vector_type(3), aligned(4)));
    if (MAX_CHANNELS >= 4 && vectorChannels == 4) {
        *reinterpret_cast<float4*>(sortedInputs + position * 4) = make_float4(row[0], row[1], row[2 % MAX_CHANNELS], row[3 % MAX_CHANNELS]);
    } else if (MAX_CHANNELS >= 3 && vectorChannels == 3) {
        const f32x3a v = {row[0], row[1], row[2 % MAX_CHANNELS]};
        *reinterpret_cast<f32x3a*>(sortedInputs + position * 3) = v;
    } else if (MAX_CHANNELS >= 2 && vectorChannels == 2) {
        *reinterpret_cast<float2*>(sortedInputs + position * 2) = make_float2(row[0], row[1]);
    } else {
#pragma unroll
        for (int c = 0; c < MAX_CHANNELS; ++c)
            if (c < channels) sortedInputs[position * channels + c] = row[c];
    }
}

/**
 * The workgroup sorts its chunk by slab in LDS, then walks the sorted chunk with consecutive lanes on
 * consecutive positions, so that the stores of a wavefront fall into a few runs (a scatter straight from the
 * unsorted chunk sent every lane's stores to a line of their own and took 80 us for 2^21 points).
 * Rows of up to four channels are read once, in the order given (consecutive lanes, consecutive rows), and wait
 * in LDS at their sorted place. Reading them a second time in sorted order, as wider rows still are, asks for 64
 * lines per instruction, many of which the chunks of the other workgroups have meanwhile pushed out of the L2:
 * 14 of the 42 us of this kernel for 2^21 rows of 16 bytes (the stores of the rows take 13 us, everything else 14).
 * \tparam MAX_CHANNELS at least the number of input channels (4, 8, 16)
 */
template <int MAX_CHANNELS>
__global__ void __launch_bounds__(POINT_ORDER_BLOCK) PointOrderScatter(
    int numel, const Tensor2Read<float> inputs, const PointOrderKey key,
    const int* __restrict__ histogram,  // as PointOrderScan left it
    const int* __restrict__ totals,
    float* __restrict__ sortedInputs,   // (numel, inputs.sizes_[1]), dense, 16-byte aligned
    int* __restrict__ order,            // (numel): sorted position -> index in the batch
    int* __restrict__ placement)        // null, or (numel): index in the batch -> sorted position (consecutive lanes, consecutive words)
{
    constexpr int CHUNK = POINT_ORDER_BLOCK * POINT_ORDER_POINTS_PER_THREAD;
    constexpr bool STAGE_ROWS = MAX_CHANNELS <= 4;
    __shared__ int sStart[POINT_ORDER_MAX_SLABS];        // first position of the chunk's points of a slab in the sorted batch
    __shared__ int sCount[POINT_ORDER_MAX_SLABS];
    __shared__ int sLocalStart[POINT_ORDER_MAX_SLABS];   // the same inside the sorted chunk
    __shared__ int sWaveSum[POINT_ORDER_BLOCK / WAVE_SIZE];
    __shared__ unsigned int sSorted[CHUNK];              // sorted chunk: slab << 16 | offset of the point in the chunk
    __shared__ __align__(16) float sRows[STAGE_ROWS ? CHUNK * MAX_CHANNELS : 4];   // the rows of the sorted chunk
    const int t = threadIdx.x;

    sCount[t] = 0;
    const int total = totals[t];
    const int slabStart = pointOrderBlockScan(total, sWaveSum);   // holds a barrier after sCount = 0
    sStart[t] = slabStart + histogram[blockIdx.x * POINT_ORDER_MAX_SLABS + t];

    const int channels = inputs.sizes_[1];
    const int vectorChannels = pointOrderVectorChannels(inputs);
    const long long chunk = static_cast<long long>(blockIdx.x) * CHUNK;
    const int chunkPoints = static_cast<int>(min(static_cast<long long>(CHUNK), numel - chunk));
    int slab[POINT_ORDER_POINTS_PER_THREAD], rank[POINT_ORDER_POINTS_PER_THREAD];
    float rows[STAGE_ROWS ? POINT_ORDER_POINTS_PER_THREAD : 1][MAX_CHANNELS] = {};
    (void)rows;
#pragma unroll
    for (int k = 0; k < POINT_ORDER_POINTS_PER_THREAD; ++k) {
        const int j = k * POINT_ORDER_BLOCK + t;
        slab[k] = 0;
        rank[k] = 0;
        if (j < chunkPoints) {
            if constexpr (STAGE_ROWS) {
                pointOrderLoadRow<MAX_CHANNELS>(inputs, chunk + j, vectorChannels, rows[k]);
                const float (&row)[MAX_CHANNELS] = rows[k];
                slab[k] = pointOrderSlabOf([&](int c) {
                    float v = row[0];
#pragma unroll
                    for (int i = 1; i < MAX_CHANNELS; ++i) v = c == i ? row[i] : v;
                    return v;
                }, key);
            } else {
                slab[k] = pointOrderSlab(inputs, chunk + j, key);
            }
            rank[k] = atomicAdd(&sCount[slab[k]], 1);
        }
    }
    __syncthreads();
    sLocalStart[t] = pointOrderBlockScan(sCount[t], sWaveSum);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < POINT_ORDER_POINTS_PER_THREAD; ++k) {
        const int j = k * POINT_ORDER_BLOCK + t;
        if (j < chunkPoints) {
            const int at = sLocalStart[slab[k]] + rank[k];
            sSorted[at] = static_cast<unsigned int>(slab[k]) << 16 | static_cast<unsigned int>(j);
            if (placement) placement[chunk + j] = sStart[slab[k]] + rank[k];
            if constexpr (STAGE_ROWS) {
#pragma unroll
                for (int c = 0; c < MAX_CHANNELS; ++c) sRows[at * MAX_CHANNELS + c] = rows[k][c];
            }
        }
    }
    __syncthreads();

#pragma unroll 4
    for (int k = 0; k < POINT_ORDER_POINTS_PER_THREAD; ++k) {
        const int j = k * POINT_ORDER_BLOCK + t;
        if (j >= chunkPoints) continue;
        const unsigned int entry = sSorted[j];
        const long long index = chunk + (entry & 0xffffu);
        const int s = static_cast<int>(entry >> 16);
        float row[MAX_CHANNELS];
        if constexpr (STAGE_ROWS) {
#pragma unroll
            for (int c = 0; c < MAX_CHANNELS; ++c) row[c] = sRows[j * MAX_CHANNELS + c];
        } else {
            pointOrderLoadRow<MAX_CHANNELS>(inputs, index, vectorChannels, row);
        }
        const long long position = sStart[s] + (j - sLocalStart[s]);
        order[position] = static_cast<int>(index);
        pointOrderStoreRow<MAX_CHANNELS>(sortedInputs, position, channels, vectorChannels, row);
    }
}

/**
 * Rows that were computed in the sorted order, added to the caller's tensor: dst[j, c] += src[placement[j], c]
 * (src dense). The rows of dst are walked in their own order, so the read-modify-write is coalesced and only the
 * reads of src are scattered (2^21 rows of 16 bytes: 76 us as a scatter through `order`, whose rows of 16 bytes
 * each cost a line read and a line written).
 */
__global__ void __launch_bounds__(POINT_ORDER_BLOCK) PointOrderGatherAddRows(
    long long elements, int channels, const float* __restrict__ src, const int* __restrict__ placement, Tensor2RW<float> dst)
{
    for (long long e = static_cast<long long>(blockIdx.x) * POINT_ORDER_BLOCK + threadIdx.x; e < elements;
         e += static_cast<long long>(gridDim.x) * POINT_ORDER_BLOCK) {
        const long long row = e / channels;
        const int c = static_cast<int>(e - row * channels);
        dst.data_[row * dst.strides_[0] + static_cast<long long>(c) * dst.strides_[1]] += src[static_cast<long long>(placement[row]) * channels + c];
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
