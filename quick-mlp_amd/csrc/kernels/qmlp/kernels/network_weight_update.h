// Template of the weight-update kernels. The host code generator replaces everything
// in $$..$$ before the source is handed to the runtime compiler.
//
// dW_l (C_out x C_in, fp32, accumulated) = sum over the batch of dpre_l (x) in_l, and
// db_l = sum over the batch of dpre_l: a batch reduction on the matrix cores with the
// points as contraction index. Both operands are read from the channel-major
// 64-point tiles the forward/adjoint kernels wrote (8 consecutive points of one
// channel per lane = one 16-byte load in operand layout); in_l is the activation of
// the previous layer re-applied on the fly, or the stored encoded input for layer 0.
// Many workgroups reduce disjoint slices of the batch; each wave accumulates in fp32
// registers, the waves of a workgroup are combined through LDS and the workgroup stores
// its partial sums (slice-major) without atomics: thousands of atomic additions onto the
// same few cache lines serialise in the memory system and took ten times longer than
// the reduction itself. WeightUpdateReduceKernel then adds the partial sums of all slices
// to the gradient tensor, in a fixed order, so the result is reproducible bit by bit.
//
// Replaces WeightUpdateSingleBlockKernel of the reference
// (src_cpp/include/qmlp/kernels/network_weight_update_block.cuh:356-494), which runs
// in a single thread block and has no bias gradient.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/layer.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

namespace activations
{
$$DEFINE_ACTIVATIONS$$
    // stands for "no activation": the operand already holds the layer input
    struct passthrough_
    {
        static __device__ __forceinline__ half forward(half x) { return x; }
    };
}

/**
 * \tparam CIN, COUT padded layer widths
 * \tparam BIAS also reduce the bias gradient
 * \tparam InputActivation activation applied to the B operand (previous layer), or passthrough_
 * \tparam MO_CHUNK number of 16-row output tiles one workgroup accumulates; the grid is
 *         (COUT/16/MO_CHUNK) chunks x batch slices, chunk index fastest
 */
template <int CIN, int COUT, bool BIAS, typename InputActivation, int MO_CHUNK>
__global__ void __launch_bounds__($$BLOCK_SIZE$$) WeightUpdateKernel(
    int numTiles,                     // 64-point tiles in the batch
    float* __restrict__ partialWeights,  // slice 0 of this layer's (COUT, CIN) row-major partial sums
    float* __restrict__ partialBias,     // slice 0 of this layer's (COUT) partial sums, or nullptr
    int sliceStride,                     // distance between the slices in floats
    const half* __restrict__ adjPreH, // dpre tiles of this layer: (numTiles, COUT, 64)
    const half* __restrict__ inputH)  // input tiles of this layer: (numTiles, CIN, 64)
{
    constexpr int KT = CIN / 16;
    constexpr int MT = COUT / 16;
    constexpr int NCHUNK = MT / MO_CHUNK;
    constexpr int WAVES = $$BLOCK_SIZE$$ / WAVE_SIZE;
    static_assert(MT % MO_CHUNK == 0, "chunk size must divide the number of output tiles");

    const f16* __restrict__ adjPre = reinterpret_cast<const f16*>(adjPreH);
    const f16* __restrict__ input = reinterpret_cast<const f16*>(inputH);

    const int wave = threadIdx.x / WAVE_SIZE;
    const int lane = threadIdx.x % WAVE_SIZE;
    const int g = lane >> 4, r = lane & 15;
    const int chunk = blockIdx.x % NCHUNK;
    const int slice = blockIdx.x / NCHUNK;
    const int numSlices = gridDim.x / NCHUNK;
    const int mo0 = chunk * MO_CHUNK;

    f32x4 acc[MO_CHUNK][KT];
    f32x4 accBias[MO_CHUNK];
#pragma unroll
    for (int mo = 0; mo < MO_CHUNK; ++mo) {
        accBias[mo] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mi = 0; mi < KT; ++mi) acc[mo][mi] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const f16x8 ones = {1, 1, 1, 1, 1, 1, 1, 1};

    for (int tile = slice * WAVES + wave; tile < numTiles; tile += numSlices * WAVES)
    {
        const f16* aTile = adjPre + static_cast<long long>(tile) * (COUT * TILE_POINTS);
        const f16* bTile = input + static_cast<long long>(tile) * (CIN * TILE_POINTS);
#pragma unroll
        for (int kb = 0; kb < TILE_POINTS / 32; ++kb) {
            f16x8 b[KT];
#pragma unroll
            for (int mi = 0; mi < KT; ++mi) {
                const f16x8 raw = *reinterpret_cast<const f16x8*>(bTile + (16 * mi + r) * TILE_POINTS + 32 * kb + 8 * g);
                b[mi] = activationForwardChannel<InputActivation>(raw, 16 * mi + r);
            }
#pragma unroll
            for (int mo = 0; mo < MO_CHUNK; ++mo) {
                const f16x8 a = *reinterpret_cast<const f16x8*>(aTile + (16 * (mo0 + mo) + r) * TILE_POINTS + 32 * kb + 8 * g);
#pragma unroll
                for (int mi = 0; mi < KT; ++mi) acc[mo][mi] = mfma32(a, b[mi], acc[mo][mi]);
                if constexpr (BIAS) accBias[mo] = mfma32(a, ones, accBias[mo]);
            }
        }
    }

    // combine the waves of the workgroup through LDS, then store the slice's partial sums
    extern __shared__ __align__(16) unsigned char sMemory[];
    float* sAcc = reinterpret_cast<float*>(sMemory);   // (MO_CHUNK*KT + MO_CHUNK) tiles of 256 floats
    constexpr int TILES = MO_CHUNK * KT + (BIAS ? MO_CHUNK : 0);
    for (int i = threadIdx.x; i < TILES * 256; i += blockDim.x) sAcc[i] = 0.f;
    __syncthreads();
#pragma unroll
    for (int mo = 0; mo < MO_CHUNK; ++mo) {
#pragma unroll
        for (int mi = 0; mi < KT; ++mi)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                atomicAdd(&sAcc[(mo * KT + mi) * 256 + (4 * g + i) * 16 + r], acc[mo][mi][i]);
        if constexpr (BIAS) {
            if (r == 0) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    atomicAdd(&sAcc[(MO_CHUNK * KT + mo) * 256 + 4 * g + i], accBias[mo][i]);
            }
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < MO_CHUNK * KT * 256; e += blockDim.x) {
        const int t = e >> 8, within = e & 255;
        const int mo = t / KT, mi = t - mo * KT;
        const int row = 16 * (mo0 + mo) + (within >> 4), col = 16 * mi + (within & 15);
        partialWeights[static_cast<long long>(slice) * sliceStride + row * CIN + col] = sAcc[e];
    }
    if constexpr (BIAS) {
        for (int e = threadIdx.x; e < MO_CHUNK * 16; e += blockDim.x) {
            const int mo = e >> 4;
            partialBias[static_cast<long long>(slice) * sliceStride + 16 * (mo0 + mo) + (e & 15)]
                = sAcc[(MO_CHUNK * KT + mo) * 256 + (e & 15)];
        }
    }
}

/**
 * gradients[i] += sum over the slices of partial[slice * count + i]. One workgroup of
 * 1024 threads per 64 parameters: 16 wavefronts each sum every 16th slice, LDS combines them.
 */
__global__ void __launch_bounds__(1024) WeightUpdateReduceKernel(
    int count, int numSlices, const float* __restrict__ partial, float* __restrict__ gradients)
{
    __shared__ float sSum[16][WAVE_SIZE];
    const int lane = threadIdx.x % WAVE_SIZE;
    const int group = threadIdx.x / WAVE_SIZE;
    const int i = blockIdx.x * WAVE_SIZE + lane;
    float sum = 0.f;
    if (i < count) {
        int s = group;
        for (; s + 7 * 16 < numSlices; s += 8 * 16) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[static_cast<long long>(s + 16 * u) * count + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += v[u];
        }
        for (; s < numSlices; s += 16) sum += partial[static_cast<long long>(s) * count + i];
    }
    sSum[group][lane] = sum;
    __syncthreads();
    if (group == 0 && i < count) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < 16; ++w) total += sSum[w][lane];
        gradients[i] += total;
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
