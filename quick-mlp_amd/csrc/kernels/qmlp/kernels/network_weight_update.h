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
// registers, the waves of a workgroup are combined through LDS in a fixed order and the workgroup stores
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
 * \tparam MO_CHUNK number of 16-row output tiles and
 * \tparam KI_CHUNK number of 16-column input tiles one workgroup accumulates: a workgroup owns a
 *         MO_CHUNK x KI_CHUNK block of the 16 x 16 tiles of dW. The grid is
 *         (COUT/16/MO_CHUNK) x (CIN/16/KI_CHUNK) blocks x batch slices.
 *         Splitting the input channels re-reads dpre, splitting the output channels re-reads
 *         the input and re-applies its activation; the host picks the cheaper split.
 */
template <int CIN, int COUT, bool BIAS, typename InputActivation, int MO_CHUNK, int KI_CHUNK>
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
    constexpr int MCHUNKS = MT / MO_CHUNK;
    constexpr int KCHUNKS = KT / KI_CHUNK;
    constexpr int NCHUNK = MCHUNKS * KCHUNKS;
    constexpr int WAVES = $$BLOCK_SIZE$$ / WAVE_SIZE;
    static_assert(MT % MO_CHUNK == 0 && KT % KI_CHUNK == 0, "chunk sizes must divide the numbers of tiles");

    const f16* __restrict__ adjPre = reinterpret_cast<const f16*>(adjPreH);
    const f16* __restrict__ input = reinterpret_cast<const f16*>(inputH);

    const int wave = threadIdx.x / WAVE_SIZE;
    const int lane = threadIdx.x % WAVE_SIZE;
    const int g = lane >> 4, r = lane & 15;
    // Workgroups are handed to the 8 XCDs in turn. The NCHUNK workgroups that read the same
    // slice of the batch (different blocks of dW) are therefore placed 8 apart, onto the same
    // XCD: the operand they share is then read from HBM once and from that XCD's L2 afterwards.
    const int numSlices = gridDim.x / NCHUNK;
    int chunk, slice;
    if (NCHUNK > 1 && numSlices % 8 == 0) {
        chunk = (blockIdx.x / 8) % NCHUNK;
        slice = (blockIdx.x / (8 * NCHUNK)) * 8 + blockIdx.x % 8;
    } else {
        chunk = blockIdx.x % NCHUNK;
        slice = blockIdx.x / NCHUNK;
    }
    const int mo0 = (chunk % MCHUNKS) * MO_CHUNK;
    const int ki0 = (chunk / MCHUNKS) * KI_CHUNK;
    const bool ownsBias = BIAS && ki0 == 0;   // the bias gradient does not depend on the input channels

    f32x4 acc[MO_CHUNK][KI_CHUNK];
    f32x4 accBias[MO_CHUNK];
#pragma unroll
    for (int mo = 0; mo < MO_CHUNK; ++mo) {
        accBias[mo] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mi = 0; mi < KI_CHUNK; ++mi) acc[mo][mi] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const f16x8 ones = {1, 1, 1, 1, 1, 1, 1, 1};

    for (int tile = slice * WAVES + wave; tile < numTiles; tile += numSlices * WAVES)
    {
        const f16* aTile = adjPre + static_cast<long long>(tile) * (COUT * TILE_POINTS);
        const f16* bTile = input + static_cast<long long>(tile) * (CIN * TILE_POINTS);
#pragma unroll
        for (int kb = 0; kb < TILE_POINTS / 32; ++kb) {
            f16x8 b[KI_CHUNK];
#pragma unroll
            for (int mi = 0; mi < KI_CHUNK; ++mi) {
                const int channel = 16 * (ki0 + mi) + r;
                const f16x8 raw = *reinterpret_cast<const f16x8*>(bTile + channel * TILE_POINTS + 32 * kb + 8 * g);
                b[mi] = activationForwardChannel<InputActivation>(raw, channel);
            }
#pragma unroll
            for (int mo = 0; mo < MO_CHUNK; ++mo) {
                const f16x8 a = *reinterpret_cast<const f16x8*>(aTile + (16 * (mo0 + mo) + r) * TILE_POINTS + 32 * kb + 8 * g);
#pragma unroll
                for (int mi = 0; mi < KI_CHUNK; ++mi) acc[mo][mi] = mfma32(a, b[mi], acc[mo][mi]);
                // every block sums the bias gradient (a branch here would split the loop body);
                // only the blocks of the first input chunk store it
                if constexpr (BIAS) accBias[mo] = mfma32(a, ones, accBias[mo]);
            }
        }
    }

    // combine the waves of the workgroup through LDS, then store the slice's partial sums
    extern __shared__ __align__(16) unsigned char sMemory[];
    float* sAcc = reinterpret_cast<float*>(sMemory);   // (MO_CHUNK*KI_CHUNK + MO_CHUNK) tiles of 256 floats
    constexpr int TILES = MO_CHUNK * KI_CHUNK + (BIAS ? MO_CHUNK : 0);
    for (int i = threadIdx.x; i < TILES * 256; i += blockDim.x) sAcc[i] = 0.f;
    __syncthreads();
    // one wave after the other, so that the sum has the same rounding in every run
    for (int w = 0; w < WAVES; ++w) {
        if (wave == w) {
#pragma unroll
            for (int mo = 0; mo < MO_CHUNK; ++mo) {
#pragma unroll
                for (int mi = 0; mi < KI_CHUNK; ++mi)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        sAcc[(mo * KI_CHUNK + mi) * 256 + (4 * g + i) * 16 + r] += acc[mo][mi][i];
                if constexpr (BIAS) {
                    if (ownsBias && r == 0) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) sAcc[(MO_CHUNK * KI_CHUNK + mo) * 256 + 4 * g + i] += accBias[mo][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    for (int e = threadIdx.x; e < MO_CHUNK * KI_CHUNK * 256; e += blockDim.x) {
        const int t = e >> 8, within = e & 255;
        const int mo = t / KI_CHUNK, mi = t - mo * KI_CHUNK;
        const int row = 16 * (mo0 + mo) + (within >> 4), col = 16 * (ki0 + mi) + (within & 15);
        partialWeights[static_cast<long long>(slice) * sliceStride + row * CIN + col] = sAcc[e];
    }
    if constexpr (BIAS) {
        if (ownsBias) {
            for (int e = threadIdx.x; e < MO_CHUNK * 16; e += blockDim.x) {
                const int mo = e >> 4;
                partialBias[static_cast<long long>(slice) * sliceStride + 16 * (mo0 + mo) + (e & 15)]
                    = sAcc[(MO_CHUNK * KI_CHUNK + mo) * 256 + (e & 15)];
            }
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
