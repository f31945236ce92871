// Template of the fused adjoint kernel. The host code generator replaces everything
// in $$..$$ before the source is handed to the runtime compiler.
//
// Per 64-point wavefront tile: dL/dy is loaded straight into the accumulator layout
// of the matrix cores, each layer (last to first) applies the activation adjoint on
// the stored pre-activations and contracts with the transposed weights
// (dX = W^T dpre, the same MFMA path as the forward pass with the weight tiles
// staged transposed). For the weight gradients dpre is either stored for the weight-update
// kernels or, where the gradient tiles of all layers fit into the registers of a wavefront,
// contracted with the layer input right here (Layer::weightGradient), the workgroup storing
// its partial sums after its last tile. Where all layers are summed here, the training pass may
// have kept the encoded input only: the kernel then runs the layers forward once more per tile
// (Layer::forwardKeep) instead of reading their pre-activations back. The adjoint of
// the encoded input finally goes through the LDS staging rows to one lane per point,
// which accumulates input gradients and scatter-adds grid gradients with hardware
// fp32 atomics.
//
// Replaces NetworkKernelBackward of the reference
// (src_cpp/include/qmlp/kernels/network_backward.cuh:33-114). Unlike the reference it
// never reads dL/dy beyond the real output channels: padded channels are zero.

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/arrays.h>
#include <qmlp/kernels/layer.h>

$$INCLUDES$$

QUICKMLP_KERNEL_NAMESPACE_BEGIN

namespace activations
{
$$DEFINE_ACTIVATIONS$$
    // stands for "no activation": the stored input of the first layer is its input
    struct passthrough_
    {
        static __device__ __forceinline__ half forward(half x) { return x; }
    };
}

/**
 * dst (cin, cout) row-major = transpose of src (cout, cin) row-major. Run before the adjoint
 * kernel for layers whose weights are too large to stay in LDS: the adjoint kernel then reads
 * its matrix-core operands (rows of W^T) from global memory with two 8-byte loads per lane.
 */
__global__ void __launch_bounds__(256) TransposeWeightsKernel(const half* __restrict__ src, half* __restrict__ dst,
                                                              int cout, int cin)
{
    __shared__ half tile[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int tilesX = cin / 16;
    for (int t = blockIdx.x; t < tilesX * (cout / 16); t += gridDim.x) {
        const int o0 = (t / tilesX) * 16, k0 = (t % tilesX) * 16;
        tile[ty][tx] = src[(o0 + ty) * cin + k0 + tx];
        __syncthreads();
        dst[(k0 + ty) * cout + o0 + tx] = tile[tx][ty];
        __syncthreads();
    }
}

__global__ void __launch_bounds__($$BLOCK_SIZE$$) $$KERNEL_ATTRIBUTES$$ NetworkKernelBackward(
    int numel,
    const Tensor2Read<float> inputs,      //shape (numel, Cin)
    const Tensor2Read<float> adjOutputs,  //shape (numel, Cout)
    Tensor2RW<float> adjInputs,           //shape (numel, Cin), accumulated; unused without input gradients
    const half* __restrict__ networkParametersH,
    const half* __restrict__ forwardTmpMemoryH,  //written by the forward kernel
    half* __restrict__ adjointTmpMemoryH,        //receives dpre if weight gradients are requested
    const half* __restrict__ transposedWeightsH, //W^T of the layers whose weights do not stay in LDS, or nullptr
    float* __restrict__ partialGradients,        //FUSED_WEIGHT_UPDATE: partialSlices x the layout of the parameters; workgroup b
    int partialSlices                            //stores the sums of its tiles into slice b (and zeroes slices b + k * gridDim.x)
#if $$HAS_OUTPUT_ORDER$$
    // Networks whose batches may train in sorted order: nullptr, or (numel) the row of adjOutputs that belongs to
    // point p. The parameter and its code exist only in the kernels of such networks: with them the run-time compiler
    // scheduled the kernel of 64 -> 64 x 4 -> 4 (which never sorts) so that it took 689 instead of 372 us.
    , const int* __restrict__ adjOutputOrder
#endif
    $$ENCODING_PARAMETERS$$)
{
    constexpr int NUM_INPUTS = $$NUM_INPUTS$$;
    constexpr int ENCODED_CHANNELS = $$ENCODED_CHANNELS$$;
    constexpr int CHANNELS_IN = $$CHANNELS_IN$$;
    constexpr int CHANNELS_OUT = $$CHANNELS_OUT$$;
    constexpr int KT0 = CHANNELS_IN / 16;
    constexpr int MTL = CHANNELS_OUT / 16;
    constexpr int STAGE_STRIDE = CHANNELS_IN + 8;
    constexpr int LDS_PARAM_HALVES = $$LDS_PARAM_HALVES$$;
    constexpr int WAVES = $$BLOCK_SIZE$$ / WAVE_SIZE;
    constexpr bool HAS_INPUT_GRADIENTS = $$HAS_INPUT_GRADIENTS$$;
    constexpr bool HAS_NETWORK_GRADIENTS = $$HAS_NETWORK_GRADIENTS$$;
    constexpr bool HAS_ENCODING_GRADIENTS = $$HAS_ENCODING_GRADIENTS$$;
    // Some layers' weights are staged into a shared LDS buffer right before the layer runs:
    // the wavefronts of the workgroup then walk the tiles and layers in lockstep (workgroup
    // barriers inside the loop), wavefronts without a tile work on zeros.
    constexpr bool HAS_STREAMED_LAYERS = $$HAS_STREAMED_LAYERS$$;
    // the adjoint of the encoded input is only needed if something sits behind it
    constexpr bool NEEDS_ENCODING_ADJOINT = $$NEEDS_ENCODING_ADJOINT$$;
    // true: the adjoint of the encoded rows is stored (channel-major per tile, behind the adjoint
    // pre-activations) for the kernels that sum the parameter gradients of grids slice by slice
    constexpr bool STORE_ENCODED_ADJOINT = $$STORE_ENCODED_ADJOINT$$;
    constexpr int OFFSET_ENCODED_ADJOINT = $$OFFSET_ENCODED_ADJOINT$$;   // channels in front of that region
    // false: nothing in this kernel reads the adjoint of an encoded row point by point
    constexpr bool NEEDS_STAGED_ADJOINT = $$NEEDS_STAGED_ADJOINT$$;
    // true: the weight gradients are summed in this kernel and dpre is not stored
    constexpr bool FUSED_WEIGHT_UPDATE = $$FUSED_WEIGHT_UPDATE$$;
    constexpr bool STORE_DPRE = HAS_NETWORK_GRADIENTS;   // of the layers that have a weight-update kernel
    (void)FUSED_WEIGHT_UPDATE;
    constexpr int NUM_PARAMETERS = $$NUM_PARAMETERS$$;
    (void)STORE_DPRE; (void)NUM_PARAMETERS;
    (void)ENCODED_CHANNELS; (void)NUM_INPUTS; (void)KT0; (void)STAGE_STRIDE;

    const f16* __restrict__ networkParameters = reinterpret_cast<const f16*>(networkParametersH);
    const f16* __restrict__ forwardTmpMemory = reinterpret_cast<const f16*>(forwardTmpMemoryH);
    f16* __restrict__ adjointTmpMemory = reinterpret_cast<f16*>(adjointTmpMemoryH);
    const f16* __restrict__ transposedWeights = reinterpret_cast<const f16*>(transposedWeightsH);
    (void)transposedWeights;

    extern __shared__ __align__(16) unsigned char sMemory[];
    f16* sParams = reinterpret_cast<f16*>(sMemory);
    const int wave = threadIdx.x / WAVE_SIZE;
    const int lane = threadIdx.x % WAVE_SIZE;
    const int g = lane >> 4, r = lane & 15;
    f16* sStage = sParams + LDS_PARAM_HALVES + wave * (TILE_POINTS * STAGE_STRIDE);
    (void)sStage;
    // FUSED_WEIGHT_UPDATE: this wavefront's tile of adjoint pre-activations, a row of 64 points per channel
    f16* sTranspose = reinterpret_cast<f16*>(sMemory + $$OFFSET_TRANSPOSE$$) + wave * $$TRANSPOSE_HALVES$$;
    (void)sTranspose;
    // RECOMPUTE: behind it, this wavefront's tile of the input of the layer whose weight gradients are being summed
    f16* sLayerInput = sTranspose + $$LAYER_INPUT_OFFSET$$;
    (void)sLayerInput;

    // stage the transposed weights in operand order
$$STAGE_PARAMETERS$$
    // FUSED_WEIGHT_UPDATE: the gradient tiles of this wavefront, summed over its tiles of the batch
$$DECLARE_WEIGHT_GRADIENTS$$
    // gradients of coarse grid levels are summed in LDS first (zeroed here, added to the
    // gradient tensor once per workgroup after the loop over the tiles)
$$ZERO_LDS_GRADIENTS$$
    __syncthreads();

    const int numTiles = (numel + TILE_POINTS - 1) / TILE_POINTS;
    const long long numel64 = static_cast<long long>(numTiles) * TILE_POINTS;
    const int actualChannelsOut = adjOutputs.sizes_[1];
    const bool adjOutputRowsOfFloat2 = actualChannelsOut == 2 && adjOutputs.strides_[1] == 1 && adjOutputs.strides_[0] % 2 == 0
        && reinterpret_cast<unsigned long long>(adjOutputs.data_) % 8 == 0;
    const bool adjOutputRowsOfFloat4 = actualChannelsOut % 4 == 0 && adjOutputs.strides_[1] == 1 && adjOutputs.strides_[0] % 4 == 0
        && reinterpret_cast<unsigned long long>(adjOutputs.data_) % 16 == 0;
#if $$HAS_OUTPUT_ORDER$$
    // a batch that trains in sorted order: the rows of dL/dy of this wavefront's next tile, asked for one tile ahead
    int adjRowAhead[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int p = (static_cast<int>(blockIdx.x) * WAVES + wave) * TILE_POINTS + 4 * r + nt;
        adjRowAhead[nt] = (adjOutputOrder && p < numel) ? adjOutputOrder[p] : p;
    }
#endif
    for (int tileBase = blockIdx.x * WAVES; tileBase < numTiles; tileBase += gridDim.x * WAVES)
    {
        const int tile = tileBase + wave;
        if (!HAS_STREAMED_LAYERS && tile >= numTiles) continue;
        const bool tileValid = tile < numTiles;
        const int tileRead = tileValid ? tile : numTiles - 1;   // stored intermediates are read from a valid tile
        (void)tileRead;
        // dL/dy -> accumulator layout (fp32 -> fp16), zero outside batch / real channels
        f16x4 dyOut[NT][MTL];
        int validMask = 0;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int p = tile * TILE_POINTS + 4 * r + nt;
            const bool pv = p < numel;
            validMask |= pv ? (1 << nt) : 0;
#if $$HAS_OUTPUT_ORDER$$
            const long long adjRow = adjRowAhead[nt];
            {
                const long long ahead = static_cast<long long>(p) + static_cast<long long>(gridDim.x) * (WAVES * TILE_POINTS);
                adjRowAhead[nt] = (adjOutputOrder && ahead < numel) ? adjOutputOrder[ahead] : static_cast<int>(ahead < numel ? ahead : 0);
            }
#else
            const long long adjRow = p;
#endif
            if (adjOutputRowsOfFloat2 || adjOutputRowsOfFloat4) {
                // channels side by side in memory: four per load (a lane holds channels
                // 16m+4g .. +3 of its points), a row of two channels as one 8-byte load
                const float* row = adjOutputs.data_ + adjRow * adjOutputs.strides_[0];
#pragma unroll
                for (int m = 0; m < MTL; ++m) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) dyOut[nt][m][i] = static_cast<f16>(0);
                    const int c = 16 * m + 4 * g;
                    if (adjOutputRowsOfFloat4 && pv && c < actualChannelsOut) {
                        const float4 v = *reinterpret_cast<const float4*>(row + c);
                        dyOut[nt][m][0] = static_cast<f16>(v.x);
                        dyOut[nt][m][1] = static_cast<f16>(v.y);
                        dyOut[nt][m][2] = static_cast<f16>(v.z);
                        dyOut[nt][m][3] = static_cast<f16>(v.w);
                    }
                }
                if (!adjOutputRowsOfFloat4 && pv && g == 0) {
                    const float2 v = *reinterpret_cast<const float2*>(row);
                    dyOut[nt][0][0] = static_cast<f16>(v.x);
                    dyOut[nt][0][1] = static_cast<f16>(v.y);
                }
            } else {
#pragma unroll
                for (int m = 0; m < MTL; ++m)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int c = 16 * m + 4 * g + i;
                        float v = 0.f;
                        if (pv && c < actualChannelsOut)
                            v = adjOutputs.data_[adjRow * adjOutputs.strides_[0]
                                                 + static_cast<long long>(c) * adjOutputs.strides_[1]];
                        dyOut[nt][m][i] = static_cast<f16>(v);
                    }
            }
        }

        // RECOMPUTE: the training pass kept the encoded input only; the layers run again, their pre-activations stay in registers
$$RECOMPUTE_FORWARD$$
        // layers, last to first
$$CALL_NETWORK_LAYERS$$

        if constexpr (STORE_ENCODED_ADJOINT) {
            if (tileValid) {
                f16* adjTile = adjointTmpMemory + (static_cast<long long>(OFFSET_ENCODED_ADJOINT) * numel64
                                                   + static_cast<long long>(tile) * (CHANNELS_IN * TILE_POINTS));
#pragma unroll
                for (int t = 0; t < KT0; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const f16x4 v = {dxIn[0][t][i], dxIn[1][t][i], dxIn[2][t][i], dxIn[3][t][i]};
                        *reinterpret_cast<f16x4*>(adjTile + (16 * t + 4 * g + i) * TILE_POINTS + 4 * r) = v;
                    }
            }
        }
        if constexpr (NEEDS_ENCODING_ADJOINT && NEEDS_STAGED_ADJOINT) {
            // adjoint of the encoded input: registers -> one staging row per point
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int t = 0; t < KT0; ++t)
                    *reinterpret_cast<f16x4*>(sStage + (16 * nt + r) * STAGE_STRIDE + 16 * t + 4 * g) = dxIn[nt][t];
            waveLdsSync();

            const int index = tile * TILE_POINTS + lane;
            if (index < numel) {
                StaticArray<float, NUM_INPUTS> encodingInput;
#pragma unroll
                for (int i = 0; i < NUM_INPUTS; ++i)
                    encodingInput[i] = inputs.data_[static_cast<long long>(index) * inputs.strides_[0]
                                                    + static_cast<long long>(i) * inputs.strides_[1]];
                StaticArray<float, NUM_INPUTS> adjEncodingInput;
#pragma unroll
                for (int i = 0; i < NUM_INPUTS; ++i) adjEncodingInput[i] = 0.f;
                WrappedArray<const f16> adjEncodingOutput{sStage + stageRow(lane) * STAGE_STRIDE};

$$CALL_ENCODINGS$$

                if constexpr (HAS_INPUT_GRADIENTS) {
                    float* adjRow = adjInputs.data_ + static_cast<long long>(index) * adjInputs.strides_[0];
                    if (!HAS_ENCODING_GRADIENTS && NUM_INPUTS % 4 == 0 && adjInputs.strides_[1] == 1 && adjInputs.strides_[0] % 4 == 0
                        && reinterpret_cast<unsigned long long>(adjInputs.data_) % 16 == 0) {
                        // the channels of a row side by side: four per load and store. Kept to
                        // kernels without a grid scatter: in front of the gradient atomics of a grid
                        // no gain was measurable.
#pragma unroll
                        for (int i = 0; i + 3 < NUM_INPUTS; i += 4) {
                            float4 v = *reinterpret_cast<float4*>(adjRow + i);
                            v.x += adjEncodingInput[i];
                            v.y += adjEncodingInput[i + 1];
                            v.z += adjEncodingInput[i + 2];
                            v.w += adjEncodingInput[i + 3];
                            *reinterpret_cast<float4*>(adjRow + i) = v;
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < NUM_INPUTS; ++i)
                            adjRow[static_cast<long long>(i) * adjInputs.strides_[1]] += adjEncodingInput[i];
                    }
                }
            }

            // parameter gradients of the grid encodings, scattered by the whole wavefront
$$CALL_ENCODING_SCATTER$$
            waveLdsSync();
        }
    }
$$FLUSH_LDS_GRADIENTS$$
$$STORE_WEIGHT_GRADIENTS$$
}

QUICKMLP_KERNEL_NAMESPACE_END
