// Template of the fused forward / inference kernel. The host code generator replaces
// everything in $$..$$ before the source is handed to the runtime compiler.
//
// One wavefront owns groups of PPL tiles of 64 points: each lane first evaluates all
// input encodings of one point of every tile into rows of the wave's LDS staging area
// (fp16; the grid encodings go level by level over the PPL points, which keeps many
// gathers in flight and lets all waves of the device sweep the level tables together),
// then the wave reads the rows of one tile after the other back as matrix-core B
// operands and runs every layer with the activations kept in registers. Weights (and biases) are staged into LDS once per
// workgroup, already permuted into operand order.
//
// Replaces NetworkKernelInferenceAndForward of the reference
// (src_cpp/include/qmlp/kernels/network_forward.cuh:34-114).

#include <qmlp/kernels/common.h>
#include <qmlp/kernels/arrays.h>
#include <qmlp/kernels/layer.h>

$$INCLUDES$$

QUICKMLP_KERNEL_NAMESPACE_BEGIN

namespace activations
{
$$DEFINE_ACTIVATIONS$$
}

/** Points the staging rows of the PPL points of a lane at the wave's LDS staging tiles. */
template <typename T, int C, int PPL>
__device__ __forceinline__ void bindEncodingRow(StageRowArray<T, C> (&rows)[PPL], T* stage, int q, int lane)
{
    rows[q].row_ = stage + (q * TILE_POINTS + stageRow(lane)) * StageLayout<C>::Stride;
    rows[q].rotation_ = StageLayout<C>::rotation(stageRow(lane));
    rows[q].offset_ = 0;
}
template <typename T, int PPL, int C, int OFFSET>
__device__ __forceinline__ void bindEncodingRow(PackedRegisterRowsView<T, PPL, C, OFFSET>&, T*, int, int)
{
}

/**
 * \tparam STORE false: inference. true: additionally stores, per 64-point tile and
 *   channel-major, the encoded network input and the pre-activations of every layer
 *   into forwardTmpMemory for the adjoint pass.
 * \tparam DERIVATIVES with STORE: grid encodings additionally store, behind these regions, the derivatives of
 *   their features with respect to the position (PositionDerivativeLayout), from which the adjoint pass forms
 *   the input gradients without a second gather.
 */
template <bool STORE, bool DERIVATIVES = false>
__global__ void __launch_bounds__($$BLOCK_SIZE$$) $$KERNEL_ATTRIBUTES$$ NetworkKernelInferenceAndForward(
    int numel,
    const Tensor2Read<float> inputs,  //shape (numel, Cin)
    Tensor2RW<float> outputs,         //shape (numel, Cout)
    const half* __restrict__ networkParametersH,
    half* __restrict__ forwardTmpMemoryH,
    int tmpTileOffset,                // STORE: index of this launch's first tile in the whole batch
    int tmpNumTiles,                  // STORE: tiles of the whole batch (a batch may be cut into several launches)
    const int* __restrict__ pointOrder  // null, or per row of inputs the row of outputs it belongs to (inputs sorted by grid slab)
    $$ENCODING_PARAMETERS$$)
{
    constexpr int NUM_INPUTS = $$NUM_INPUTS$$;            // raw input channels
    constexpr int ENCODED_CHANNELS = $$ENCODED_CHANNELS$$;  // sum of encoding outputs
    constexpr int CHANNELS_IN = $$CHANNELS_IN$$;          // padded to a multiple of 16
    constexpr int CHANNELS_OUT = $$CHANNELS_OUT$$;        // padded width of the last layer
    constexpr int KT0 = CHANNELS_IN / 16;
    constexpr int MTL = CHANNELS_OUT / 16;
    typedef StageLayout<CHANNELS_IN> Stage;               // padded or rotated rows, see arrays.h
    constexpr int STAGE_STRIDE = Stage::Stride;           // halves
    constexpr int LDS_PARAM_HALVES = $$LDS_PARAM_HALVES$$;
    constexpr int WAVES = $$BLOCK_SIZE$$ / WAVE_SIZE;
    constexpr int PPL = $$POINTS_PER_LANE$$;              // tiles a wave encodes together
    // true: the encoded rows of the PPL tiles wait in registers and go through one LDS staging
    // tile per wave, one after the other (the register file holds more points than the LDS);
    // false: every tile has its own staging rows in LDS
    constexpr bool REGISTER_STAGING = $$REGISTER_STAGING$$;
    constexpr int STAGED_TILES = REGISTER_STAGING ? 1 : PPL;
    // Some layers' weights are staged into a shared LDS buffer right before the layer runs:
    // the wavefronts of the workgroup then walk the tiles and layers in lockstep (workgroup
    // barriers inside the loops), wavefronts without a tile compute on zero rows.
    constexpr bool HAS_STREAMED_LAYERS = $$HAS_STREAMED_LAYERS$$;
    // >= 0: the only encoding is an identity encoding of the input channels from this one on.
    // Lanes then load their matrix-core operands (4 consecutive channels of 4 points) straight
    // from the input rows, and nothing goes through the LDS staging rows.
    constexpr int DIRECT_INPUT_START = $$DIRECT_INPUT_START$$;
    constexpr bool DIRECT_INPUT = DIRECT_INPUT_START >= 0;
    static_assert(!DIRECT_INPUT || PPL == 1, "direct input rows: one tile per wave");

    const f16* __restrict__ networkParameters = reinterpret_cast<const f16*>(networkParametersH);
    f16* __restrict__ forwardTmpMemory = reinterpret_cast<f16*>(forwardTmpMemoryH);

    extern __shared__ __align__(16) unsigned char sMemory[];
    f16* sParams = reinterpret_cast<f16*>(sMemory);
    const int wave = threadIdx.x / WAVE_SIZE;
    const int lane = threadIdx.x % WAVE_SIZE;
    const int g = lane >> 4, r = lane & 15;
    f16* sStage = sParams + LDS_PARAM_HALVES + wave * (STAGED_TILES * TILE_POINTS * STAGE_STRIDE);
    (void)sStage;

    // stage the weights in operand order, then the biases
$$STAGE_PARAMETERS$$
    __syncthreads();

    const int numTiles = (numel + TILE_POINTS - 1) / TILE_POINTS;
    constexpr int INPUT_VECTOR = NUM_INPUTS % 4 == 0 ? 4 : 2;   // floats per load
    const bool inputRowsAreVectors = inputs.strides_[1] == 1 && inputs.strides_[0] % INPUT_VECTOR == 0
        && reinterpret_cast<unsigned long long>(inputs.data_) % (INPUT_VECTOR * sizeof(float)) == 0;
    (void)inputRowsAreVectors;
    // the regions of the temporary memory are laid out for the whole batch
    const long long numel64 = static_cast<long long>(tmpNumTiles) * TILE_POINTS;
    (void)numel64;
    for (int tileBase = blockIdx.x * WAVES * PPL; tileBase < numTiles; tileBase += gridDim.x * WAVES * PPL)
    {
        const int tile0 = tileBase + wave * PPL;
        if (!HAS_STREAMED_LAYERS && tile0 >= numTiles) continue;

        // encodings: PPL points per lane (one of each tile), each into its staging row.
        // Rows outside the batch are evaluated at the origin and zeroed afterwards so that
        // no NaN enters the matrix cores.
        PackedRegisterRows<f16, REGISTER_STAGING ? PPL : 1, CHANNELS_IN> encodedRegisters = {};   // halves are merged into it
        (void)encodedRegisters;
        if constexpr (!DIRECT_INPUT) {
            StaticArray<float, NUM_INPUTS> encodingInput[PPL];
            $$ENCODING_OUTPUT_ROWS$$
            bool valid[PPL];
#pragma unroll
            for (int q = 0; q < PPL; ++q) {
                const int index = (tile0 + q) * TILE_POINTS + lane;
                valid[q] = index < numel;
                bindEncodingRow(encodingOutput, sStage, q, lane);
                const float* inputRow = inputs.data_ + static_cast<long long>(index) * inputs.strides_[0];
                if ((NUM_INPUTS == 2 || NUM_INPUTS % 4 == 0) && inputRowsAreVectors) {
                    // the channels of a row lie side by side: 16 (or 8) bytes per load
                    if (NUM_INPUTS % 4 == 0) {
#pragma unroll
                        for (int i = 0; i + 3 < NUM_INPUTS; i += 4) {
                            const float4 v = valid[q] ? *reinterpret_cast<const float4*>(inputRow + i) : make_float4(0.f, 0.f, 0.f, 0.f);
                            encodingInput[q][i] = v.x;
                            encodingInput[q][i + 1] = v.y;
                            encodingInput[q][i + 2] = v.z;
                            encodingInput[q][i + 3] = v.w;
                        }
                    } else {
                        const float2 v = valid[q] ? *reinterpret_cast<const float2*>(inputRow) : make_float2(0.f, 0.f);
                        encodingInput[q][0] = v.x;
                        encodingInput[q][NUM_INPUTS > 1 ? 1 : 0] = v.y;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NUM_INPUTS; ++i)
                        encodingInput[q][i] = valid[q] ? inputRow[static_cast<long long>(i) * inputs.strides_[1]] : 0.f;
                }
            }
$$CALL_ENCODINGS$$
#pragma unroll
            for (int q = 0; q < PPL; ++q) {
#pragma unroll
                for (int c = ENCODED_CHANNELS; c < CHANNELS_IN; ++c) encodingOutput[q][c] = static_cast<f16>(0);
                if (!valid[q]) {
#pragma unroll
                    for (int c = 0; c < ENCODED_CHANNELS; ++c) encodingOutput[q][c] = static_cast<f16>(0);
                }
            }
            waveLdsSync();
        }

$$TILE_LOOP_PRAGMA$$
        for (int q = 0; q < PPL; ++q)
        {
        const int tile = tile0 + q;
        if (!HAS_STREAMED_LAYERS && tile >= numTiles) break;
        const bool tileValid = tile < numTiles;
        const int tmpTile = tile + tmpTileOffset;
        (void)tmpTile;
        const f16* sTile = sStage + (REGISTER_STAGING ? 0 : q) * (TILE_POINTS * STAGE_STRIDE);
        (void)sTile;
        if (REGISTER_STAGING) {
            // the lane's row of this tile: registers -> staging row, 8 bytes at a time
            if (q > 0) waveLdsSync();   // the operands of the previous tile have been read
#pragma unroll
            for (int chunk = 0; chunk < CHANNELS_IN / 4; ++chunk) {
                typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
                const u32x2 v = {encodedRegisters.data_[REGISTER_STAGING ? q : 0][2 * chunk],
                                 encodedRegisters.data_[REGISTER_STAGING ? q : 0][2 * chunk + 1]};
                *reinterpret_cast<u32x2*>(sStage + Stage::chunkOffset(stageRow(lane), chunk)) = v;
            }
            waveLdsSync();
        }

        // B operands of the first layer
        f16x4 x0[NT][KT0];
        if constexpr (DIRECT_INPUT) {
            const bool rowsOfFloat4 = DIRECT_INPUT_START % 4 == 0 && inputs.strides_[1] == 1 && inputs.strides_[0] % 4 == 0
                && reinterpret_cast<unsigned long long>(inputs.data_) % 16 == 0;
            const float* row0 = inputs.data_ + static_cast<long long>(tile * TILE_POINTS + 4 * r) * inputs.strides_[0]
                + static_cast<long long>(DIRECT_INPUT_START) * inputs.strides_[1];
            if (rowsOfFloat4 && (tile + 1) * TILE_POINTS <= numel) {
                // a whole tile of rows whose channels lie side by side: nothing is predicated
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float* row = row0 + static_cast<long long>(nt) * inputs.strides_[0];
#pragma unroll
                    for (int t = 0; t < KT0; ++t) {
                        const int c = 16 * t + 4 * g;   // first of this lane's four encoded channels
                        f32x4 v = {0.f, 0.f, 0.f, 0.f};
                        if (16 * t + 15 < ENCODED_CHANNELS) {
                            v = *reinterpret_cast<const f32x4*>(row + c);
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (c + i < ENCODED_CHANNELS) v[i] = row[c + i];
                        }
                        x0[nt][t] = toF16(v);
                    }
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const bool pv = tile * TILE_POINTS + 4 * r + nt < numel;
                    const float* row = row0 + static_cast<long long>(nt) * inputs.strides_[0];
#pragma unroll
                    for (int t = 0; t < KT0; ++t) {
                        const int c = 16 * t + 4 * g;
                        f32x4 v = {0.f, 0.f, 0.f, 0.f};
                        if (16 * t + 15 < ENCODED_CHANNELS && rowsOfFloat4) {
                            if (pv) v = *reinterpret_cast<const f32x4*>(row + c);
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (pv && c + i < ENCODED_CHANNELS) v[i] = row[static_cast<long long>(c + i) * inputs.strides_[1]];
                        }
                        x0[nt][t] = toF16(v);
                    }
                }
            }
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int t = 0; t < KT0; ++t)
                    x0[nt][t] = *reinterpret_cast<const f16x4*>(sTile + Stage::chunkOffset(16 * nt + r, 4 * t + g));
        }

        if (STORE && tileValid) {
            // encoded input, channel-major per tile, for the weight update of layer 0
            f16* encTile = forwardTmpMemory + static_cast<long long>(tmpTile) * (CHANNELS_IN * TILE_POINTS);
#pragma unroll
            for (int t = 0; t < KT0; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f16x4 v = {x0[0][t][i], x0[1][t][i], x0[2][t][i], x0[3][t][i]};
                    *reinterpret_cast<f16x4*>(encTile + (16 * t + 4 * g + i) * TILE_POINTS + 4 * r) = v;
                }
        }

        // layers
$$CALL_NETWORK_LAYERS$$

        // output: lane holds channels 16m+4g+i of the points 4r+nt
        const int actualChannelsOut = outputs.sizes_[1];
        long long outputRow[NT];   // -1: outside the batch
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int p = tile * TILE_POINTS + 4 * r + nt;
            outputRow[nt] = p < numel ? (pointOrder ? pointOrder[p] : p) : -1;
        }
        // output channels that lie side by side in memory leave four at a time (a lane holds
        // channels 16m+4g .. +3 of its points), rows of two channels as one 8-byte store
        const bool rowsOfFloat2 = actualChannelsOut == 2 && outputs.strides_[1] == 1 && outputs.strides_[0] % 2 == 0
            && reinterpret_cast<unsigned long long>(outputs.data_) % 8 == 0;
        const bool rowsOfFloat4 = actualChannelsOut % 4 == 0 && outputs.strides_[1] == 1 && outputs.strides_[0] % 4 == 0
            && reinterpret_cast<unsigned long long>(outputs.data_) % 16 == 0;
        if (rowsOfFloat4) {
#pragma unroll
            for (int m = 0; m < MTL; ++m) {
                const int c = 16 * m + 4 * g;
                if (c >= actualChannelsOut) continue;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    if (outputRow[nt] < 0) continue;
                    *reinterpret_cast<float4*>(outputs.data_ + outputRow[nt] * outputs.strides_[0] + c) =
                        make_float4(static_cast<float>(xOut[nt][m][0]), static_cast<float>(xOut[nt][m][1]),
                                    static_cast<float>(xOut[nt][m][2]), static_cast<float>(xOut[nt][m][3]));
                }
            }
        } else if (rowsOfFloat2) {
            if (g == 0) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    if (outputRow[nt] < 0) continue;
                    *reinterpret_cast<float2*>(outputs.data_ + outputRow[nt] * outputs.strides_[0]) =
                        make_float2(static_cast<float>(xOut[nt][0][0]), static_cast<float>(xOut[nt][0][1]));
                }
            }
        } else {
#pragma unroll
            for (int m = 0; m < MTL; ++m)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int c = 16 * m + 4 * g + i;
                    if (c < actualChannelsOut) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) {
                            if (outputRow[nt] >= 0)
                                outputs.data_[outputRow[nt] * outputs.strides_[0] + static_cast<long long>(c) * outputs.strides_[1]]
                                    = static_cast<float>(xOut[nt][m][i]);
                        }
                    }
                }
        }
        }
        if constexpr (!DIRECT_INPUT) waveLdsSync();   // the staging rows are overwritten by the next group of tiles
    }
}

QUICKMLP_KERNEL_NAMESPACE_END
