#pragma once
// One fully-connected layer of the fused network on a 64-point wavefront tile.
//
// Every layer is the contraction  Y^T (C_out x points) = W (C_out x C_in) * X^T (C_in x points)
// on the matrix cores: A = a 16-row tile of W, B = activations of 16 points,
// fp16 operands, fp32 accumulation (v_mfma_f32_16x16x32_f16; an odd trailing
// 16-channel tile is paired with a zero tile). The accumulator layout (lane 16g+r
// holds channels 4g..4g+3 of point column r) is exactly the layout the next
// layer's B operand needs once the contraction index is permuted accordingly: a
// k-block of 32 channels built from the 16-channel tiles t0,t1 assigns to lane
// group g the channels 16*t0+4g+{0..3} and 16*t1+4g+{0..3}. Because only the
// weights have to follow that permutation (done once while staging them into LDS),
// activations stay in registers from the first to the last layer.
//
// Only one MFMA shape is used on purpose: with the ROCm 7.2 compiler at -O3, a
// v_mfma_f32_16x16x16_f16 accumulating onto the result of the v_mfma_f32_16x16x32_f16
// issued right before it was observed to deliver wrong accumulator elements 0 and 1
// on gfx950 (fewer of them when MFMAs were padded with wait states).
//
// Replaces Layer<...>::inference / ::adjoint of the reference
// (src_cpp/include/qmlp/kernels/layer.cuh:86-266), which round-trips the activations
// through shared memory between layers and accumulates in half precision.

#include <qmlp/kernels/common.h>

QUICKMLP_KERNEL_NAMESPACE_BEGIN

__device__ __forceinline__ f32x4 mfma32(f16x8 a, f16x8 b, f32x4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

template <int A>
__device__ __forceinline__ void zeroTiles(f32x4 (&acc)[A])
{
#pragma unroll
    for (int a = 0; a < A; ++a) acc[a] = f32x4{0.f, 0.f, 0.f, 0.f};
}

template <int A, int B>
__device__ __forceinline__ void zeroTiles(f32x4 (&acc)[A][B])
{
#pragma unroll
    for (int a = 0; a < A; ++a) zeroTiles(acc[a]);
}

/**
 * \tparam CIN padded input channels (multiple of 16)
 * \tparam COUT padded output channels (multiple of 16)
 * \tparam BIAS layer has a bias vector
 * \tparam Activation struct with static half forward(half), half adjoint(half x, half adjz), or a
 *         per-channel composite with forwardAt(half, channel), adjointAt(half x, half adjz, channel)
 */
template <int CIN, int COUT, bool BIAS, typename Activation>
struct Layer
{
    static constexpr int KT = CIN / 16;     // 16-channel tiles of the input
    static constexpr int MT = COUT / 16;    // 16-channel tiles of the output
    // forward operand order: per output tile m, ceil(KT/2) blocks of 64 lanes x 8 halves;
    // if KT is odd the upper 4 halves of the last block are zero
    static constexpr int F_KB = (KT + 1) / 2;
    static constexpr int F_MSTRIDE = F_KB * 512;
    static constexpr int F_LDS_HALVES = MT * F_MSTRIDE;
    // adjoint (transposed) operand order: per input tile, ceil(MT/2) blocks
    static constexpr int A_KB = (MT + 1) / 2;
    static constexpr int A_MSTRIDE = A_KB * 512;
    static constexpr int A_LDS_HALVES = KT * A_MSTRIDE;

    /**
     * Copies the row-major (COUT, CIN) weight matrix into LDS in forward operand order.
     * Called by all threads of the block; 'W' must be 16-byte aligned. The matrix is read in
     * memory order with 16-byte loads, four of them in flight per thread (layers that are
     * streamed through LDS are staged once per group of tiles, so this is on the critical
     * path there), and scattered into the operand layout.
     */
    __device__ static void stageForward(const f16* __restrict__ W, f16* __restrict__ dst, int tid, int nthreads)
    {
        if constexpr ((KT & 1) != 0) {
            // the upper half of the last k-block has no channels: zero
            for (int u = tid; u < MT * 64; u += nthreads)
                *reinterpret_cast<f16x4*>(dst + (u >> 6) * F_MSTRIDE + (F_KB - 1) * 512 + (u & 63) * 8 + 4) = f16x4{0, 0, 0, 0};
        }
        constexpr int NV = COUT * CIN / 8;   // 16-byte pieces
        constexpr int INFLIGHT = 4;
        for (int v0 = tid; v0 < NV; v0 += nthreads * INFLIGHT) {
            f16x8 val[INFLIGHT];
#pragma unroll
            for (int j = 0; j < INFLIGHT; ++j) {
                const int v = v0 + j * nthreads;
                if (v < NV) val[j] = *reinterpret_cast<const f16x8*>(W + v * 8);
            }
#pragma unroll
            for (int j = 0; j < INFLIGHT; ++j) {
                const int v = v0 + j * nthreads;
                if (v >= NV) continue;
                const int o = (v * 8) / CIN, k = (v * 8) % CIN;
                const int m = o >> 4, r = o & 15, tile = k >> 4, g = (k & 15) >> 2;   // g is 0 or 2
                f16* base = dst + m * F_MSTRIDE + (tile >> 1) * 512 + (tile & 1) * 4 + r * 8;
                *reinterpret_cast<f16x4*>(base + (16 * g) * 8) = f16x4{val[j][0], val[j][1], val[j][2], val[j][3]};
                *reinterpret_cast<f16x4*>(base + (16 * (g + 1)) * 8) = f16x4{val[j][4], val[j][5], val[j][6], val[j][7]};
            }
        }
    }

    /**
     * Copies the weight matrix into LDS in adjoint operand order (A = tiles of W^T): a thread
     * reads 8 consecutive columns of 4 consecutive rows (four 16-byte loads) and writes, per
     * column, the 4 row values that are neighbours in the operand.
     */
    __device__ static void stageAdjoint(const f16* __restrict__ W, f16* __restrict__ dst, int tid, int nthreads)
    {
        if constexpr ((MT & 1) != 0) {
            for (int u = tid; u < KT * 64; u += nthreads)
                *reinterpret_cast<f16x4*>(dst + (u >> 6) * A_MSTRIDE + (A_KB - 1) * 512 + (u & 63) * 8 + 4) = f16x4{0, 0, 0, 0};
        }
        constexpr int COLS8 = CIN / 8;
        constexpr int ITEMS = (COUT / 4) * COLS8;
        for (int item = tid; item < ITEMS; item += nthreads) {
            const int q = item / COLS8, k0 = (item % COLS8) * 8;
            const int o0 = 4 * q;                       // rows o0..o0+3: same tile and lane group, j = 0..3
            f16x8 rows[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) rows[j] = *reinterpret_cast<const f16x8*>(W + (o0 + j) * CIN + k0);
            const int tile = o0 >> 4, g = (o0 & 15) >> 2;
            const int mi = k0 >> 4, r0 = k0 & 15;
            f16* base = dst + mi * A_MSTRIDE + (tile >> 1) * 512 + (tile & 1) * 4 + (16 * g + r0) * 8;
#pragma unroll
            for (int c = 0; c < 8; ++c)
                *reinterpret_cast<f16x4*>(base + c * 8) = f16x4{rows[0][c], rows[1][c], rows[2][c], rows[3][c]};
        }
    }

    /**
     * A operand of the forward pass: rows 16m..16m+15 of W, k-block kb.
     * \tparam GLOBAL_W false: w is the LDS copy in forward operand order. true: w is the
     *   row-major (COUT, CIN) matrix in global memory (networks whose weights exceed the LDS):
     *   the lane gathers its two runs of 4 halves itself.
     */
    template <bool GLOBAL_W>
    __device__ __forceinline__ static f16x8 forwardOperand(const f16* __restrict__ w, int m, int kb, int lane)
    {
        if constexpr (!GLOBAL_W) {
            return *reinterpret_cast<const f16x8*>(w + m * F_MSTRIDE + kb * 512 + lane * 8);
        } else {
            const int g = lane >> 4, r = lane & 15;
            const f16* row = w + (16 * m + r) * CIN + 32 * kb + 4 * g;
            const f16x4 lo = *reinterpret_cast<const f16x4*>(row);
            f16x4 hi = {0, 0, 0, 0};
            if (2 * kb + 1 < KT) hi = *reinterpret_cast<const f16x4*>(row + 16);
            return concat(lo, hi);
        }
    }

    /**
     * A operand of the adjoint pass: rows 16mi..16mi+15 of W^T, k-block kb.
     * \tparam GLOBAL_W false: wT is the LDS copy in adjoint operand order. true: wT is the
     *   transposed matrix, row-major (CIN, COUT), in global memory.
     */
    template <bool GLOBAL_W>
    __device__ __forceinline__ static f16x8 adjointOperand(const f16* __restrict__ wT, int mi, int kb, int lane)
    {
        if constexpr (!GLOBAL_W) {
            return *reinterpret_cast<const f16x8*>(wT + mi * A_MSTRIDE + kb * 512 + lane * 8);
        } else {
            const int g = lane >> 4, r = lane & 15;
            const f16* row = wT + (16 * mi + r) * COUT + 32 * kb + 4 * g;
            const f16x4 lo = *reinterpret_cast<const f16x4*>(row);
            f16x4 hi = {0, 0, 0, 0};
            if (2 * kb + 1 < MT) hi = *reinterpret_cast<const f16x4*>(row + 16);
            return concat(lo, hi);
        }
    }

    /**
     * Forward pass of the layer for one 64-point tile.
     * \param w weights: LDS copy in forward operand order, or (GLOBAL_W) the row-major matrix
     * \param bias LDS bias vector (COUT halves) or nullptr
     * \param x input activations: x[nt][t] = channels 16t+4g+{0..3} of point 4r+nt
     * \param y output activations in the same layout
     * \param preTile [STORE] where the pre-activations of this tile go (with GUARDED, nullptr means
     *        nowhere; the test is compiled in only then, as its branches break up the instruction
     *        scheduling of the layer): (COUT, 64) halves,
     *        channel-major, so that both the adjoint pass (per channel, 4 points of one
     *        lane) and the weight update (per channel, 8 consecutive points) read it
     *        with wide loads
     */
    template <bool STORE, bool GLOBAL_W = false, bool GUARDED = false>
    __device__ __forceinline__ static void forward(const f16* __restrict__ w, const f16* __restrict__ bias,
                                                   const f16x4 (&x)[NT][KT], f16x4 (&y)[NT][MT],
                                                   f16* __restrict__ preTile, int lane)
    {
        const int g = lane >> 4, r = lane & 15;
        const f16x4 zero4 = {0, 0, 0, 0};
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            f32x4 acc[NT];
            if constexpr (BIAS) {
                const f16x4 b = *reinterpret_cast<const f16x4*>(bias + 16 * m + 4 * g);
                const f32x4 bf = {static_cast<float>(b[0]), static_cast<float>(b[1]),
                                  static_cast<float>(b[2]), static_cast<float>(b[3])};
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = bf;
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int kb = 0; kb < F_KB; ++kb) {
                const f16x8 a = forwardOperand<GLOBAL_W>(w, m, kb, lane);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const f16x4 hi = (2 * kb + 1 < KT) ? x[nt][(2 * kb + 1 < KT) ? 2 * kb + 1 : 0] : zero4;
                    acc[nt] = mfma32(a, concat(x[nt][2 * kb], hi), acc[nt]);
                }
            }
            f16x4 p[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) p[nt] = toF16(acc[nt]);
            if (STORE && (!GUARDED || preTile != nullptr)) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f16x4 v = {p[0][i], p[1][i], p[2][i], p[3][i]};
                    *reinterpret_cast<f16x4*>(preTile + (16 * m + 4 * g + i) * TILE_POINTS + 4 * r) = v;
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) y[nt][m] = activationForwardChannels<Activation>(p[nt], 16 * m + 4 * g);
        }
    }

    /**
     * forward<false> that also hands out the pre-activations, in the layout in which forward<true> stores them and
     * adjoint reads them (lane: channels 16m + 4g + i of the points 4r + nt): the adjoint kernel of a network whose
     * training pass kept the encoded input only runs the layers again (the same operations: the same bits) instead
     * of reading 2 C_out bytes per point and layer back from memory.
     */
    __device__ __forceinline__ static void forwardKeep(const f16* __restrict__ w, const f16* __restrict__ bias,
                                                       const f16x4 (&x)[NT][KT], f16x4 (&pre)[NT][MT], f16x4 (&y)[NT][MT], int lane)
    {
        const int g = lane >> 4;
        const f16x4 zero4 = {0, 0, 0, 0};
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            f32x4 acc[NT];
            if constexpr (BIAS) {
                const f16x4 b = *reinterpret_cast<const f16x4*>(bias + 16 * m + 4 * g);
                const f32x4 bf = {static_cast<float>(b[0]), static_cast<float>(b[1]),
                                  static_cast<float>(b[2]), static_cast<float>(b[3])};
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = bf;
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int kb = 0; kb < F_KB; ++kb) {
                const f16x8 a = forwardOperand<false>(w, m, kb, lane);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const f16x4 hi = (2 * kb + 1 < KT) ? x[nt][(2 * kb + 1 < KT) ? 2 * kb + 1 : 0] : zero4;
                    acc[nt] = mfma32(a, concat(x[nt][2 * kb], hi), acc[nt]);
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                pre[nt][m] = toF16(acc[nt]);
                y[nt][m] = activationForwardChannels<Activation>(pre[nt][m], 16 * m + 4 * g);
            }
        }
    }

    /**
     * Adjoint pass of the layer for one 64-point tile.
     * \param wT transposed weights: LDS copy in adjoint operand order, or (GLOBAL_W) the
     *        row-major (CIN, COUT) matrix in global memory
     * \param dy in: adjoint of the layer output (after the activation);
     *           out: adjoint of the pre-activation, zeroed for points outside the batch
     * \param dx adjoint of the layer input (only written if COMPUTE_DX)
     * \param preTile pre-activations stored by forward<true>
     * \param dpreTile [STORE_DPRE] receives the pre-activation adjoints, same layout with DPRE_STRIDE halves
     *        between the channels (T_STRIDE: the LDS tile that weightGradient reads)
     * \param validMask bit nt set iff point 4r+nt of this lane is inside the batch
     */
    template <bool STORE_DPRE, bool COMPUTE_DX, bool GLOBAL_W = false, bool GUARDED = false, int DPRE_STRIDE = TILE_POINTS>
    __device__ __forceinline__ static void adjoint(const f16* __restrict__ wT, f16x4 (&dy)[NT][MT],
                                                   f16x4 (&dx)[NT][KT], const f16* __restrict__ preTile,
                                                   f16* __restrict__ dpreTile, int validMask, int lane)
    {
        const int g = lane >> 4, r = lane & 15;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f16x4 pre = *reinterpret_cast<const f16x4*>(preTile + (16 * m + 4 * g + i) * TILE_POINTS + 4 * r);
                f16x4 d;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const half a = activationAdjointChannel<Activation>(toHalf(pre[nt]), toHalf(dy[nt][m][i]), 16 * m + 4 * g + i);
                    d[nt] = ((validMask >> nt) & 1) ? fromHalf(a) : static_cast<f16>(0);
                    dy[nt][m][i] = d[nt];
                }
                if (STORE_DPRE && (!GUARDED || dpreTile != nullptr))
                    *reinterpret_cast<f16x4*>(dpreTile + (16 * m + 4 * g + i) * DPRE_STRIDE + 4 * r) = d;
            }
        }
        if constexpr (COMPUTE_DX) {
            const f16x4 zero4 = {0, 0, 0, 0};
#pragma unroll
            for (int mi = 0; mi < KT; ++mi) {
                f32x4 acc[NT];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < A_KB; ++kb) {
                    const f16x8 a = adjointOperand<GLOBAL_W>(wT, mi, kb, lane);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const f16x4 hi = (2 * kb + 1 < MT) ? dy[nt][(2 * kb + 1 < MT) ? 2 * kb + 1 : 0] : zero4;
                        acc[nt] = mfma32(a, concat(dy[nt][2 * kb], hi), acc[nt]);
                    }
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) dx[nt][mi] = toF16(acc[nt]);
            }
        }
    }

    /**
     * adjoint<true, COMPUTE_DX, false, false, T_STRIDE> with the pre-activations in registers (forwardKeep) instead of
     * in memory: the adjoint pre-activations go to the wavefront's LDS tile for weightGradient.
     */
    template <bool COMPUTE_DX>
    __device__ __forceinline__ static void adjointKept(const f16* __restrict__ wT, f16x4 (&dy)[NT][MT], f16x4 (&dx)[NT][KT],
                                                       const f16x4 (&pre)[NT][MT], f16* __restrict__ dpreTile, int validMask, int lane)
    {
        const int g = lane >> 4, r = lane & 15;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f16x4 d;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const half a = activationAdjointChannel<Activation>(toHalf(pre[nt][m][i]), toHalf(dy[nt][m][i]), 16 * m + 4 * g + i);
                    d[nt] = ((validMask >> nt) & 1) ? fromHalf(a) : static_cast<f16>(0);
                    dy[nt][m][i] = d[nt];
                }
                *reinterpret_cast<f16x4*>(dpreTile + (16 * m + 4 * g + i) * (TILE_POINTS + 8) + 4 * r) = d;
            }
        }
        if constexpr (COMPUTE_DX) {
            const f16x4 zero4 = {0, 0, 0, 0};
#pragma unroll
            for (int mi = 0; mi < KT; ++mi) {
                f32x4 acc[NT];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < A_KB; ++kb) {
                    const f16x8 a = adjointOperand<false>(wT, mi, kb, lane);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const f16x4 hi = (2 * kb + 1 < MT) ? dy[nt][(2 * kb + 1 < MT) ? 2 * kb + 1 : 0] : zero4;
                        acc[nt] = mfma32(a, concat(dy[nt][2 * kb], hi), acc[nt]);
                    }
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) dx[nt][mi] = toF16(acc[nt]);
            }
        }
    }

    /** The input of the layer (before the activation of the layer in front of it), from registers into the
     *  wavefront's LDS tile of CIN rows of T_STRIDE halves that weightGradient<.., T_STRIDE> reads. */
    __device__ __forceinline__ static void stageInput(const f16x4 (&x)[NT][KT], f16* __restrict__ inTile, int lane)
    {
        const int g = lane >> 4, r = lane & 15;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f16x4 v = {x[0][t][i], x[1][t][i], x[2][t][i], x[3][t][i]};
                *reinterpret_cast<f16x4*>(inTile + (16 * t + 4 * g + i) * (TILE_POINTS + 8) + 4 * r) = v;
            }
    }

    // halves between the channel rows of the tile that weightGradient transposes in LDS: 64 points and 16 bytes,
    // so that the sixteen rows a 16-byte operand read touches start in different banks
    static constexpr int T_STRIDE = TILE_POINTS + 8;
    static constexpr int T_HALVES = COUT * T_STRIDE;

    /**
     * Adds this tile's share to the gradients of the layer's weights and bias: dW (COUT x CIN) += dpre^T * in and
     * db += dpre^T * 1 on the matrix cores, the 64 points of the tile as contraction index (two k-blocks of 32).
     * The bias sums of all output tiles share one accumulator tile: output tile m is multiplied with a B operand
     * that is one in column m and zero elsewhere, so column m of the tile receives its 16 sums.
     * The A operand needs 8 consecutive points of one channel per lane, the registers hold 4 channels of 4 points:
     * adjoint<true, .., T_STRIDE> has written the adjoint pre-activations into rows of 64 points per channel in
     * this wavefront's LDS tile. The B
     * operand is read from the channel-major tile the forward kernel stored, the activation of the previous layer
     * applied again (as WeightUpdateKernel does, which this replaces for networks whose gradient tiles fit into
     * the registers of a wavefront; replaces network_weight_update_block.cuh:356-494 of the reference).
     * \param sTile T_HALVES halves of LDS of this wavefront: the adjoint pre-activations (zero for points outside the batch)
     * \param inTile CIN rows of IN_STRIDE halves (64 points each): the input of the layer before InputActivation, as
     *        the forward kernel stored it, or (IN_STRIDE = T_STRIDE) as stageInput put it into LDS
     */
    template <typename InputActivation, int IN_STRIDE = TILE_POINTS>
    __device__ __forceinline__ static void weightGradient(const f16* sTile, const f16* __restrict__ inTile,
                                                          f32x4 (&accW)[MT][KT], f32x4& accB, int lane)
    {
        static_assert(MT <= 16, "one column of the bias tile per output tile");
        const int g = lane >> 4, r = lane & 15;
        __builtin_amdgcn_sched_barrier(0);
        waveLdsSync();
        const f16x8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
        const f16x8 zeros = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int kb = 0; kb < TILE_POINTS / 32; ++kb) {
            f16x8 b[KT];
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                const int channel = 16 * k + r;
                const f16x8 raw = *reinterpret_cast<const f16x8*>(inTile + channel * IN_STRIDE + 32 * kb + 8 * g);
                b[k] = activationForwardChannel<InputActivation>(raw, channel);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const f16x8 a = *reinterpret_cast<const f16x8*>(sTile + (16 * m + r) * T_STRIDE + 32 * kb + 8 * g);
#pragma unroll
                for (int k = 0; k < KT; ++k) accW[m][k] = mfma32(a, b[k], accW[m][k]);
                if constexpr (BIAS) accB = mfma32(a, r == m ? ones : zeros, accB);
            }
        }
        waveLdsSync();   // the next layer writes its rows over these
        __builtin_amdgcn_sched_barrier(0);
    }

    /**
     * After the last tile: the gradient tiles of the wavefronts of a workgroup are added up in LDS, one wavefront
     * after the other (so that the sum rounds the same way in every run), and stored as this workgroup's partial sums,
     * (COUT, CIN) row-major and COUT bias sums, into slice blockIdx.x of numSlices slices that lie sliceStride floats
     * apart; the slices beyond the grid are zeroed, each by one workgroup. All threads of the workgroup call this;
     * sAcc: (MT * KT + 1) * 256 floats.
     */
    template <int WAVES>
    __device__ __forceinline__ static void storeWeightGradient(const f32x4 (&accW)[MT][KT], const f32x4& accB, float* sAcc,
                                                               float* __restrict__ partialWeights, float* __restrict__ partialBias,
                                                               int numSlices, int sliceStride, int wave, int lane)
    {
        const int g = lane >> 4, r = lane & 15;
        constexpr int TILES = MT * KT + (BIAS ? 1 : 0);
        __syncthreads();   // whatever used this LDS before is done
        for (int i = threadIdx.x; i < TILES * 256; i += blockDim.x) sAcc[i] = 0.f;
        __syncthreads();
        for (int w = 0; w < WAVES; ++w) {
            if (wave == w) {
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int k = 0; k < KT; ++k)
#pragma unroll
                        for (int i = 0; i < 4; ++i) sAcc[(m * KT + k) * 256 + (4 * g + i) * 16 + r] += accW[m][k][i];
                if constexpr (BIAS) {
                    // column r of the bias tile: the sums of the channels 16r + 4g .. + 3
                    if (r < MT) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) sAcc[MT * KT * 256 + 16 * r + 4 * g + i] += accB[i];
                    }
                }
            }
            __syncthreads();
        }
        for (int e = threadIdx.x; e < MT * KT * 256; e += blockDim.x) {
            const int t = e >> 8, within = e & 255;
            const int m = t / KT, k = t - m * KT;
            partialWeights[(16 * m + (within >> 4)) * CIN + 16 * k + (within & 15)] = sAcc[e];
        }
        if constexpr (BIAS) {
            for (int e = threadIdx.x; e < COUT; e += blockDim.x) partialBias[e] = sAcc[MT * KT * 256 + e];
        }
        for (int slice = blockIdx.x + gridDim.x; slice < numSlices; slice += gridDim.x) {
            const long long offset = static_cast<long long>(slice - static_cast<int>(blockIdx.x)) * sliceStride;
            for (int e = threadIdx.x; e < COUT * CIN; e += blockDim.x) partialWeights[offset + e] = 0.f;
            if constexpr (BIAS) {
                for (int e = threadIdx.x; e < COUT; e += blockDim.x) partialBias[offset + e] = 0.f;
            }
        }
    }
};

QUICKMLP_KERNEL_NAMESPACE_END
