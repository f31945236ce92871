#pragma once

#include "activation.h"
#include "common.h"
#include "iencoding.h"
#include "json.h"
#include "kernel_loader.h"
#include "tensor.h"

#include <optional>
#include <unordered_map>
#include <random>
#include <vector>

QUICKMLP_NAMESPACE_BEGIN

/**
 * A fully fused coordinate MLP: input encodings, linear layers and activations in one
 * generated kernel per pass (inference, forward with stored intermediates, adjoint),
 * plus one batch-reduction kernel per layer for the weight gradients.
 */
class FusedNetwork : NonAssignable
{
public:
    /** additive flags specifying what gradients to compute in the adjoint pass */
    enum AdjointMode
    {
        //Compute gradients with respect to the network input
        GRADIENTS_INPUT = 0x1,
        //Compute gradients with respect to the network weights
        GRADIENTS_NETWORK_WEIGHTS = 0x2,
        //Compute gradients with respect to the input encodings
        GRADIENTS_INPUT_ENCODINGS = 0x4,

        ADJOINT_MODE_MAX_COMBINATIONS = 8
    };
    typedef int AdjointModeFlags;

    /** Compile options, loaded from the json ("options"). */
    struct CompileOptions
    {
        //Overwrites the kernel block size (threads, multiple of the wavefront size).
        //If <=0 (the default), the library chooses.
        int overwriteBlocksizeInference = -1;
        int overwriteBlocksizeForward = -1;
        int overwriteBlocksizeBackward = -1;
        int overwriteBlocksizeWeightUpdate = -1;

        //Tiles of 64 points that one wavefront of the inference / forward kernel encodes
        //together (level by level for grid encodings). If <=0, the library chooses.
        int pointsPerLane = -1;

        // If true (default), networks with grid encodings and at most 32 encoded channels get a
        // kernel shape whose encoded rows wait in registers instead of LDS: a wavefront then
        // takes 8 tiles at once, and 2^20 points are one sweep over the level tables.
        bool registerStaging = true;

        // If true (default), a network whose only encoding is the identity loads its first
        // matrix-core operands straight from the input rows; false sends them through the LDS
        // staging rows like every other encoding (same results bit for bit).
        bool directInput = true;

        // Inference only: evaluate the points slab by slab of a dense grid that exceeds the L2
        // (a counting sort of the batch in front of the fused kernel, see point_order.h; the
        // results are those of the order given). <0 (default): the library decides from the
        // encodings and the batch size; 0: never; >0: whenever an encoding offers a slab key.
        // The sorted copy of the inputs lives in device memory that the network allocates on
        // the first such call and keeps (grown when a larger batch comes); calls of one
        // network on several streams at once would share it.
        int sortPoints = -1;
        //true: a training pass (forward with stored intermediates + adjoint) evaluates the batches that
        //inference would sort in the same sorted order; the sorted rows and the order travel in the
        //forward memory. false: training passes take the batch as given.
        bool sortTraining = true;

        // Parameter gradients of grid encodings: summed slice by slice in LDS by a kernel of its own
        // (kernels/grid_gradient.h) instead of scattered with float atomics by the backward kernel.
        // <0 (default): for batches of SLICE_GRADIENTS_MIN_BATCH points or more (of half as many for grids of 8
        // levels or more); 0: never; >0: always.
        int sliceGradients = -1;

        // Input gradients through grid encodings whose parameter gradients take the slice kernels: a training
        // pass (forward) also stores, per point and level, the derivatives of the interpolated features with
        // respect to the position (16 bytes per level for a 3-D grid with 2 half features), and the adjoint pass
        // reads them instead of gathering all corners of every cell a second time. <0 (default): when the
        // adjoint flags announced last (forwardMemory(), adjoint()) ask for input and encoding gradients;
        // 0: never (no room for them in the forward memory either); >0: every training pass.
        int inputDerivatives = -1;

        // Parameter gradients of a dense single-level grid whose batch trains sorted by grid slab: summed owner by
        // owner of the grid's nodes in LDS, without gradient records (kernels/grid_gradient_columns.h).
        // <0 (default) and >0: wherever the encoding offers it; 0: never (records and slices as for other grids).
        int columnGradients = -1;

        // Networks whose backward kernel sums the weight gradients of all layers: a training pass keeps the encoded
        // input only (2 C_in0 bytes per point instead of 2 (C_in0 + sum C_out)) and the backward kernel runs the layers
        // forward again per tile, the pre-activations staying in registers. <0 (default): when the adjoint flags
        // announced last (forwardMemory(), prepare(), adjoint()) lead to such a backward kernel; 0: never; >0: as <0.
        // An adjoint pass with other flags than announced, whose kernels need the stored intermediates, first runs
        // the forward pass again into the same forward memory.
        int recomputeIntermediates = -1;

        // Gradients of the layer weights: summed inside the backward kernel, which holds the adjoint
        // pre-activations in registers (Layer::weightGradient), instead of by one kernel per layer that reads
        // them back from memory. <0 (default): the layers with the fewest gradient tiles, up to 16 tiles (64
        // registers of a wavefront), in networks whose weights all stay in LDS; 0: never; >0: up to 32 tiles.
        int fusedWeightUpdate = -1;

        // Accepted for compatibility; the LDS layouts of this implementation are
        // bank-conflict free for 64 lanes by construction and need no skew.
        bool skewSharedMemory = false;

        // If true, the per-layer weight update kernels are launched on separate
        // streams that fork from / join into the caller's stream. Off by default (the
        // reference's default is on: its kernel runs in a single block per layer): every
        // weight update kernel here fills the device on its own, and running them one after
        // the other measured 2-3 % faster per train step than running them side by side.
        bool parallelWeightUpdate = false;
    };

private:
    struct LayerSpecification
    {
        //specs from Json
        int channelsOut;
        bool useBias;
        //Either a single entry, used for every channel, or one per channel (unsupported in the kernels)
        std::vector<Activation_ptr> activations;

        //cached parameter for easy access
        int channelsIn;
        //prefix sum, offset into parameter array
        int weightsStart;
        int biasStart;
    };

    CompileOptions compileOptions_;
    int channelsIn_;
    int channelsOut_;
    int encodedChannels_;
    int networkInputPadding_;
    std::vector<IEncoding_ptr> encodings_;
    std::vector<LayerSpecification> layers_;

    int numParameters_;
    Tensor parametersInference_;
    Tensor parametersGradients_;

    struct CompiledKernel
    {
        KernelFunction fun;
        int blockSize = 0;
        int pointsPerLane = 1;
        int sharedMemorySize = 0;
        int fullGrid = 0;
    };
    // [store intermediates][variant], see ForwardVariant
    // [0]: inference, [1]: forward (stores the intermediates), [2]: forward that also stores position derivatives
    // ([3], [4]: as [1], [2], but of the intermediates only the encoded input is stored)
    std::optional<CompiledKernel> forwardKernels_[5][4];
    // set once the compiled REGISTERS shape turned out to spill heavily: it is not used then
    bool registerShapeSpills_[5] = {false, false, false, false, false};

    // counting sort of the batch by grid slab in front of the inference kernel
    struct PointOrder
    {
        std::optional<KernelFunction> count, scan, scatter;
        std::optional<KernelFunction> gatherAddRows;   // rows of the input gradients out of the sorted order
        Tensor workspace;           // slab totals and per-chunk histograms (ints), sorted inputs (floats), order (ints)
        long long capacityWords = 0;   // 32-bit words the workspace holds
    };
    PointOrder pointOrder_;
    /** Smaller batches are never sorted when sortPoints < 0; larger ones if the encoding expects a gain. */
    static constexpr int SORT_POINTS_MIN_BATCH = 1 << 19;
    /** Slabs of the sort (POINT_ORDER_MAX_SLABS of kernels/point_order.h). */
    static constexpr int SORT_SLABS = 1024;
    /**
     * Sorts the batch by the slab key of the first encoding that offers one.
     * \return false if the batch stays as it is; else sortedInput views the sorted copy and
     *   order holds, per row of it, the row of the caller's batch
     */
    bool sortPoints(const Tensor& input, kernel::Tensor2Read<float>& sortedInput, const int*& order, stream_t stream,
                    bool noAlloc = false, void* destination = nullptr);
    void loadPointOrderKernels(bool rowMoves);
    /** True if some batch size makes this network train in sorted order (its backward kernels then take the order). */
    bool trainsSortedBatches() const;
    /** The slab key of the encoding that orders a batch of numel points, if such a batch is ordered at all
     *  (a function of the specification and numel alone). */
    bool pointOrderFor(int numel, kernel::PointOrderKey& key) const;
    /** Does a training pass over numel points run in sorted order? Then the forward memory holds, behind the
     *  intermediates and 256-byte aligned, the sorted input rows (numel x channelsIn floats) and the order (numel ints). */
    bool sortsTraining(int numel) const;
    /** adjointMemory() of a batch that is processed in the order given. */
    size_t adjointMemoryAsGiven(int numElements, AdjointModeFlags adjointFlags) const;
    /** Bytes at the end of the adjoint memory of a batch that trains in sorted order (with the gap that aligns them
     *  behind bytesInFront): the rows of dL/dy and of the input gradients in that order. */
    size_t sortedAdjointBytes(int numElements, AdjointModeFlags adjointFlags, size_t bytesInFront) const;
    /** Byte offset of the sorted rows within the forward memory of a batch of numel points. */
    size_t sortedRowsOffset(int numel) const;

    struct AdjointLayerInfo
    {
        //channel prefix of this layer's adjoint pre-activations in the adjoint tmp memory
        int offsetAdjOut;
        //channel prefix of this layer's input in the forward tmp memory (encoded input for layer 0)
        int offsetIn;
        //channel prefix of this layer's pre-activations in the forward tmp memory
        int offsetPre;

        stream_t stream = nullptr;
        event_t event = nullptr;
    };
    struct WeightUpdateKernel
    {
        CompiledKernel kernel;
        int numChunks = 1;
    };
    /** Kernels that sum the parameter gradients of one grid encoding slice by slice (grid_gradient.h). */
    struct SliceGradientKernel
    {
        int encoding = -1;
        IEncoding::GradientSliceLayout layout;
        // GridGradientRecordsKernel with layout.pointsPerWorkgroup >> i lanes per workgroup (down to 128), compiled
        // when a batch first asks for it: a batch of fewer points than the largest workgroups of all compute units
        // hold goes to smaller ones
        std::vector<std::optional<CompiledKernel>> records;
        // the same with the input gradients from the position derivatives that the forward pass stored
        std::vector<std::optional<CompiledKernel>> recordsFromDerivatives;
        long long derivativeOffset = 0;   // bytes per point of the batch in front of this encoding's derivatives in the forward memory
        std::string recordsSource;
        int channelOffset = 0;
        CompiledKernel kernel;       // GridGradientSlicesKernel
        Tensor items;                // device copy of layout.items
        // For batches that train sorted by grid slab, where the encoding offers it: the kernels of
        // kernels/grid_gradient_columns.h (compiled on first use), which take the place of records and slices
        bool columnsOffered = false;
        IEncoding::GradientColumnLayout columnLayout;
        std::optional<CompiledKernel> columnsPlan;
        std::optional<CompiledKernel> columns[2];   // [1]: input gradients from the position derivatives of the forward pass
    };
    struct AdjointKernel
    {
        CompiledKernel adjoint;
        std::vector<SliceGradientKernel> sliceGradients;
        std::vector<WeightUpdateKernel> layers;
        CompiledKernel reduce;
        CompiledKernel transpose;
        int perEntryAdjointMemoryBytes = 0;
        std::vector<bool> fusedLayers;    // layers whose weight gradients the adjoint kernel sums (no kernel in 'layers')
        bool fusedWeightUpdate = false;   // any of them
        bool outputOrder = false;         // the kernel takes the order of a sorted batch for its rows of dL/dy
    };
    // [adjoint flags][grid gradients by slices instead of atomics][the layers run again instead of reading their intermediates]
    std::optional<AdjointKernel> backwardKernel_[ADJOINT_MODE_MAX_COMBINATIONS][2][2];
    // Below this the two slice kernels cost more than the atomics they save (their work items zero and write
    // back whole slices whatever the batch): a train step of a 16-level hash grid at 2^14 / 2^15 / 2^16 / 2^17
    // points 0.18 / 0.24 / 0.37 / 0.63 ms with atomics, 0.18 / 0.19 / 0.22 / 0.30 ms by slices; of one dense
    // 4-D level with 8 features 0.08 / 0.09 / 0.12 / 0.19 against 0.10 / 0.11 / 0.12 / 0.23 ms. The atomics of a
    // point grow with the number of levels, the fixed work of the slice kernels with the size of the table: grids
    // of 8 levels or more take the slices from half the batch size on.
    static constexpr int SLICE_GRADIENTS_MIN_BATCH = 1 << 16;
    static constexpr int SLICE_GRADIENTS_MIN_BATCH_MANY_LEVELS = 1 << 15;
    /** True if some encoding of the network offers gradient slices (the adjoint memory then has room for the adjoint of the encoded rows). */
    bool hasSliceGradients() const;
    /** Bytes per point of adjoint memory for the adjoint of the encoded rows (read by the records kernels); 0 without them. */
    int sliceGradientBytesPerPoint() const;
    /** Bytes of bucket cursors and records of all encodings with gradient slices for a batch of numel (padded) points. */
    size_t sliceGradientWorkspaceBytes(long long numel) const;
    /** Whether a batch of numel points with these flags takes the slice kernels. */
    bool useSliceGradients(int numel, int flags) const;

    int perEntryForwardMemoryBytes_;
    /**
     * Position derivatives of the grid encodings (options.input_derivatives): per encoding the bytes per point of
     * the batch in front of its derivatives within their region of the forward memory (-1: the encoding keeps
     * none), and the bytes per point of the whole region, which lies behind the intermediates.
     */
    std::vector<long long> derivativeOffsets_;
    int derivativeBytesPerPoint_ = 0;
    /** The adjoint flags that the caller announced last: forwardMemory(n, flags), adjoint(..., flags, ...). */
    int announcedFlags_ = 0;
    /** What the last training pass left in a forward memory. */
    struct ForwardRecord
    {
        int numel = 0;
        bool derivatives = false;   // position derivatives of the grids
        bool inputOnly = false;     // of the intermediates only the encoded input
    };
    std::unordered_map<const void*, ForwardRecord> forwardRecords_;
    /** Whether adjoint(flags) over numel points runs the layers again in its backward kernel instead of reading
     *  their intermediates: a training pass that is followed by it keeps the encoded input only. */
    bool recomputesFor(int numel, int flags) const;
    /**
     * recomputesFor(), and the backward kernel that runs the layers again holds its registers: loaded on the first
     * call for these flags (it is the kernel that adjoint() will run), and not used if it spills more than a few
     * words (16 -> 64 -> 64 -> 16 with biases: 27 gradient tiles and 72 registers of pre-activations, 316 bytes).
     */
    bool recomputes(int numel, int flags);
    int recomputeVerdict_[ADJOINT_MODE_MAX_COMBINATIONS][2];   // -1: not known yet
    static constexpr int MAX_RECOMPUTE_SCRATCH = 64;
    /** Bytes per point of the forward memory: intermediates and, where kept, position derivatives. */
    size_t forwardBytesPerPoint() const { return static_cast<size_t>(perEntryForwardMemoryBytes_) + static_cast<size_t>(derivativeBytesPerPoint_); }
    /** Whether a training pass over numel points that is followed by adjoint(flags) stores position derivatives. */
    bool storesDerivatives(int numel, int flags) const;
    std::vector<AdjointLayerInfo> backwardInfo_;
    event_t adjointEvent_;
    bool streamsCreated_;

public:
    //Size of the matrix fragments: all layer widths are padded to multiples of this.
    static constexpr int MATRIX_SIZE = 16;
    //Wavefront size; one wavefront processes a tile of this many points and
    //temporary memory is a multiple of that value
    static constexpr int WARP_SIZE = 64;

    //LDS available to one workgroup on the current device
    static int MaxSharedMemoryBytes();

    /**
     * Constructs the network from the Json configuration 'cfg'. 'parent' is the folder
     * relative to which activation files are resolved. After constructing, the
     * configuration is immutable, so that kernels are compiled once and cached.
     */
    FusedNetwork(const json& cfg, const std::filesystem::path& parent);
    ~FusedNetwork();

    [[nodiscard]] const std::vector<IEncoding_ptr>& encodings() const { return encodings_; }
    [[nodiscard]] int numEncodings() const { return static_cast<int>(encodings_.size()); }
    [[nodiscard]] IEncoding_ptr encoding(int idx);

    [[nodiscard]] int channelsIn() const { return channelsIn_; }
    [[nodiscard]] int channelsOut() const { return channelsOut_; }
    [[nodiscard]] Tensor::Precision precisionIn() const { return Tensor::FLOAT; }
    [[nodiscard]] Tensor::Precision precisionOut() const { return Tensor::FLOAT; }
    [[nodiscard]] int numLayers() const { return static_cast<int>(layers_.size()); }
    [[nodiscard]] const CompileOptions& compileOptions() const { return compileOptions_; }
    [[nodiscard]] bool isParallelStreams() const { return compileOptions_.parallelWeightUpdate; }
    void setParallelStreams(bool enabled) { compileOptions_.parallelWeightUpdate = enabled; }

    [[nodiscard]] int networkParameterCount() const;
    [[nodiscard]] Tensor::Precision networkParameterPrecision(Tensor::Usage usage) const;

    /**
     * Sets the network parameters to the specified tensor: 1D, networkParameterCount()
     * entries of type networkParameterPrecision(usage). The memory stays owned by the caller.
     * Layout: all weight matrices in layer order (row-major (C_out, C_in), padded widths),
     * then the bias vectors of the layers that have one.
     */
    void setNetworkParameter(const Tensor& tensor, Tensor::Usage usage);

    /**
     * Initializes the inference weights to U(-1/sqrt(C_in), 1/sqrt(C_in)) (the default
     * initialization of torch.nn.Linear), drawn row-major layer by layer.
     */
    void initializeInferenceParameters(std::default_random_engine& rng);

    /**
     * Returns the slice of the parameters for the weight matrix (bias=false) or bias
     * vector (bias=true) of layer 'layer'; shares memory with 'rawPtr'.
     */
    Tensor networkParameter(int layer, bool bias, void* rawPtr, Tensor::Precision precision);
    Tensor networkParameter(int layer, bool bias, Tensor::Usage usage);

    /**
     * Inference.
     * \param input (N, channelsIn) float  \param output (N, channelsOut) float
     * \param stream the stream the kernel is enqueued on
     */
    void inference(const Tensor& input, Tensor& output, stream_t stream);

    /**
     * inference() for callers that cannot allocate device memory (code under HIP graph
     * capture, tight serving loops): same results, but nothing on the way allocates.
     * The workspace that orders a batch by grid slab is the library's static device buffer
     * of QMLP_STATIC_SCRATCH_BYTES per GPU instead of the network's own: a batch that
     * needs more is refused. Kernels are only taken if they are loaded already, so
     * inference() has to have run once on a batch of the same size. All calls on one GPU
     * share the buffer: calls that overlap in time (other streams, other networks) race.
     * No counterpart in the reference.
     */
    void inferenceNoAlloc(const Tensor& input, Tensor& output, stream_t stream);

    /** Bytes of temporary memory forward() needs for 'numElements' points. */
    size_t forwardMemory(int numElements, AdjointModeFlags adjointFlags);
    size_t forwardMemory(const Tensor& input, AdjointModeFlags adjointFlags);

    /**
     * Forward pass that stores intermediate results in 'tmpMemory' (forwardMemory() bytes,
     * 16-byte aligned) for a following adjoint().
     */
    void forward(const Tensor& input, Tensor& output, void* tmpMemory, stream_t stream);

    /** Zeros the gradients of the network weights and of the encodings. */
    void zeroGradients();

    /** Bytes of temporary memory adjoint() needs for 'numElements' points. */
    size_t adjointMemory(int numElements, AdjointModeFlags adjointFlags);
    size_t adjointMemory(const Tensor& input, AdjointModeFlags adjointFlags);

    /**
     * Adjoint pass following forward(). Weight and encoding gradients are added to the
     * gradient tensors set via setNetworkParameter / IEncoding::setParameter with
     * Usage::GRADIENTS; input gradients are added to 'adjInput'.
     */
    void adjoint(const Tensor& input, const Tensor& adjOutput, AdjointModeFlags adjointFlags, Tensor& adjInput,
                 const void* tmpMemoryForward, void* tmpMemoryAdjoint, stream_t stream);

    /** For debugging, clears all cached kernels. */
    void clearCachedKernels();

    /**
     * Generates and compiles all kernels for the given adjoint flags without a GPU
     * (flags < 0: inference and forward only). Fills the kernel disk cache.
     */
    void precompile(int adjointFlags);

    /**
     * Everything a later call on a batch of numel points would otherwise do on its first use, on the current
     * device: loads (or compiles) the kernels that inference() takes for a batch of this size and, with
     * adjointFlags > 0, those of forward() and adjoint(); allocates the workspace that orders such a batch by
     * grid slab. After it, calls on batches of this size only enqueue kernels (nothing is loaded or
     * allocated), e.g. under HIP graph capture. No counterpart in the reference.
     */
    void prepare(int numel, int adjointFlags);

    /** The generated device source of a kernel kind: "inference", "backward", "weight_update". */
    std::string generatedSource(const std::string& kind, int adjointFlags = 0);

private:
    // Shapes of the inference / forward kernel. LARGE: 8 wavefronts with 4 tiles each, for grid
    // encodings on batches that still fill the device that way (fewer sweeps over the level
    // tables); DEFAULT: 4 wavefronts, 2 tiles each with grid encodings; NARROW: one tile per
    // wavefront for small batches.
    // REGISTERS: 8 wavefronts whose encoded rows wait in registers (up to 8 tiles each) and pass
    // through one LDS staging tile per wavefront: one sweep over the level tables per 2^20 points.
    enum ForwardVariant { VARIANT_DEFAULT = 0, VARIANT_NARROW = 1, VARIANT_LARGE = 2, VARIANT_REGISTERS = 3 };
    bool hasLargeVariant(bool store) const;
    /** Tiles per wavefront of the REGISTERS shape, 0 if the network has none. */
    int registerVariantTiles(bool store) const;
    /** Workgroup size and tiles per wavefront of a shape of the forward kernel. */
    void forwardShape(bool store, int variant, int& blockSize, int& pointsPerLane) const;
    void compileForwardKernel(bool store, int variant, bool compileOnly = false, bool derivatives = false, bool inputOnly = false);
    /**
     * The kernel shape for the next launch over a batch of numTiles tiles and, in launchTiles,
     * how many of them that launch should take (whole steps of a large shape first; the caller
     * asks again for the rest).
     */
    const CompiledKernel& forwardKernelFor(bool store, int numTiles, int* launchTiles = nullptr, bool noAlloc = false, bool derivatives = false, bool inputOnly = false);
    /** Points per launch of a forward kernel: the whole batch, or two passes of the grid for networks that gather. */
    int gatherChunkPoints(const CompiledKernel& ck) const;
    /** inference (store = false) or forward with stored intermediates, in one or several launches. */
    /** Function attributes of the generated forward / backward kernels. */
    std::string kernelAttributes(int blockSize) const;
    /** First input channel of the identity encoding if that is the network's only encoding and
     *  options.direct_input is on; -1 otherwise. */
    int directInputStart() const;
    /** Throws unless every encoding with parameters has a tensor bound for 'usage'. */
    void checkEncodingParameters(Tensor::Usage usage) const;
    void launchForward(bool store, const Tensor& input, Tensor& output, half* tmpMemory, stream_t stream, bool noAlloc = false, bool derivatives = false, bool inputOnly = false);
    void compileBackwardKernel(int flags, bool sliceGradients = false, bool compileOnly = false, bool recompute = false);
    /** The records kernel of a batch of numel points (compiled on first use; compileOnly: all of them into the cache). */
    const CompiledKernel& recordsKernelFor(SliceGradientKernel& sk, int flags, int numel, bool fromDerivatives = false);
    /** Compiles (compileOnly: into the cache) or loads the two kernels of kernels/grid_gradient_columns.h for sk. */
    void compileColumnKernels(SliceGradientKernel& sk, int flags, bool compileOnly, bool fromDerivatives = false);
    /** Bytes at the start of the slice workspace that the column kernels use: slab starts, the number of work items, the items. */
    static size_t columnWorkspaceBytes(const IEncoding::GradientColumnLayout& layout, long long numel, int* maxItems = nullptr);
    /** The slab totals of the sort of a training pass: behind the sorted rows and the order in the forward memory. */
    size_t sortedTotalsOffset(int numel) const;
    /** Behind them: per point of the batch its place in the sorted order. */
    size_t sortedPlacementOffset(int numel) const;
    void compileRecordsKernel(SliceGradientKernel& sk, int flags, size_t variant, bool compileOnly, bool fromDerivatives = false);

    std::string forwardSource(int blockSize, int pointsPerLane, bool registerStaging = false, bool derivatives = false, bool inputOnly = false) const;
    std::string backwardSource(int flags, int blockSize, bool sliceGradients = false, bool recompute = false, bool twoWavefrontsPerSimd = false) const;
    std::string weightUpdateSource(int blockSize) const;
    std::string weightUpdateKernelName(int layer, int& numChunks, int& tilesPerBlock) const;
    void fillEncodingsAndActivations(std::string& codeTemplate) const;
    int forwardBlockSize(int overwrite, bool adjoint, int* pointsPerLane = nullptr, int fixedPointsPerLane = 0) const;
    int weightUpdateBlockSize() const;
    // number of batch slices whose partial weight gradients are kept in the adjoint memory
    int weightUpdateSlices(int numTiles) const;
    /** Layers whose weight gradients the backward kernel sums itself (options.fused_weight_update).
     *  wideRegisters: receives whether that kernel runs one wavefront per SIMD with 512 registers (the gradient
     *  tiles of all layers in its accumulation registers). */
    std::vector<bool> fusedWeightUpdateLayers(int adjointFlags, bool sliceGradients, bool* wideRegisters = nullptr) const;
    /** LDS halves per wavefront of the backward kernel for the tile that Layer::weightGradient transposes. */
    int fusedWeightUpdateTransposeHalves(bool recompute = false) const;
    /** Channels of adjoint pre-activations that the backward kernel stores per point for the weight-update kernels. */
    int storedAdjointChannels(int adjointFlags, bool sliceGradients) const;
    // Where a kernel finds the weights of a layer. RESIDENT: in LDS for the whole kernel.
    // STREAMED: staged into a shared LDS buffer by the whole workgroup right before the layer
    // runs, for every group of tiles (networks whose weights exceed the LDS). GLOBAL: gathered
    // from global memory by every wavefront (single layers that exceed the LDS on their own).
    enum WeightPlacement { WEIGHTS_RESIDENT = 0, WEIGHTS_STREAMED = 1, WEIGHTS_GLOBAL = 2 };
    std::vector<int> weightPlacement(bool adjoint) const;
    // LDS offsets in halves: resident weights, then biases (forward), then the stream buffer
    // (streamOffset, -1 if no layer is streamed); weightOffsets is -1 for global layers and
    // streamOffset for streamed ones. Returns the total size in halves.
    int ldsLayout(bool adjoint, std::vector<int>& weightOffsets, std::vector<int>& biasOffsets,
                  int* streamOffset = nullptr) const;
    // offsets (in halves) of the transposed copies of the weights the adjoint kernel reads from
    // global memory, -1 for resident layers; returns their total size in halves
    size_t transposedWeightLayout(int adjointFlags, std::vector<long long>& offsets) const;
    int ldsParamHalves(bool adjoint) const;
    // definitions of all activations in use, plus one composite per layer with per-channel activations
    std::string activationDefinitions() const;
    // name (inside namespace activations) of the activation type of a layer
    std::string activationTypeName(int layer) const;
    int stageBytesPerWave(bool adjoint) const;
    /** Leading gradient levels of one encoding that the backward kernel sums in LDS. */
    struct LdsGradients
    {
        int levels = 0;      // scatterTile<levels>
        int floats = 0;      // size of the LDS region
        int byteOffset = 0;  // of the region in the kernel's dynamic LDS
    };
    /** One entry per encoding; returns the LDS bytes of the backward kernel including these regions. */
    int ldsGradientLayout(int adjointFlags, int blockSize, std::vector<LdsGradients>& perEncoding, bool sliceGradients = false, bool recompute = false) const;
    std::vector<char> encodingArguments(std::vector<void*>& args, std::vector<std::vector<char>>& storage);
    void ensureStreams();
};
typedef std::shared_ptr<FusedNetwork> FusedNetwork_ptr;

QUICKMLP_NAMESPACE_END
