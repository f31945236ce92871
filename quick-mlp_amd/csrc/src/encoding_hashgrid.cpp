#include <qmlp/encoding_hashgrid.h>

#include <qmlp/fused_network.h>
#include <qmlp/qmlp.h>

#include <cmath>
#include <cstring>
#include <functional>

QUICKMLP_NAMESPACE_BEGIN

static std::vector<float> vectorOrUnit(const std::vector<float>& vx, int d, float v)
{
    if (vx.empty()) return std::vector<float>(d, v);
    CHECK_ERROR(static_cast<int>(vx.size()) == d,
                "If a bounding box vector is specified, its dimension must match the configured dimension. Expected ",
                d, ", actual ", vx.size());
    return vx;
}

static std::vector<float> invert(const std::vector<float>& vx)
{
    std::vector<float> o(vx.size());
    for (size_t i = 0; i < vx.size(); ++i) o[i] = 1.f / vx[i];
    return o;
}

static LayerCombinationMode parseCombinationMode(const json& j)
{
    const std::string s = j.get<std::string>();
    if (s == "concat" || s == "cat") return LayerCombinationMode::CONCAT;
    if (s == "add") return LayerCombinationMode::ADD;
    throw configuration_error("Unknown combination_mode '%s', expected 'concat' or 'add'", s.c_str());
}

static Tensor::Precision parsePrecision(const json& cfg)
{
    const std::string s = cfg.value<std::string>("parameter_precision", "float");
    if (s == "float" || s == "float32") return Tensor::FLOAT;
    if (s == "half" || s == "float16") return Tensor::HALF;
    throw configuration_error("Unknown parameter_precision '%s', expected 'float' or 'half'", s.c_str());
}

EncodingHashGrid::EncodingHashGrid(int start_channel, int dimension, int num_levels, int num_features_per_level,
                                   int log2_hashmap_size, int min_resolution, int max_resolution,
                                   LayerCombinationMode combination_mode,
                                   const std::vector<float>& bounding_box_min,
                                   const std::vector<float>& bounding_box_size,
                                   Tensor::Precision parameter_precision)
    : startChannel_(start_channel)
    , dimension_(dimension)
    , numLevels_(num_levels)
    , numFeaturesPerLevel_(num_features_per_level)
    , log2HashmapSize_(log2_hashmap_size)
    , hashmapSize_(log2_hashmap_size > 0 ? 1 << log2_hashmap_size : -1)
    , minResolution_(min_resolution)
    , maxResolution_(max_resolution)
    , combinationMode_(combination_mode)
    , boundingBoxMin_(vectorOrUnit(bounding_box_min, dimension, -0.5f))
    , boundingBoxSize_(vectorOrUnit(bounding_box_size, dimension, 1.0f))
    , boundingBoxInvSize_(invert(boundingBoxSize_))
    , parameterPrecision_(parameter_precision)
{
    CHECK_ERROR(start_channel >= 0, "start_in must be non-negative but is ", start_channel);
    CHECK_ERROR(dimension >= 1 && dimension <= 6, "Expected 'dimension' to be in [1,6], but got ", dimension);
    CHECK_ERROR(num_levels > 0, "num_levels must be positive but is ", num_levels);
    CHECK_ERROR(num_features_per_level > 0, "num_features_per_level must be positive but is ", num_features_per_level);
    CHECK_ERROR(log2_hashmap_size < 31, "log2_hashmap_size must be below 31 but is ", log2_hashmap_size);
    CHECK_ERROR(min_resolution > 0, "min_resolution must be positive but is ", min_resolution);
    CHECK_ERROR(max_resolution >= min_resolution, "max_resolution must be larger than min_resolution");
    CHECK_ERROR(parameter_precision == Tensor::FLOAT || parameter_precision == Tensor::HALF,
                "the grid parameters are stored as float or half");

    // Level table: geometric progression of resolutions, evaluated in double precision.
    numParameters_ = 0;
    double levelScale = 1;
    if (num_levels > 1)
        levelScale = std::exp((std::log(max_resolution) - std::log(min_resolution)) / (num_levels - 1));

    long long total = 0;
    for (int l = 0; l < num_levels; ++l) {
        const int resolution = static_cast<int>(std::floor(min_resolution * (std::pow(levelScale, l))));
        // saturating R^D so that huge fine levels simply count as "too large to be dense"
        size_t requiredCells = 1;
        bool overflow = false;
        for (int d = 0; d < dimension; ++d) {
            if (requiredCells > (size_t(1) << 40)) overflow = true;
            requiredCells *= static_cast<size_t>(resolution);
        }
        if (!overflow && (hashmapSize_ < 0 || requiredCells <= static_cast<size_t>(hashmapSize_))) {
            layers_.push_back({static_cast<int>(total), resolution, 0, false});
            total += static_cast<long long>(requiredCells) * num_features_per_level;
            QuickMLP::Instance().getLogger()->debug("HashGrid layer %d is dense. Resolution=%d", l, resolution);
        } else {
            CHECK_ERROR(hashmapSize_ > 0, "HashGrid level ", l, " with resolution ", resolution,
                        " is too large for a dense grid and no hash map size is configured");
            layers_.push_back({static_cast<int>(total), resolution, hashmapSize_, true});
            total += static_cast<long long>(hashmapSize_) * num_features_per_level;
            QuickMLP::Instance().getLogger()->debug(
                "HashGrid layer %d is sparse and will be hashed. Resolution=%d, hashmap size=%d", l, resolution,
                hashmapSize_);
        }
        CHECK_ERROR(total < (1ll << 31), "The HashGrid needs more than 2^31 parameters, which the 32-bit offsets cannot address");
    }
    numParameters_ = static_cast<int>(total);
}

EncodingHashGrid::EncodingHashGrid(const json& cfg)
    : EncodingHashGrid(cfg.at("start_in").get<int>(), cfg.at("n_in").get<int>(), cfg.at("n_levels").get<int>(),
                       cfg.at("n_features_per_level").get<int>(), cfg.at("log2_hashmap_size").get<int>(),
                       cfg.at("min_resolution").get<int>(), cfg.at("max_resolution").get<int>(),
                       parseCombinationMode(cfg.at("combination_mode")),
                       cfg.value("bounding_box_min", std::vector<float>()),
                       cfg.value("bounding_box_size", std::vector<float>()), parsePrecision(cfg))
{}

json EncodingHashGrid::toJson() const
{
    return json::object({
        {"id", id()},
        {"start_in", startChannel_},
        {"n_in", dimension_},
        {"n_levels", numLevels_},
        {"n_features_per_level", numFeaturesPerLevel_},
        {"log2_hashmap_size", log2HashmapSize_},
        {"min_resolution", minResolution_},
        {"max_resolution", maxResolution_},
        {"combination_mode", combinationMode_ == LayerCombinationMode::CONCAT ? "concat" : "add"},
        {"bounding_box_min", json(boundingBoxMin_)},
        {"bounding_box_size", json(boundingBoxSize_)},
        {"parameter_precision", parameterPrecision_ == Tensor::HALF ? "half" : "float"},
    });
}

std::string EncodingHashGrid::ID() { return "HashGrid"; }

std::string EncodingHashGrid::id() const { return ID(); }

int EncodingHashGrid::maxInputChannel() const { return startChannel_ + dimension_ - 1; }

int EncodingHashGrid::numOutputChannels() const
{
    switch (combinationMode_) {
    case LayerCombinationMode::CONCAT: return numLevels_ * numFeaturesPerLevel_;
    case LayerCombinationMode::ADD: return numFeaturesPerLevel_;
    default: throw std::runtime_error("Unknown enum");
    }
}

std::string EncodingHashGrid::configName() const
{
    // the generated configuration struct is a pure function of these values
    std::string key = format("%d_%d_%d_%d_%d_%d_%d_%d_%d", startChannel_, dimension_, numLevels_, numFeaturesPerLevel_,
                             log2HashmapSize_, minResolution_, maxResolution_,
                             static_cast<int>(combinationMode_), static_cast<int>(parameterPrecision_));
    return "HashGridCfg_" + format("%zx", std::hash<std::string>()(key));
}

std::string EncodingHashGrid::qualifiedName() const
{
    return "qmlp::kernel::EncodingHashGrid<qmlp::kernel::" + configName() + ">";
}

void EncodingHashGrid::fillCode(std::stringstream& code) const
{
    const std::string name = configName();
    code << KernelLoader::MainFile("qmlp/kernels/encoding_hashgrid.h");
    code << "#ifndef QMLP_DEFINED_" << name << "\n#define QMLP_DEFINED_" << name << "\n";
    code << "namespace qmlp { namespace kernel {\n";
    code << "struct " << name << "\n{\n";
    code << "    static constexpr int Start = " << startChannel_ << ";\n";
    code << "    static constexpr int Dim = " << dimension_ << ";\n";
    code << "    static constexpr int Levels = " << numLevels_ << ";\n";
    code << "    static constexpr int Features = " << numFeaturesPerLevel_ << ";\n";
    code << "    static constexpr bool Concat = "
         << (combinationMode_ == LayerCombinationMode::CONCAT ? "true" : "false") << ";\n";
    code << "    static constexpr bool ResolutionFactor = true;\n";
    code << "    static constexpr int ParameterCount = " << numParameters_ << ";\n";
    code << "    typedef " << (parameterPrecision_ == Tensor::HALF ? "f16" : "float") << " table_t;\n";
    auto emit = [&](const char* type, const char* field, auto getter) {
        code << "    static constexpr " << type << " " << field << "[" << numLevels_ << "] = {";
        for (int l = 0; l < numLevels_; ++l) code << (l ? ", " : "") << getter(layers_[l]);
        code << "};\n";
    };
    emit("int", "resolution", [](const HashGridLayerConfig& c) { return std::to_string(c.resolution); });
    emit("int", "memoryOffset", [](const HashGridLayerConfig& c) { return std::to_string(c.memoryOffset); });
    emit("unsigned", "hashGridSize",
         [](const HashGridLayerConfig& c) { return std::to_string(c.hashed ? c.hashGridSize : 1) + "u"; });
    emit("bool", "hashed", [](const HashGridLayerConfig& c) { return std::string(c.hashed ? "true" : "false"); });
    code << "};\n}}\n#endif\n";
}

bool EncodingHashGrid::hasParameters() const { return true; }

std::string EncodingHashGrid::parameterName() const
{
    return format("qmlp::kernel::HashGridParams<%s, %d>",
                  parameterPrecision_ == Tensor::HALF ? "qmlp::kernel::f16" : "float", ndim());
}

Tensor::Precision EncodingHashGrid::parameterPrecision(Tensor::Usage usage) const
{
    return usage == Tensor::INFERENCE ? parameterPrecision_ : Tensor::FLOAT;
}

int EncodingHashGrid::parameterCount() const { return numParameters_; }

int EncodingHashGrid::gatherRegistersPerPoint() const
{
    const int entryBytes = numFeaturesPerLevel_ * (parameterPrecision_ == Tensor::HALF ? 2 : 4);
    return std::max(1, ((1 << dimension_) * entryBytes + 3) / 4);
}

bool EncodingHashGrid::pointOrderKey(kernel::PointOrderKey& key, long long numPoints) const
{
    // Worth it if most of what a point gathers comes from dense levels (the entries of a cell's
    // corners are then close in memory for points that are close in space; a hashed level
    // spreads them over its table whatever the order) and if the largest of them exceeds the
    // 4 MB L2 of one accelerator die. Measured on a dense 32^4 grid with 8 fp16 features
    // (16.8 MB): 2^21 uniformly random points in 245 us as given, 77 us sorted by 32 x 32 slabs
    // of the two leading coordinates, 120-139 us sorted by the leading coordinate alone.
    const long long entryBytes = static_cast<long long>(numFeaturesPerLevel_) * (parameterPrecision_ == Tensor::HALF ? 2 : 4);
    long long denseBytes = 0, largestDense = 0, allBytes = 0;
    int largestResolution = 1;
    // The order pays off through lines of a table that several points of the batch share: per
    // dense level beyond the L2, gathers of the batch (2^(D-1) lines per point) per 128-byte
    // line of the level. Measured with 3-D grids: 32 gathers per line 1.3-1.8 x faster sorted
    // (256^3 x 2 fp16 at 2^22 points, 128^3..161^3 at 2^20), 8 per line no gain, 2-8 per line
    // (256^3 x 8 fp16, 268 MB) 13-38 % slower because of what the sort costs.
    constexpr long long MIN_GATHERS_PER_LINE = 24;
    bool denseEnough = false;
    for (int l = 0; l < numLevels_; ++l) {
        const int end = l + 1 < numLevels_ ? layers_[l + 1].memoryOffset : numParameters_;
        const long long bytes = static_cast<long long>(end - layers_[l].memoryOffset) / numFeaturesPerLevel_ * entryBytes;
        allBytes += bytes;
        if (!layers_[l].hashed) {
            denseBytes += bytes;
            if (bytes > largestDense) largestResolution = layers_[l].resolution;
            largestDense = std::max(largestDense, bytes);
            if (bytes >= (4ll << 20) && numPoints * (1ll << (dimension_ - 1)) * 128 >= MIN_GATHERS_PER_LINE * bytes)
                denseEnough = true;
        }
    }
    key = kernel::PointOrderKey{};
    key.slabs0 = key.slabs1 = key.slabs2 = 1;
    if (largestDense < (4ll << 20) || 2 * denseBytes < allBytes) return hashedPointOrderKey(key, numPoints);
    if (numPoints > 0 && !denseEnough) return false;
    // slabs of whole cells of the largest dense level (a slab that cuts through cells makes its
    // points gather from one more layer of entries per coordinate)
    const int slabsPerCoordinate = dimension_ > 1 ? 32 : 1024;
    const int cells = std::max(1, largestResolution - 1);
    const int cellsPerSlab = (cells + slabsPerCoordinate - 1) / slabsPerCoordinate;
    const int slabs = (cells + cellsPerSlab - 1) / cellsPerSlab;
    const float slabsPerUnit = static_cast<float>(cells) / static_cast<float>(cellsPerSlab);
    key.channel0 = startChannel_;
    key.channel1 = startChannel_ + (dimension_ > 1 ? 1 : 0);
    key.slabs0 = slabs;
    key.slabs1 = dimension_ > 1 ? slabs : 1;
    key.min0 = boundingBoxMin_[0];
    key.min1 = boundingBoxMin_[dimension_ > 1 ? 1 : 0];
    key.scale0 = slabsPerUnit * boundingBoxInvSize_[0];
    key.scale1 = slabsPerUnit * boundingBoxInvSize_[dimension_ > 1 ? 1 : 0];
    return true;
}

bool EncodingHashGrid::hashedPointOrderKey(kernel::PointOrderKey& key, long long numPoints) const
{
    // A multi-level grid with hashed levels: its tables are swept level by level and stay in the L2, so an order
    // of the batch does not pay through the caches but through the lanes of a gather instruction: 64 points that are
    // close in space ask for few lines of a level whose cells are larger than the distance between the points, and
    // the instruction then costs its issue (17 to 35 cycles of the address unit) instead of 2.3 cycles per line. The
    // two corners along coordinate 0 lie in the same line of a hashed level (its multiplier is 1), the corners along
    // the other coordinates anywhere: so the slabs cut coordinates 1 and 2 and leave coordinate 0 whole.
    // Measured on 16 levels of 2^19 entries x 2 fp16 (resolutions 16 .. 4096), 2^20 uniform points, 32 x 32 slabs
    // numbered along a Z curve: the fused kernel takes 245 instead of 277 us (227 us on a batch that arrives in this
    // order; the scattered result rows cost the difference) -- the levels from resolution 300 on have more cells than
    // the batch has points and keep their four lines per point, 8 levels x 20 us. The sort takes 37 us
    // (9 + 5 + 23 us), more than it gains: offered when the caller asks for it (options.sort_points = 1, e.g. to
    // amortise one sort over several networks that share a batch), never chosen by itself.
    if (dimension_ < 2 || numLevels_ < 2 || numPoints > 0) return false;
    key.channel0 = startChannel_;
    key.min0 = boundingBoxMin_[0];
    key.scale0 = boundingBoxInvSize_[0];
    key.slabs0 = 1;
    const int slabs = dimension_ > 2 ? 32 : 1024;
    key.channel1 = startChannel_ + 1;
    key.min1 = boundingBoxMin_[1];
    key.scale1 = static_cast<float>(slabs) * boundingBoxInvSize_[1];
    key.slabs1 = slabs;
    if (dimension_ > 2) {
        key.channel2 = startChannel_ + 2;
        key.min2 = boundingBoxMin_[2];
        key.scale2 = static_cast<float>(slabs) * boundingBoxInvSize_[2];
        key.slabs2 = slabs;
        key.interleave12 = 1;
    }
    return true;
}

int EncodingHashGrid::ldsGradientFloats(int maxBytes, int& levels) const
{
    levels = 0;
    // the device code scatters per tile only for these feature counts (HasTileScatter)
    const int F = numFeaturesPerLevel_;
    if ((F & (F - 1)) != 0 || 2 * F > 64) return 0;
    int floats = 0;
    for (int l = 0; l < numLevels_; ++l) {
        const int end = l + 1 < numLevels_ ? layers_[l + 1].memoryOffset : numParameters_;
        const int upTo = end - layers_[0].memoryOffset;
        if (static_cast<long long>(upTo) * static_cast<long long>(sizeof(float)) > maxBytes) break;
        levels = l + 1;
        floats = upTo;
    }
    return floats;
}

bool EncodingHashGrid::gradientSlices(GradientSliceLayout& layout) const
{
    if (dimension_ > 4 || numParameters_ >= (1 << 30)) return false;   // up to 8 records per point and level in registers
    const int lds = FusedNetwork::MaxSharedMemoryBytes();
    // the slice kernel sums in 64-bit fixed point: 8 bytes of LDS per element
    // Slices of 8192 sums (64 KiB, two workgroups of the slice kernel per compute unit: one streams records while the
    // other zeroes or writes back; a train step of a 16-level hash grid 0.557 -> 0.533 ms) where no level then has
    // more than 512 of them, else of 16384.
    int largestLevel = 0;
    for (int l = 0; l < numLevels_; ++l)
        largestLevel = std::max(largestLevel, (l + 1 < numLevels_ ? layers_[l + 1].memoryOffset : numParameters_) - layers_[l].memoryOffset);
    const int smallSlice = 8192 / numFeaturesPerLevel_ * numFeaturesPerLevel_;
    const int sliceSums = smallSlice > 0 && divUp(largestLevel, smallSlice) <= 512 ? 8192 : 16384;
    const int entries = std::min(sliceSums, lds / 8) / numFeaturesPerLevel_;
    if (entries < 64) return false;
    layout = GradientSliceLayout{};
    layout.sliceFloats = entries * numFeaturesPerLevel_;
    layout.configType = "qmlp::kernel::" + configName();
    layout.pairs = std::max(1, (1 << dimension_) / 2);
    // as GridGradientLayout::RECORD_WORDS: two 16-bit offsets, two weights, the adjoint halves, padded to 16 / 32 bytes
    const int usedWords = 3 + (numFeaturesPerLevel_ + 1) / 2;
    layout.recordWords = usedWords % 4 == 3 ? usedWords + 1 : usedWords;
    // the records of a workgroup and level are sorted in LDS: 96 KiB for them, the rest for the book-keeping
    int points = 1024;
    while (points > 64 && points * layout.pairs * layout.recordWords * 4 > 96 * 1024) points /= 2;
    layout.pointsPerWorkgroup = points;
    {
        // as kernel::PositionDerivativeLayout: Dim * Features values per level in the precision of the table, in whole chunks of 16 bytes
        // Kept where they are at most 32 bytes per point and level. The gathers they save the adjoint pass cost a
        // line of the L2 per pair of corners in a hashed level (a 3-D grid with 2 half features: 4 lines against 16
        // bytes of derivatives; records kernel of 16 such levels at 2^18 points 197 -> 126 us, forward pass 96 ->
        // 103 us). A dense 4-D grid with 8 features would keep 64 bytes per point, which its forward kernel (4 tiles
        // per wavefront, 64 registers of gathered entries per point) no longer holds in registers (219 -> 736 us),
        // while its gathers of a batch sorted by slab mostly hit the L1 anyway (records kernel 281 -> 256 us).
        const int perChunk = parameterPrecision_ == Tensor::HALF ? 8 : 4;
        const int chunks = divUp(dimension_ * numFeaturesPerLevel_, perChunk);
        layout.derivativeBytesPerPoint = chunks <= 2 ? numLevels_ * chunks * 16 : 0;
    }
    if (layout.recordsLdsBytes(points) > lds) return false;
    // every level gets about this many work items: the bucket of a slice that holds more than its share is split
    constexpr int ITEMS_PER_LEVEL = 32;
    for (int l = 0; l < numLevels_; ++l) {
        const int begin = layers_[l].memoryOffset;
        const int end = l + 1 < numLevels_ ? layers_[l + 1].memoryOffset : numParameters_;
        const int count = divUp(end - begin, layout.sliceFloats);
        if (count > 512) return false;   // the records kernel keeps a histogram of 512 slices
        layout.slicesPerLevel.push_back(count);
        const int parts = std::max(1, ITEMS_PER_LEVEL / count);
        for (int k = 0; k < count; ++k)
            for (int part = 0; part < parts; ++part)
                layout.items.push_back({l, static_cast<unsigned>(begin + k * layout.sliceFloats),
                                        std::min(layout.sliceFloats, end - begin - k * layout.sliceFloats), k, part, parts, 0, 0});
    }
    return true;
}

bool EncodingHashGrid::gradientColumns(const kernel::PointOrderKey& key, GradientColumnLayout& layout) const
{
    // one dense level whose batch is sorted by slabs of whole cells of its first two coordinates
    if (numLevels_ != 1 || layers_[0].hashed || dimension_ < 2 || dimension_ > 4) return false;
    kernel::PointOrderKey own{};
    if (!pointOrderKey(own, 0) || own.slabs2 != 1 || own.slabs0 != own.slabs1) return false;
    if (key.channel0 != own.channel0 || key.channel1 != own.channel1 || key.slabs0 != own.slabs0 || key.slabs1 != own.slabs1
        || key.slabs2 != own.slabs2 || key.scale0 != own.scale0 || key.scale1 != own.scale1 || key.min0 != own.min0 || key.min1 != own.min1)
        return false;   // sorted for another encoding
    const int nodes = layers_[0].resolution;
    const int cells = std::max(1, nodes - 1);
    const int cellsPerSlab = divUp(cells, own.slabs0);
    if (divUp(cells, cellsPerSlab) != own.slabs0) return false;
    long long sums = static_cast<long long>(cellsPerSlab) * cellsPerSlab * numFeaturesPerLevel_;
    long long region = static_cast<long long>(cellsPerSlab + 1) * (cellsPerSlab + 1) * numFeaturesPerLevel_;
    for (int d = 2; d < dimension_; ++d) {
        sums *= nodes;
        region *= nodes;
    }
    // as GridGradientColumns::LDS_BYTES: the 64-bit sums of an owner, later the entries of the table around its slab;
    // two workgroups per compute unit
    const long long ldsBytes = roundUp<long long>(std::max(sums * 8, region * (parameterPrecision_ == Tensor::HALF ? 2 : 4)), 16);
    if (ldsBytes > (FusedNetwork::MaxSharedMemoryBytes() - 1024) / 2) return false;
    layout.configType = "qmlp::kernel::" + configName();
    layout.cellsPerSlab = cellsPerSlab;
    layout.owners = divUp(nodes, cellsPerSlab);
    layout.ldsBytes = static_cast<int>(ldsBytes);
    return true;
}

void EncodingHashGrid::setParameter(const Tensor& tensor, Tensor::Usage usage)
{
    if (tensor.defined()) {
        CHECK_DTYPE(tensor, parameterPrecision(usage));
        CHECK_DIM(tensor, 1);
        CHECK_SIZE(tensor, 0, parameterCount());
        CHECK_ERROR(tensor.stride(0) == 1, "The grid parameters must be contiguous");
        CHECK_ERROR(reinterpret_cast<uintptr_t>(tensor.rawPtr()) % 16 == 0,
                    "The grid parameters must be aligned to 16 bytes");
    }
    if (usage == Tensor::INFERENCE)
        parametersForward_ = tensor;
    else
        parametersGradients_ = tensor;
}

int EncodingHashGrid::fillParameterMemory(char* dst, int dstSize)
{
    // mirrors qmlp::kernel::HashGridParams<T, D>: two pointers, then 2*D floats
    const int needed = static_cast<int>(2 * sizeof(void*) + 2 * dimension_ * sizeof(float));
    CHECK_ERROR(dstSize >= needed, "parameter buffer too small");
    const void* fwd = parametersForward_.defined() ? parametersForward_.rawPtr() : nullptr;
    void* bwd = parametersGradients_.defined() ? parametersGradients_.rawPtr() : nullptr;
    std::memcpy(dst, &fwd, sizeof(void*));
    std::memcpy(dst + sizeof(void*), &bwd, sizeof(void*));
    std::memcpy(dst + 2 * sizeof(void*), boundingBoxMin_.data(), dimension_ * sizeof(float));
    std::memcpy(dst + 2 * sizeof(void*) + dimension_ * sizeof(float), boundingBoxInvSize_.data(),
                dimension_ * sizeof(float));
    return roundUp(needed, 8);
}

void EncodingHashGrid::zeroGradients()
{
    if (parametersGradients_.defined()) parametersGradients_.zero_();
}

QUICKMLP_NAMESPACE_END
