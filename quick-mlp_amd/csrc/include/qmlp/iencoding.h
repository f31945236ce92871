#pragma once

#include "common.h"
#include "json.h"
#include "kernel_loader.h"
#include "tensor.h"
#include <qmlp/kernels/point_order_key.h>

#include <functional>
#include <optional>
#include <sstream>
#include <unordered_map>
#include <vector>

QUICKMLP_NAMESPACE_BEGIN

/**
 * Defines an input encoding.
 *
 * What the device-side implementation must provide:
 * <code>
 * struct NameOfEncoding
 * {
 *     static constexpr int NumOutputs;
 *     template<typename I, typename O>
 *     static __device__ void forward(const I& input, O& output [, const param-type& params ]);
 *
 *     template<bool EvaluateInputGradients, bool EvaluateParameterGradients, typename I, typename O, typename AdjI>
 *     static __device__ void adjoint(const I& input, const O& adjOutput, AdjI& adjInput [, const param-type& params ]);
 * }
 * </code>
 * 'input' is indexable with operator[] and yields the raw float inputs of one point;
 * 'output' is indexable, assignable and has a typedef ValueType (float or a half type).
 * Encodings with parameters receive them as one by-value kernel argument of the type
 * named by parameterName(), whose bytes fillParameterMemory() produces.
 */
class IEncoding
{
public:
    virtual ~IEncoding() = default;

    [[nodiscard]] virtual json toJson() const = 0;
    [[nodiscard]] virtual std::string id() const = 0;

    /** The maximal addressed input channel, e.g. 2 for a 3D index. */
    [[nodiscard]] virtual int maxInputChannel() const = 0;

    /** The number of output channels */
    [[nodiscard]] virtual int numOutputChannels() const = 0;

    /** The qualified device type of the encoding including all template arguments. */
    [[nodiscard]] virtual std::string qualifiedName() const = 0;

    /** Appends the device code needed by qualifiedName(): includes and generated definitions. */
    virtual void fillCode(std::stringstream& code) const = 0;

    /** True iff the encoding has a parameter structure (and trainable parameters). */
    [[nodiscard]] virtual bool hasParameters() const { return false; }

    /** Fully-qualified device type of the parameter structure. */
    [[nodiscard]] virtual std::string parameterName() const { return ""; }

    [[nodiscard]] virtual Tensor::Precision parameterPrecision(Tensor::Usage usage) const { return Tensor::FLOAT; }

    [[nodiscard]] virtual int parameterCount() const { return 0; }

    /**
     * Sets the underlying parameter to the specified tensor: 1D with parameterCount()
     * entries of type parameterPrecision(usage). An undefined tensor clears it.
     */
    virtual void setParameter(const Tensor& tensor, Tensor::Usage usage) {}

    /** True iff a tensor is currently bound for this usage (always true without parameters). */
    [[nodiscard]] virtual bool hasParameterTensor(Tensor::Usage usage) const { return true; }

    /**
     * Writes the bytes of the parameter structure (kernel argument) into 'dst' with a
     * capacity of 'dstSize' bytes; returns the number of bytes written.
     */
    [[nodiscard]] virtual int fillParameterMemory(char* dst, int dstSize) { return 0; }

    /** Zeros the gradients of this encoding's parameters (no-op without parameters). */
    virtual void zeroGradients() {}

    /**
     * For the fused backward kernel: how many leading levels (or other leading parts) of the
     * parameter gradients a workgroup may sum in LDS before adding them to the gradient
     * tensor, if it has maxBytes of LDS for that. Returns the number of floats needed (0: none)
     * and sets 'levels', which the device code receives as scatterTile<levels>.
     */
    /**
     * Number of parameter tables that the fused forward kernel sweeps one after the other
     * (the levels of a grid). With two or more, the workgroups of a launch should stay in
     * step so that only the table in use occupies the L2; 0 for encodings without tables.
     */
    [[nodiscard]] virtual int numSweptTables() const { return 0; }

    /**
     * 32-bit registers that the gathers of one point from one table occupy while they are in
     * flight (all corners of a cell); 0 for encodings that gather nothing. The fused forward
     * kernel keeps the gathers of several points per lane in flight and sizes that number by it.
     */
    [[nodiscard]] virtual int gatherRegistersPerPoint() const { return 0; }

    /**
     * Encodings that gather from a table too large for the L2 of one accelerator die, and whose
     * gathers are close in memory for points that are close in space (dense grids), fill in how
     * points are assigned to slabs of that table and return true: the fused inference kernel
     * then evaluates the points slab by slab.
     * \param numPoints size of the batch; >0: only say yes if so many points are also expected
     *   to gain more from the order than the sort costs. 0: say whether an order exists at all.
     */
    [[nodiscard]] virtual bool pointOrderKey(kernel::PointOrderKey& key, long long numPoints = 0) const
    {
        (void)key;
        (void)numPoints;
        return false;
    }

    /** Output channels that the device code writes together (the features of a grid entry). */
    [[nodiscard]] virtual int channelsWrittenTogether() const { return 1; }

    /** One work item of GridGradientSlicesKernel (mirrors kernel::GridGradientSlice). */
    struct GradientSlice
    {
        int level;
        unsigned first;
        int floats;
        int slice;
        int part;
        int parts;
        int reserved0;
        int reserved1;
    };
    /** What the host needs to run the kernels of kernels/grid_gradient.h for an encoding. */
    struct GradientSliceLayout
    {
        std::string configType;            // device type of the level table
        int sliceFloats = 0;               // floats of a full slice (= LDS of the slice kernel / 4)
        int recordWords = 0;               // 32-bit words of a record
        int pairs = 0;                     // records per point and level
        int pointsPerWorkgroup = 0;        // most lanes of a workgroup of the records kernel (a power of two)
        int derivativeBytesPerPoint = 0;   // of kernel::PositionDerivativeLayout: what a training pass may keep for the input gradients
        /** Dynamic LDS of the records kernel with this many lanes: its records of one level with the slice of each
         *  (16 bits), and per slice of the level (at most 512) room in the bucket, count and place among the records. */
        int recordsLdsBytes(int points) const { return points * pairs * (recordWords * 4 + 2) + 512 * 8 + (2 * 512 + 1) * 4 + 64; }
        std::vector<int> slicesPerLevel;
        std::vector<GradientSlice> items;  // one workgroup of the slice kernel each
        /** Records a bucket of level l holds for a batch of numel points (as in the device code). */
        long long capacity(int l, long long numel) const { return ((5 * numel * pairs / 4) / slicesPerLevel[l] + 2048) & ~3ll; }
        long long totalRecords(long long numel) const
        {
            long long n = 0;
            for (size_t l = 0; l < slicesPerLevel.size(); ++l) n += slicesPerLevel[l] * capacity(static_cast<int>(l), numel);
            return n;
        }
        int numBuckets() const
        {
            int n = 0;
            for (int s : slicesPerLevel) n += s;
            return n;
        }
    };
    /** What the host needs to run the kernels of kernels/grid_gradient_columns.h for an encoding. */
    struct GradientColumnLayout
    {
        std::string configType;      // device type of the level table
        int cellsPerSlab = 0;        // cells per slab and sorted coordinate (the kernels' CPS)
        int owners = 0;              // owners per sorted coordinate: workgroups that share out the nodes of the grid
        int ldsBytes = 0;            // 64-bit sums of one owner
    };
    /**
     * Encodings whose parameter gradients, for a batch that is sorted by the slabs of `key` (pointOrderKey()), can
     * be summed owner by owner in LDS without any records (see kernels/grid_gradient_columns.h) return true and
     * fill in the layout.
     */
    [[nodiscard]] virtual bool gradientColumns(const kernel::PointOrderKey& key, GradientColumnLayout& layout) const
    {
        (void)key;
        (void)layout;
        return false;
    }

    /**
     * Encodings whose parameter gradients can be summed slice by slice in LDS instead of being
     * scattered with global atomics (see kernels/grid_gradient.h) return true and fill in the layout.
     */
    [[nodiscard]] virtual bool gradientSlices(GradientSliceLayout& layout) const
    {
        (void)layout;
        return false;
    }

    [[nodiscard]] virtual int ldsGradientFloats(int maxBytes, int& levels) const
    {
        levels = 0;
        return 0;
    }

    /**
     * Standalone forward pass.
     * \param input shape (B, Cin), float32
     * \param output shape (B, >= numOutputChannels()), float32, unit stride along the channels
     * \param parametersForward optional override of the inference parameters for this call
     */
    virtual void forward(const Tensor& input, Tensor& output, stream_t stream,
                         const std::optional<const Tensor>& parametersForward);

    enum AdjointMode
    {
        INPUT_GRADIENTS = 0x1,
        PARAM_GRADIENTS = 0x2,
        ALL_GRADIENTS = INPUT_GRADIENTS | PARAM_GRADIENTS
    };

    /**
     * Standalone adjoint pass; adjInput (B, Cin) and the parameter gradients are accumulated.
     */
    virtual void adjoint(const Tensor& input, const Tensor& adjOutput, Tensor& adjInput, stream_t stream,
                         const std::optional<const Tensor>& parametersForward,
                         const std::optional<const Tensor>& parametersGradients,
                         int adjointMode = AdjointMode::ALL_GRADIENTS);

    /**
     * Compiles the standalone forward kernel and, for adjointMode > 0, the adjoint kernel of
     * that mode into the kernel cache without loading them; needs no GPU.
     */
    void precompile(int adjointMode = AdjointMode::ALL_GRADIENTS);

private:
    std::string forwardKernelSource() const;
    std::string adjointKernelSource(int adjointMode) const;
    std::optional<KernelFunction> forwardKernel_;
    std::optional<KernelFunction> adjointKernel_[AdjointMode::ALL_GRADIENTS + 1];
};
typedef std::shared_ptr<IEncoding> IEncoding_ptr;

/**
 * Encodings over a bounded volume; can serve as child of other encodings.
 */
class IVolumetricEncoding : public IEncoding
{
public:
    [[nodiscard]] virtual int ndim() const = 0;

    typedef std::vector<float> BoundingBoxVector_t;
    [[nodiscard]] virtual BoundingBoxVector_t boundingBoxMin() const = 0;
    [[nodiscard]] virtual BoundingBoxVector_t boundingBoxSize() const = 0;
    [[nodiscard]] virtual BoundingBoxVector_t boundingBoxInvSize() const = 0;
};

class EncodingFactory
{
private:
    EncodingFactory();
    typedef std::function<IEncoding_ptr(const json&)> factory_t;
    std::unordered_map<std::string, factory_t> encodings_;

public:
    static EncodingFactory& Instance();
    IEncoding_ptr create(const json& cfg);
};

QUICKMLP_NAMESPACE_END
