#pragma once
// How the points of a batch are assigned to slabs of a dense grid before they are sorted:
// passed by value to the point-order kernels. The same definition is compiled by the host
// code and, at run time, by the device compiler.

namespace qmlp { namespace kernel {

struct PointOrderKey
{
    int channel0, channel1;   // input channels of the two leading grid coordinates (channel1 unused if slabs1 == 1)
    int slabs0, slabs1;       // slabs per coordinate, slabs0 * slabs1 <= 1024
    float min0, min1;         // lower corner of the grid's bounding box
    float scale0, scale1;     // slabs / extent of the bounding box
};

}} // namespace qmlp::kernel
