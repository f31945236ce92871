#pragma once
// How the points of a batch are assigned to slabs of a grid before they are sorted:
// passed by value to the point-order kernels. The same definition is compiled by the host
// code and, at run time, by the device compiler.

namespace qmlp { namespace kernel {

struct PointOrderKey
{
    int channel0, channel1, channel2;   // input channels of up to three grid coordinates (unused where slabs == 1)
    int slabs0, slabs1, slabs2;         // slabs per coordinate, slabs0 * slabs1 * slabs2 <= 1024
    float min0, min1, min2;             // lower corner of the grid's bounding box
    float scale0, scale1, scale2;       // slabs / extent of the bounding box
    // 1: the slabs of coordinates 1 and 2 (equal powers of two) are numbered along a Z curve instead of row by row,
    // so that the slabs a workgroup walks through one after the other are neighbours in both coordinates
    int interleave12;
};

}} // namespace qmlp::kernel
