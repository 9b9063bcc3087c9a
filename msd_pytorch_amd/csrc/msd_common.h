// Shared host/device definitions for the gfx950 dilated-convolution kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace msd {

constexpr int kWave = 64;  // CDNA wavefront width

// MI355X has 8 accelerator dies (XCDs), each with its own L2; workgroups are
// handed to the XCDs round-robin in launch order.  block_for_xcd() renumbers
// the workgroups of a grid whose x extent is a multiple of kXcds so that each
// XCD works on one contiguous range of logical blocks (neighbouring rows and
// planes, whose halos overlap, then share an L2).  Logical ids >= nblocks are
// padding and must exit.
constexpr int kXcds = 8;

inline int xcd_grid(int nblocks) { return (nblocks + kXcds - 1) / kXcds * kXcds; }

__device__ __forceinline__ int block_for_xcd(int bid, int grid, bool remap)
{
    return remap ? (bid % kXcds) * (grid / kXcds) + bid / kXcds : bid;
}

// Problem geometry.  2D problems are carried as D == 1 with NDIM == 2 kernels
// that have no z taps.
struct Geom {
    int ndim;
    int B, C, Wd;       // batch, input channels, output channels
    int D, H, W;        // spatial extents (D == 1 in 2D)
    int dil;
    int nvox;           // D * H * W, checked on the host to fit in 31 bits
    int reverse;        // walk the input channels from the last to the first (same sums, other order);
                        // set by the dense block's layer loops for every second layer
};

// Strided view: element strides {batch, channel, z, y, x}.
template <typename T>
struct View {
    T *p;
    int64_t sb, sc, sz, sy, sx;
};

// Symmetric index fold: -1 -> 0, n -> n-1 (the edge sample is repeated).
// Same map as the reference's reflect(), kernel_utils.cuh:30-38.
__host__ __device__ __forceinline__ int reflect_idx(int i, int n)
{
    return i < 0 ? -i - 1 : (i >= n ? 2 * n - i - 1 : i);
}

// Adjoint of the fold along one axis.  The forward pass reads, for weight tap
// t in {0,1,2}, the input at reflect(y + (t-1)*dil).  For an input coordinate
// h the output coordinates y that read h through tap t are at most two:
//   t = 0:  y = h + dil        (if < n)      and  y = dil - h - 1      (if h < dil)
//   t = 1:  y = h
//   t = 2:  y = h - dil        (if >= 0)     and  y = 2n - h - 1 - dil (if h + dil >= n)
// The reference's backward_x kernels express the same set through a swapped
// weight tap per slot (conv2d_backward_x.cu:153-185); this form keeps the
// weight index uniform across lanes.
struct AxisSources {
    int c[3][2];
    bool ok[3][2];
};

__device__ __forceinline__ AxisSources adjoint_sources(int h, int n, int dil)
{
    AxisSources s;
    s.c[0][0] = h + dil;              s.ok[0][0] = h + dil < n;
    s.c[0][1] = dil - h - 1;          s.ok[0][1] = h < dil;
    s.c[1][0] = h;                    s.ok[1][0] = true;
    s.c[1][1] = 0;                    s.ok[1][1] = false;
    s.c[2][0] = h - dil;              s.ok[2][0] = h >= dil;
    s.c[2][1] = 2 * n - h - 1 - dil;  s.ok[2][1] = h + dil >= n;
    return s;
}

__device__ __forceinline__ AxisSources single_source()
{
    AxisSources s;
    for (int t = 0; t < 3; t++) {
        s.c[t][0] = 0; s.ok[t][0] = (t == 0);
        s.c[t][1] = 0; s.ok[t][1] = false;
    }
    return s;
}

}  // namespace msd
