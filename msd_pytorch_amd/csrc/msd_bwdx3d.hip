// backward_x, 3D instantiations (one file per rank so they compile in parallel).
#include "msd_bwdx_impl.h"

namespace msd {

bool fast_backward_x_supported_3d(const Geom &g, bool relu, const View<const float> &out,
                                   const View<const float> &gy, const View<float> &gx)
{
    return bwdx::fast_backward_x_supported_nd<3>(g, relu, out, gy, gx);
}

hipError_t fast_backward_x_3d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                               const float *k, const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    // one input and one output channel: the lean kernel ("bwdx.lean1" = 0: the general one)
    if (!relu && knob(kKnobBwdxLean1, 1) && bwdx::one_channel_vec<3>(g, gy, gx, pm) != 0)
        return bwdx::one_channel_nd<3>(g, gy, k, gx, pm, s);
    return bwdx::fast_backward_x_nd<3>(g, relu, out, gy, k, gx, pm, s);
}

bool fast_backward_x_pair_supported_3d(const Geom &g, const View<const float> &gy, const View<float> &gx)
{
    return bwdx::pair_vec<3>(g, gy, gx) != 0;
}

hipError_t fast_backward_x_pair_3d(const Geom &g, const View<const float> &gy, const float *k, const View<float> &gx,
                                   const PostMask &pm, hipStream_t s, const LayerGroup *group)
{
    return bwdx::pair_nd<3>(g, gy, k, gx, pm, s, group);
}

}  // namespace msd
