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
    return bwdx::fast_backward_x_nd<3>(g, relu, out, gy, k, gx, pm, s);
}

}  // namespace msd
