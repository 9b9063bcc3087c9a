// fused backward_x + backward_k, 3D instantiations (one file per rank so they compile in parallel).
#include "msd_bwdxk_impl.h"

namespace msd {

bool fast_backward_xkb_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                    const View<float> &gx)
{
    return bwdxk::xkb_supported_nd<3>(g, gy, x, gx);
}

hipError_t fast_backward_xkb_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                                const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws,
                                hipStream_t s, ReduceJob *defer)
{
    return bwdxk::xkb_nd<3>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer);
}

}  // namespace msd
