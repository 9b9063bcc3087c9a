// fused backward_x + backward_k, 2D instantiations of the variant for long rows and big stacks.
#include "msd_bwdxk_impl.h"

namespace msd {

hipError_t fast_backward_xkb_2d_long(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                     const float *k, const View<float> &gx, const PostMask &pm, float *gk, float *gb,
                                     float *ws, hipStream_t s, ReduceJob *defer, const LayerGroup *group)
{
    return bwdxk::xkb_nd<2, true>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
}

}  // namespace msd
