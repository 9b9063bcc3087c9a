// fused backward_x + backward_k, 2D instantiations (one file per rank and variant so they compile in parallel).
#include "msd_bwdxk_impl.h"

namespace msd {

bool fast_backward_xkb_supported_2d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                    const View<float> &gx)
{
    return bwdxk::xkb_mode<2>(g, gy, x, gx) != bwdxk::kUnsupported;
}

hipError_t fast_backward_xkb_2d(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                                const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws,
                                hipStream_t s, ReduceJob *defer, const LayerGroup *group)
{
    if (group) {
        if (group->n != g.Wd || group->n < 2 || group->n > kMaxLayerGroup) return hipErrorInvalidValue;
        int dmax = 0;
        for (int j = 0; j < group->n; j++) dmax = std::max(dmax, group->dil[j]);
        if (g.dil != dmax) return hipErrorInvalidValue;
    }
    switch (bwdxk::xkb_mode<2>(g, gy, x, gx)) {
    case bwdxk::kPlain: return bwdxk::xkb_nd<2, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
    case bwdxk::kLong: return fast_backward_xkb_2d_long(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
    default: return hipErrorInvalidConfiguration;
    }
}

}  // namespace msd
