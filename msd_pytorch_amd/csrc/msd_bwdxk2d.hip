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
                                hipStream_t s, ReduceJob *defer, const LayerPair *pair)
{
    if (pair && (g.Wd != 2 || g.dil != std::max(pair->dil0, pair->dil1))) return hipErrorInvalidValue;
    switch (bwdxk::xkb_mode<2>(g, gy, x, gx)) {
    case bwdxk::kPlain: return bwdxk::xkb_nd<2, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, pair);
    case bwdxk::kLong: return fast_backward_xkb_2d_long(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, pair);
    default: return hipErrorInvalidConfiguration;
    }
}

}  // namespace msd
