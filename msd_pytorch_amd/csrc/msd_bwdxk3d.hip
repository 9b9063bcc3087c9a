// fused backward_x + backward_k, 3D instantiations (one file per rank and variant so they compile in parallel).
#include "msd_bwdxk_impl.h"

namespace msd {

bool fast_backward_xkb_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                    const View<float> &gx)
{
    return bwdxk::xkb_mode<3>(g, gy, x, gx) != bwdxk::kUnsupported;
}

hipError_t fast_backward_xkb_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                                const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws,
                                hipStream_t s, ReduceJob *defer)
{
    switch (bwdxk::xkb_mode<3>(g, gy, x, gx)) {
    case bwdxk::kPlain: return bwdxk::xkb_nd<3, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer);
    case bwdxk::kLong: return fast_backward_xkb_3d_long(g, gy, x, k, gx, pm, gk, gb, ws, s, defer);
    default: return hipErrorInvalidConfiguration;
    }
}

bool fast_backward_k_pair_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x)
{
    return bwdxk::k_pair_supported_3d(g, gy, x);
}

hipError_t fast_backward_k_pair_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk,
                                   float *gb, float *ws, hipStream_t s, ReduceJob *defer, const LayerGroup *group)
{
    return bwdxk::k_pair_3d(g, gy, x, gk, gb, ws, s, defer, group);
}

bool fast_backward_k_only_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x)
{
    return bwdxk::k_only_supported_3d(g, gy, x);
}

hipError_t fast_backward_k_only_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk,
                                   float *gb, float *ws, hipStream_t s)
{
    return bwdxk::k_only_3d(g, gy, x, gk, gb, ws, s);
}

}  // namespace msd
