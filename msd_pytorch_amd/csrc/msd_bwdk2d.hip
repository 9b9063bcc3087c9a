// backward_k, 2D instantiations (one file per rank so they compile in parallel).
#include "msd_bwdk_impl.h"

namespace msd {

bool fast_backward_kb_supported_2d(const Geom &g, bool relu, const View<const float> &out,
                                    const View<const float> &gy, const View<const float> &x)
{
    return bwdk::supported_nd<2>(g, relu, out, gy, x);
}

hipError_t fast_backward_kb_2d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                                const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    return bwdk::run_nd<2>(g, relu, out, gy, x, gk, gb, ws, s);
}

}  // namespace msd
