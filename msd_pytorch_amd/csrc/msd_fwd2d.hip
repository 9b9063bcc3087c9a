// forward, 2D instantiations (one file per rank so they compile in parallel).
#include "msd_fwd_impl.h"

namespace msd {

bool fast_forward_supported_2d(const Geom &g, const View<const float> &x, const View<float> &out)
{
    return fwd::supported_nd<2>(g, x, out);
}

hipError_t fast_forward_2d(const Geom &g, bool relu, const View<const float> &x, const float *k, const float *bias,
                            const View<float> &out, hipStream_t s)
{
    return fwd::run_nd<2>(g, relu, x, k, bias, out, s);
}

}  // namespace msd
