// Internal interface between the C ABI (msd_api.hip) and the kernel files.
#pragma once

#include "msd_common.h"

namespace msd {

// Upper bound on the number of partial-sum rows of the weight/bias gradient
// reduction (one row per workgroup of the first pass).
constexpr int kMaxPartialRows = 512;

// Scratch elements needed by generic_backward_kb for this geometry.
int64_t generic_workspace_elems(const Geom &g);

template <typename T>
hipError_t generic_forward(const Geom &g, bool relu, View<const T> x, const T *k, const T *bias, View<T> out,
                           hipStream_t s);

template <typename T>
hipError_t generic_backward_x(const Geom &g, bool relu, View<const T> out, View<const T> gy, const T *k, View<T> gx,
                              hipStream_t s);

// gk and/or gb may be null (that gradient is then skipped).
template <typename T>
hipError_t generic_backward_kb(const Geom &g, bool relu, View<const T> out, View<const T> gy, View<const T> x, T *gk,
                               T *gb, T *ws, hipStream_t s);

}  // namespace msd
