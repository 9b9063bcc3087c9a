// Internal interface between the C ABI (msd_api.hip) and the kernel files.
#pragma once

#include "msd_common.h"

namespace msd {

// Upper bound on the number of partial-sum rows of the weight/bias gradient
// reduction (one row per workgroup of the first pass).
constexpr int kMaxPartialRows = 1024;

// Elements at the start of the workspace that hold the masked output gradient
// of the matrix-core backward_k (a multiple of 64 so the partial sums behind it
// stay aligned).
inline int64_t backward_k_mask_floats(const Geom &g) { return ((int64_t)g.B * g.Wd * g.nvox + 63) / 64 * 64; }

// Scratch elements any backward_k / backward_bias path needs for this geometry.
int64_t generic_workspace_elems(const Geom &g);

template <typename T>
hipError_t generic_forward(const Geom &g, bool relu, View<const T> x, const T *k, const T *bias, View<T> out,
                           hipStream_t s);

template <typename T>
hipError_t generic_backward_x(const Geom &g, bool relu, View<const T> out, View<const T> gy, const T *k, View<T> gx,
                              hipStream_t s);

// gy = gy * [0 < out] in place.
template <typename T>
hipError_t generic_relu_mask(const Geom &g, View<const T> out, View<T> gy, hipStream_t s);

// gk and/or gb may be null (that gradient is then skipped).
template <typename T>
hipError_t generic_backward_kb(const Geom &g, bool relu, View<const T> out, View<const T> gy, View<const T> x, T *gk,
                               T *gb, T *ws, hipStream_t s);

// Final 1x1 layer over the channel stack (msd_final.hip); voxels are contiguous, batch and
// channel strides in elements.  The backward overwrites gx, gw and gb (each may be null).
int64_t final_workspace_elems(int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox);
template <typename T>
hipError_t final_forward(int64_t batch, int c_in, int c_out, int64_t nvox, const T *x, int64_t xsb, int64_t xsc,
                         const T *w, const T *bias, T *out, int64_t osb, int64_t osc, hipStream_t s);
template <typename T>
hipError_t final_backward(int64_t batch, int c_in, int c_out, int64_t nvox, const T *x, int64_t xsb, int64_t xsc,
                          const T *go, int64_t gsb, int64_t gsc, const T *w, T *gx, int64_t gxsb, int64_t gxsc,
                          T *gw, T *gb, T *ws, hipStream_t s);

// Final layer + loss + the loss's gradient in one pass (kind 0: mean squared error, 1: mean
// absolute error, 2: log-softmax over the output channels + negative log-likelihood of int64
// labels); c_out <= 8.  Writes out, gout = d loss / d (layer output), the scalar loss and (unless
// both null) gw, gb.  ws as for final_backward.
template <typename T>
hipError_t final_forward_loss(int kind, int64_t batch, int c_in, int c_out, int64_t nvox, const T *x, int64_t xsb,
                              int64_t xsc, const T *w, const T *bias, const void *target, int64_t tsb, int64_t tsc,
                              T *out, int64_t osb, int64_t osc, T *gout, int64_t gsb, int64_t gsc, T *gw, T *gb,
                              T *loss, T *ws, hipStream_t s);

// Launch-shape knobs (msd_set_tuning in the C ABI).  A value < 0 means "library default".
enum Knob {
    kKnobBwdxVec2d, kKnobBwdxVec3d, kKnobBwdxUnroll2d, kKnobBwdxUnroll3d, kKnobBwdxMinBlocks,
    kKnobXcdRemap, kKnobBwdkVec2d, kKnobBwdkVec3d, kKnobBwdkBlocks,
    kKnobFwdVec2d, kKnobFwdVec3d, kKnobFwdSplit, kKnobFwdRows2d, kKnobBwdkRows, kKnobBlockFuse,
    kKnobBlockDefer, kKnobBwdkInterleave, kKnobBlockSnake, kKnobFwdClass3d, kKnobFwdLattice3d,
    kKnobBlockPair, kKnobBlockTriple, kKnobFinalTiled, kKnobBlockSplit3d, kKnobBlockChainPair, kKnobBwdkFused3d, kKnobBwdxLean1,
    kKnobCount
};
int knob(Knob k, int dflt);
extern const char *const kKnobNames[kKnobCount];
extern int g_knobs[kKnobCount];

// Specialised fp32 kernels (unit x-stride, one or two output channels).
// Optional epilogue of the specialised backward_x: grad_input channels >= from are
// multiplied by [0 < act] after the update (act is viewed like grad_input).  The
// dense block uses it to apply the ReLU mask of the layer below while its gradient
// is written for the last time.  from >= C disables it.
struct PostMask {
    int from;
    View<const float> act;
};

bool fast_backward_x_supported_2d(const Geom &g, bool relu, const View<const float> &out,
                                  const View<const float> &gy, const View<float> &gx);
bool fast_backward_x_supported_3d(const Geom &g, bool relu, const View<const float> &out,
                                  const View<const float> &gy, const View<float> &gx);
hipError_t fast_backward_x_2d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                              const float *k, const View<float> &gx, const PostMask &pm, hipStream_t s);
hipError_t fast_backward_x_3d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                              const float *k, const View<float> &gx, const PostMask &pm, hipStream_t s);

inline bool fast_backward_x_supported(const Geom &g, bool relu, const View<const float> &out,
                                      const View<const float> &gy, const View<float> &gx)
{
    return g.ndim == 3 ? fast_backward_x_supported_3d(g, relu, out, gy, gx)
                       : fast_backward_x_supported_2d(g, relu, out, gy, gx);
}
inline hipError_t fast_backward_x(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                                  const float *k, const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    return g.ndim == 3 ? fast_backward_x_3d(g, relu, out, gy, k, gx, pm, s)
                       : fast_backward_x_2d(g, relu, out, gy, k, gx, pm, s);
}

bool fast_forward_supported_2d(const Geom &g, const View<const float> &x, const View<float> &out);
bool fast_forward_supported_3d(const Geom &g, const View<const float> &x, const View<float> &out);
hipError_t fast_forward_2d(const Geom &g, bool relu, const View<const float> &x, const float *k, const float *bias,
                           const View<float> &out, hipStream_t s);
hipError_t fast_forward_3d(const Geom &g, bool relu, const View<const float> &x, const float *k, const float *bias,
                           const View<float> &out, hipStream_t s);

inline bool fast_forward_supported(const Geom &g, const View<const float> &x, const View<float> &out)
{
    return g.ndim == 3 ? fast_forward_supported_3d(g, x, out) : fast_forward_supported_2d(g, x, out);
}
inline hipError_t fast_forward(const Geom &g, bool relu, const View<const float> &x, const float *k,
                               const float *bias, const View<float> &out, hipStream_t s)
{
    return g.ndim == 3 ? fast_forward_3d(g, relu, x, k, bias, out, s) : fast_forward_2d(g, relu, x, k, bias, out, s);
}

// Weight (+ bias) gradient on the matrix cores; gk must not be null, gb may be.
// ws holds kMaxPartialRows rows of (Wd * C * K + Wd) floats.
bool fast_backward_kb_supported_2d(const Geom &g, bool relu, const View<const float> &out,
                                   const View<const float> &gy, const View<const float> &x);
bool fast_backward_kb_supported_3d(const Geom &g, bool relu, const View<const float> &out,
                                   const View<const float> &gy, const View<const float> &x);
hipError_t fast_backward_kb_2d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                               const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s);
hipError_t fast_backward_kb_3d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                               const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s);

inline bool fast_backward_kb_supported(const Geom &g, bool relu, const View<const float> &out,
                                       const View<const float> &gy, const View<const float> &x)
{
    return g.ndim == 3 ? fast_backward_kb_supported_3d(g, relu, out, gy, x)
                       : fast_backward_kb_supported_2d(g, relu, out, gy, x);
}
inline hipError_t fast_backward_kb(const Geom &g, bool relu, const View<const float> &out,
                                   const View<const float> &gy, const View<const float> &x, float *gk, float *gb,
                                   float *ws, hipStream_t s)
{
    return g.ndim == 3 ? fast_backward_kb_3d(g, relu, out, gy, x, gk, gb, ws, s)
                       : fast_backward_kb_2d(g, relu, out, gy, x, gk, gb, ws, s);
}

// A column reduction that has not been launched yet: `rows` partial sums per column, laid
// out part[column][kMaxPartialRows]; columns [0, nk) accumulate into gk, the rest into gb.
struct ReduceJob {
    const float *part;
    float *gk, *gb;
    int64_t nk, ncols;
    int rows;
    float *gk_up[2];  // columns [split, 2 split) and [2 split, nk) go here instead of to gk (the weight
                      // gradients of a second and a third layer)
    int64_t split;    // nk where there is no other destination
    int64_t valid0;   // columns [valid0, split) are dropped (= split: none)
};
// Two or three layers of a dense block as the output channels of one fused backward pass over
// the input channels they share: output channel 0 is the lowest layer (dilation dil[0], the
// call's weights k and weight gradient gk), output channel j the j-th layer above it (dil[j],
// k_up[j - 1], gk_up[j - 1]; the first g.C of its input channels).  The Geom's dilation is the
// largest of them.
constexpr int kMaxLayerGroup = 3;
struct LayerGroup {
    int n;
    int dil[kMaxLayerGroup];
    const float *k_up[kMaxLayerGroup - 1];
    float *gk_up[kMaxLayerGroup - 1];
    int lowest_channels;   // > 0: the lowest layer has only this many of the pass's input channels
    int max_workgroups;    // > 0: workgroups of the launch (a pass that shares the chip with another stream's)
};
constexpr int kReduceBatch = 16;
// One launch for up to kReduceBatch pending reductions; every column is added in the same
// order as by a launch of its own, so the sums are the same bits.
hipError_t reduce_columns_batch(const ReduceJob *jobs, int n, hipStream_t s);

// backward_x and backward_k (+ bias) of one layer in one pass (one output channel, the
// ReLU mask already applied to gy); gk must not be null, gb may be.  Same workspace as
// fast_backward_kb.  With `defer` the partial sums are left in the workspace and the
// reduction that finishes gk / gb is described there instead of being launched.
bool fast_backward_xkb_supported_2d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                    const View<float> &gx);
bool fast_backward_xkb_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                    const View<float> &gx);
hipError_t fast_backward_xkb_2d(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                                const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws,
                                hipStream_t s, ReduceJob *defer, const LayerGroup *group = nullptr);
hipError_t fast_backward_xkb_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                                const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws,
                                hipStream_t s, ReduceJob *defer);
// Weight and bias gradients of two 3D layers of a dense block (one output channel each, own
// dilations) in one pass over x: output channel 0 is the lower layer (gk, group->dil[0]), output
// channel 1 the upper one (group->gk_up[0], group->dil[1]); g.C is the upper layer's channel
// count, group->lowest_channels the lower one's; gy holds the two (masked) output gradients as
// consecutive channels, gb two consecutive bias gradients.  No grad_input is touched.
bool fast_backward_k_pair_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x);
hipError_t fast_backward_k_pair_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk,
                                   float *gb, float *ws, hipStream_t s, ReduceJob *defer, const LayerGroup *group);
// Weight and bias gradients of one 3D layer of one or two output channels from its masked
// output gradient, by the same kernel (no grad_input is touched; gk must not be null, gb may
// be); partial sums behind the first backward_k_mask_floats(g) floats of ws, as for
// fast_backward_kb.
bool fast_backward_k_only_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x);
hipError_t fast_backward_k_only_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk,
                                   float *gb, float *ws, hipStream_t s);
// grad_input of two 3D layers of a dense block (one output channel each, own dilations) in one
// read-modify-write pass over the g.C input channels they share: output channel 0 is the lower
// layer (k, group->dil[0]), output channel 1 the upper one (group->k_up[0], group->dil[1]); gy
// holds the two (masked) output gradients as consecutive channels.  Per channel and voxel the
// lower layer's taps are summed first, then the upper one's, and the sum is added to grad_input.
bool fast_backward_x_pair_supported_3d(const Geom &g, const View<const float> &gy, const View<float> &gx);
hipError_t fast_backward_x_pair_3d(const Geom &g, const View<const float> &gy, const float *k, const View<float> &gx,
                                   const PostMask &pm, hipStream_t s, const LayerGroup *group);
// the instances for rows longer than a workgroup covers (2D) and for stacks whose offsets do
// not fit 32 bits; chosen by fast_backward_xkb_2d / _3d, not called directly
hipError_t fast_backward_xkb_2d_long(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                     const float *k, const View<float> &gx, const PostMask &pm, float *gk, float *gb,
                                     float *ws, hipStream_t s, ReduceJob *defer, const LayerGroup *group = nullptr);
hipError_t fast_backward_xkb_3d_long(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                     const float *k, const View<float> &gx, const PostMask &pm, float *gk, float *gb,
                                     float *ws, hipStream_t s, ReduceJob *defer);

// One layer, or two (g.Wd output channels; `group`: two layers of a dense block), over one input
// channel (2D): grad_input, the channel's nine weight gradients per layer, its ReLU mask
// (pm.from == 0) on the way out.  msd_bwd1.hip.
bool fast_backward_one_channel_supported_2d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                            const View<float> &gx);
hipError_t fast_backward_one_channel_2d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                        const float *k, const View<float> &gx, const PostMask &pm, float *gk,
                                        float *ws, hipStream_t s, ReduceJob *defer,
                                        const LayerGroup *group = nullptr);

inline bool fast_backward_xkb_supported(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                        const View<float> &gx)
{
    return g.ndim == 3 ? fast_backward_xkb_supported_3d(g, gy, x, gx) : fast_backward_xkb_supported_2d(g, gy, x, gx);
}
inline hipError_t fast_backward_xkb(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                    const float *k, const View<float> &gx, const PostMask &pm, float *gk, float *gb,
                                    float *ws, hipStream_t s, ReduceJob *defer = nullptr)
{
    return g.ndim == 3 ? fast_backward_xkb_3d(g, gy, x, k, gx, pm, gk, gb, ws, s, defer)
                       : fast_backward_xkb_2d(g, gy, x, k, gx, pm, gk, gb, ws, s, defer);
}

}  // namespace msd
