// backward_k, 3D instantiations (one file per rank so they compile in parallel).
#include "msd_bwdk_impl.h"

namespace msd {

// One or two output channels go through the weight-gradient-only instances of the fused
// backward kernel (msd_bwdxk_impl.h: row tiles staged in LDS, x requested pairs of voxel groups
// ahead, the next tile's rows during the current tile's channels) where those take the shapes
// ("bwdk.fused3d"; 128^3, 32 input channels: 103 against 151 us for one output channel, 173
// against 294 us for two).  They expect the ReLU mask applied: the masked gradient is written
// to the head of the workspace first, as for bwdk_mfma.
bool fast_backward_kb_supported_3d(const Geom &g, bool relu, const View<const float> &out,
                                    const View<const float> &gy, const View<const float> &x)
{
    return bwdk::supported_nd<3>(g, relu, out, gy, x);
}

hipError_t fast_backward_kb_3d(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                                const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    if (gk && g.Wd <= 2 && knob(kKnobBwdkFused3d, 1) && reinterpret_cast<uintptr_t>(ws) % 16 == 0) {
        // (the layout of the masked copy is known before it is written)
        const View<const float> m =
            relu ? View<const float>{ws, (int64_t)g.Wd * g.nvox, (int64_t)g.nvox, (int64_t)g.H * g.W, (int64_t)g.W, 1} : gy;
        if (fast_backward_k_only_supported_3d(g, m, x)) {
            if (relu) {
                const int64_t total = (int64_t)g.B * g.Wd * g.nvox;
                const int blocks = (int)std::min<int64_t>((total + 255) / 256, 4096);
                hipLaunchKernelGGL(bwdk::mask_gradient, dim3(blocks), dim3(256), 0, s, g, out, gy, ws);
                const hipError_t e = hipGetLastError();
                if (e != hipSuccess) return e;
            }
            return fast_backward_k_only_3d(g, m, x, gk, gb, ws, s);
        }
    }
    return bwdk::run_nd<3>(g, relu, out, gy, x, gk, gb, ws, s);
}

}  // namespace msd
